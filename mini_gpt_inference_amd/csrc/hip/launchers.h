// Every launcher of the kernel library that takes a stream, declared in one place: the files that
// define them include this header, so that a declaration that has drifted from its definition does
// not compile, and launch_plan.hip builds its table of launchers from it.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {
// attention_decode.hip
int mgpt_paged_attention_split_bf16(const void* q, long ldq, void* out, long ldo, const void* kpool, const
    void* vpool, const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, const int*
    q_req, int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window,
    const float* sinks, float softcap, const void* gate, long ldg, int keep_first, const float* score_bias,
    hipStream_t stream);
// attention_decode.hip
int mgpt_paged_attention_split_fast_bf16(const void* q, long ldq, void* out, long ldo, const void* kpool,
    const void* vpool, const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, const
    int* q_req, int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window,
    const float* sinks, float softcap, const void* gate, long ldg, int keep_first, const float* score_bias,
    hipStream_t stream);
// attention_decode_wide.hip
int mgpt_paged_attention_decode_bf16(const void* q, long ldq, void* out, long ldo, const void* kpool, const
    void* vpool, const int* block_tables, int max_blocks, const int* positions, const int* q_req, const int*
    cu_q, int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, int num_pages, float scale,
    int window, int identity, const float* sinks, float softcap, const void* gate, long ldg, int keep_first, const
    float* score_bias, hipStream_t stream);
// attention_generic.hip
int mgpt_kv_write(const void* qkv, int dtype, long ld, int k_off, int v_off, void* kpool, void* vpool, const
    int* slot_mapping, int n_tokens, int n_kv_head, int head_dim, int page_size, hipStream_t stream);
// attention_generic.hip
int mgpt_paged_attention_generic(const void* q, long ldq, void* out, long ldo, const void* kpool, const void*
    vpool, const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, const int* q_req,
    int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window, int dtype,
    int fast_exp, const float* sinks, float softcap, const void* gate, long ldg, int keep_first, const float*
    score_bias, hipStream_t stream);
// attention_prefill.hip
int mgpt_prefill_attention_bf16(const void* q, long ldq, void* out, long ldo, const void* kpool, const void*
    vpool, const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, int n_req, int
    max_q_len, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window, int
    single_below, const float* sinks, float softcap, const void* gate, long ldg, int keep_first, const float*
    score_bias, hipStream_t stream);
// embed_norm.hip
int mgpt_embed(const int* ids, const int* pos, const void* tok, const void* postab, float* x, int n_tokens,
    int width, int table_dtype, hipStream_t stream);
// embed_norm.hip
int mgpt_layernorm(const float* x, const float* w, const float* b, void* out, const int* rows, int n_rows, int
    width, float eps, int out_dtype, hipStream_t stream);
// fold_norm.hip
int mgpt_fold_layernorm(const void* w, const float* gain, const float* beta, const float* bias, void* w_out,
    float* colsum, float* bias_out, int n_out, int k_dim, hipStream_t stream);
// fold_norm.hip
int mgpt_pack_weight(const void* w, void* packed, int n_out, int k_dim, hipStream_t stream);
// fused_decode.hip
int mgpt_fused_attention_decode(const float* base, const float* partials, int n_parts, long part_stride, const
    void* tok_table, const void* pos_table, const int* ids, const int* token_positions, float* settled, const
    void* normed, const float* gain, const float* beta, float eps, const void* wqkv_packed, const float* bqkv,
    const void* wproj_packed, const float* bproj, float* out_partials, long out_part_stride, void* kpool, void* vpool,
    const int* slot_mapping, const int* block_tables, int max_blocks, const int* positions, const int* q_req,
    int n_rows, int width, int n_head, int head_dim, int page_size, int num_pages, float scale, hipStream_t
    stream);
// fused_decode.hip
int mgpt_fused_mlp_decode(const float* base, const float* partials, int n_parts, long part_stride, const void*
    tok_table, const void* pos_table, const int* ids, const int* token_positions, float* settled, const float*
    gain, const float* beta, float eps, const void* wfc_packed, const float* bfc, const void* wproj_packed,
    const float* bproj, float* out_partials, long out_part_stride, int n_rows, int width, int hidden,
    hipStream_t stream);
// fused_decode.hip
int mgpt_residual_layernorm(const float* base, const float* partials, int n_parts, long part_stride, const
    void* tok_table, const void* pos_table, const int* ids, const int* token_positions, const float* gain,
    const float* beta, float eps, const int* rows, void* out, int out_dtype, int n_rows, int width, float*
    settled, hipStream_t stream);
// fused_decode.hip
int mgpt_residual_settle(const float* base, const float* partials, int n_parts, long part_stride, const void*
    tok_table, const void* pos_table, const int* ids, const int* token_positions, float* settled, int n_rows,
    int width, hipStream_t stream);
// linear_generic.hip
int mgpt_linear_generic(const void* A, int a_dtype, long lda, const void* W, int w_dtype, const float* bias,
    void* out, int out_dtype, long ldo, int n_rows, int n_out, int k_dim, int epilogue, hipStream_t stream);
// linear_mfma.hip
int mgpt_linear_mfma_parts(const void* act, long lda, const void* w, const float* bias, float* partials,
                           long partials_floats, int n_rows, int n_out, int k_dim, hipStream_t stream);
int mgpt_linear_mfma(const void* act, long lda, const void* w, const float* bias, void* out, int out_dtype,
    long ldo, int n_rows, int n_out, int k_dim, int epilogue, float* partials, long partials_floats,
    hipStream_t stream);
// linear_mfma.hip
int mgpt_linear_mfma_xielu(const void* act, long lda, const void* w, const float* bias, void* out, long ldo,
    int n_rows, int n_out, int k_dim, const float* coef, float* partials, long partials_floats, hipStream_t stream);
int mgpt_linear_mfma_shape(int shape, int k_parts, const void* act, long lda, const void* w, const float*
    bias, void* out, int out_dtype, long ldo, int n_rows, int n_out, int k_dim, int epilogue, float* partials,
    long partials_floats, hipStream_t stream);
// linear_mfma.hip
int mgpt_linear_mfma_qkv(const void* act, long lda, const void* w, const float* bias, void* out, long ldo, int
    n_rows, int n_out, int k_dim, void* kpool, void* vpool, const int* slot_mapping, int q_width, int
    kv_width, int head_dim, int n_kv_head, int page_size, int shape, hipStream_t stream);
// linear_skinny.hip
int mgpt_linear_skinny(const void* act, long lda, const float* x, const int* rows, const float* colsum, float
    eps, const void* w, const void* w_packed, const float* bias, void* out, int out_dtype, long ldo, int
    n_rows, int n_out, int k_dim, int epilogue, void* kpool, void* vpool, const int* slot_mapping, int
    q_width, int kv_width, int head_dim, int n_kv_head, int page_size, int mode, float* partials, long
    partials_floats, hipStream_t stream);
// linear_skinny.hip
int mgpt_linear_head_best(const void* act, long lda, const float* x, const int* rows, const float* colsum,
    float eps, const void* w, const void* w_packed, const float* bias, float* out, long ldo, int n_rows, int
    n_out, int k_dim, float* best_val, int* best_idx, int best_limit, hipStream_t stream);
// linear_decode_rows.hip
int mgpt_linear_decode_parts(const void* act, long lda, const void* w, const void* w_packed, const float* bias,
    float* partials, int n_rows, int n_out, int k_dim, hipStream_t stream);
// sampling.hip
int mgpt_sample(const float* logits, long ld, int n_rows, int vocab, int real_vocab, const float* temperature,
    const int* top_k, const float* top_p, const uint64_t* request_seed, const int* out_index, uint64_t
    engine_seed, int* out_tokens, const float* tile_best, const int* tile_best_idx, int n_tiles, hipStream_t
    stream);
// sampling.hip
int mgpt_sample_advance(const float* logits, long ld, int n_rows, int vocab, int real_vocab, const float*
    temperature, const int* top_k, const float* top_p, const uint64_t* request_seed, int* out_index, uint64_t
    engine_seed, int* out_tokens, int* token_ids, int* positions, int* seq_lens, const int* q_req, int*
    slot_mapping, const int* block_tables, const int* page_sizes, int n_groups, int n_stride, int r_stride,
    int max_blocks, int* history, int* history_pos, int history_rows, int history_stride, const float*
    tile_best, const int* tile_best_idx, int n_tiles, hipStream_t stream);
// streams.hip
int mgpt_embed_scaled(const int* ids, const void* tok, float* x, int n_tokens, int width, int table_dtype, float
    scale, int copies, hipStream_t stream);
int mgpt_streams_read(const float* x, const float* coef, float* u, float* zero, int n_rows, int width, int
    streams, hipStream_t stream);
int mgpt_streams_write(float* x, const float* mix, const float* out, const float* y, int n_rows, int width, int
    streams, hipStream_t stream);
int mgpt_streams_step(float* x, const float* mix, const float* out, float* y, int fold, int clear, const float*
    coef, float* u, const float* gain, const float* beta, float eps, void* h, int h_dtype, int n_rows, int width,
    int streams, hipStream_t stream);
int mgpt_scale_softcap(float* logits, long ld, int n_rows, int vocab, float scale, float cap, int fast,
    hipStream_t stream);
// latent.hip
int mgpt_rms_norm_store(const void* src, int dtype, long ld, const float* gain, float eps, void* pool, const int*
    slot_mapping, int n_tokens, int rank, hipStream_t stream);
int mgpt_latent_prepare(void* z, int dtype, long ldz, int q_off, int n_head, int head_dim, int rot_dim, int c_off,
    int rank, const float* gain, float eps, const int* positions, const float* freq, float rot_mag, void* pool,
    int row_width, const int* slot_mapping, int n_tokens, hipStream_t stream);
int mgpt_heads_linear(const void* a, long lda, const void* w, void* out, long ldo, const void* gate, long ldg,
    int n_rows, int n_head, int n_out, int k_dim, int dtype, int fast, hipStream_t stream);
int mgpt_heads_linear_mfma(const void* a, long lda, const void* w, void* out, long ldo, const void* gate, long ldg,
    int n_rows, int n_head, int n_out, int k_dim, hipStream_t stream);
// token_shift.hip
int mgpt_parallel_norm(float* x, float* y, float mult, const float* gain, float offset, float eps, void* h, void* hs,
    int dtype, const float* shift, float* state, long ld_state, const int* state_slots, const int* q_req,
    const int* positions, int n_rows, int width, hipStream_t stream);
int mgpt_token_shift(const void* h, void* hs, int dtype, const float* shift, const float* state, long ld_state,
    const int* state_slots, const int* q_req, const int* cu_q, const int* positions, int n_rows, int width,
    hipStream_t stream);
int mgpt_token_shift_keep(const void* h, int dtype, float* state, long ld_state, const int* state_slots,
    const int* cu_q, int n_req, int width, hipStream_t stream);
int mgpt_xielu(const void* z, long ldz, void* out, long ldo, int dtype, const float* coef, int n_rows, int hidden,
    int fast, hipStream_t stream);
// experts.hip
int mgpt_gated_unit(const void* z, long ldz, void* act, long lda, int n_rows, int hidden, int dtype, int fast,
    int kind, hipStream_t stream);
int mgpt_expert_route(const int* ids, const int* q_req, const int* table, int top, int n_rows, int n_experts,
    int* slot_token, int* slot_pair, int* pair_slot, int* tile_expert, int n_slots, int n_tiles, int tile_rows,
    hipStream_t stream);
int mgpt_gather_rows(const void* src, long ld, const int* slot_token, void* sorted, long lds, int n_slots, int width,
    hipStream_t stream);
int mgpt_router_topk(const void* h, int dtype, long ldh, const void* w, int w_dtype, const int* q_req, int n_rows,
    int width, int n_experts, int top, int kind, int* chosen, float* weight, hipStream_t stream);
int mgpt_gather_scale_rows(const void* src, int dtype, long ld, const int* slot_token, const int* slot_pair,
    const float* pair_weight, void* sorted, long lds, int n_slots, int width, hipStream_t stream);
int mgpt_grouped_linear(const void* a, long lda, const int* a_rows, const void* w, long w_stride, const int*
    tile_expert, const int* slot_token, void* out, int out_dtype, long ldo, const int* out_rows, int n_tiles,
    int tile_rows, int n_out, int k_dim, int dtype, hipStream_t stream);
int mgpt_grouped_linear_mfma(const void* a, long lda, const int* a_rows, const void* w, long w_stride, const int*
    tile_expert, const int* slot_token, void* out, int out_dtype, long ldo, const int* out_rows, int n_tiles,
    int tile_rows, int n_out, int k_dim, hipStream_t stream);
int mgpt_expert_combine(const float* pair_out, const int* pair_slot, const int* q_req, float* y, int n_rows, int
    width, int top, float weight, hipStream_t stream);
// rms_norm.hip
int mgpt_rms_norm(const void* x, int x_dtype, long ldx, const int* rows, const float* gain, float offset, float eps,
    float mult, const void* gate, int gate_dtype, long ldg, int gate_act, void* out, int out_dtype, long ldo,
    int accumulate, float* zero, long ldz, int zero_width, int n_rows, int groups, int x_gstride, int o_gstride,
    int width, hipStream_t stream);
int mgpt_rms_post_norm(float* y0, float* y1, float* y2, float* y3, const float* g0, const float* g1, const float* g2,
    const float* g3, int n_branches, float coef, int join_unit, float* x, const float* gain_post, const float* scale_post,
    float offset, float eps, float mult, const float* gain_next, void* h, int h_dtype, int n_rows, int width,
    hipStream_t stream);
// gated_state.hip
int mgpt_gated_state(const void* z, int dtype, long ldz, int q_off, int k_off, int v_off, int n_head, int n_group,
    int head_dim, int value_dim, const void* a, int a_dtype, long lda, int a_off, int mode, float q_scale, float inv_tau,
    const float* dt_bias, const float* a_log, const float* skip, float* state, long ld_state, const int* state_slots,
    const int* cu_q, int n_req, const int* positions, float* out, long ldo, hipStream_t stream);
int mgpt_gated_state_chunked(const void* z, int dtype, long ldz, int q_off, int k_off, int v_off, int n_head, int n_group,
                             int head_dim, int value_dim, const void* a, int a_dtype, long lda, int a_off, int mode,
                             float q_scale, float inv_tau, const float* dt_bias, const float* a_log, const float* skip,
                             float* state, long ld_state, const int* state_slots, const int* cu_q, int n_req, int n_tokens,
                             const int* positions, float* qkg, float* out, long ldo, hipStream_t stream);
// short_conv.hip
int mgpt_short_conv(const void* u, int dtype, long ldu, int u_off, const float* w, const float* bias, int act,
    float* state, long ld_state, const int* state_slots, const int* cu_q, const int* q_req, const int* positions,
    int n_req, void* out, int out_dtype, long ldo, int o_off, int n_tokens, int channels, int taps, hipStream_t stream);
// qk_prepare.hip
int mgpt_qk_prepare(void* z, int dtype, long ldz, int q_off, int k_off, int v_off, int n_head, int n_kv_head,
    int head_dim, int value_dim, int head_stride, const int* positions, const float* freq, int rot_dims, float norm_eps,
    const float* mix_lambda, void* v_other, long ld_other, int mix_mode, void* kpool, void* vpool,
    const int* slot_mapping, int page_size, int n_tokens, int norm_mode, const float* q_norm_w, const float* k_norm_w,
    int v_from_k, float rot_mag, hipStream_t stream);
// decay_state.hip
int mgpt_decay_state(const void* z, int dtype, long ldz, int q_off, int k_off, int v_off, int g_off, int n_head,
    int head_dim, int value_dim, int act, const int* positions, const float* freq, int rot_dims, float k_scale,
    const float* decay, float* state, const int* state_slots, const int* cu_q, int n_req, float norm_eps, void* out,
    int out_dtype, long ldo, hipStream_t stream);
int mgpt_decay_state_chunked(const void* z, int dtype, long ldz, int q_off, int k_off, int v_off, int n_head,
    int head_dim, int value_dim, int act, const int* positions, const float* freq, int rot_dims, float k_scale,
    const float* decay, float* state, const int* state_slots, const int* cu_q, int n_req, int n_tokens, float* qk,
    float* out, long ldo, hipStream_t stream);
// linear_mfma.hip
int mgpt_linear_mfma_grouped(const void* act, long lda, const void* w, long w_stride, const int* row_expert, const
    int* row_valid, int group_rows, void* out, int out_dtype, long ldo, int n_rows, int n_out, int k_dim,
    hipStream_t stream);
}

// MGPT_FOR_EACH_LAUNCHER(X) expands X(name) for every launcher above
#define MGPT_FOR_EACH_LAUNCHER(X) \
  X(mgpt_paged_attention_split_bf16) \
  X(mgpt_paged_attention_split_fast_bf16) \
  X(mgpt_paged_attention_decode_bf16) \
  X(mgpt_kv_write) \
  X(mgpt_paged_attention_generic) \
  X(mgpt_prefill_attention_bf16) \
  X(mgpt_embed) \
  X(mgpt_layernorm) \
  X(mgpt_fold_layernorm) \
  X(mgpt_pack_weight) \
  X(mgpt_fused_attention_decode) \
  X(mgpt_fused_mlp_decode) \
  X(mgpt_residual_layernorm) \
  X(mgpt_residual_settle) \
  X(mgpt_linear_generic) \
  X(mgpt_linear_mfma) \
  X(mgpt_linear_mfma_parts) \
  X(mgpt_linear_mfma_shape) \
  X(mgpt_linear_mfma_xielu) \
  X(mgpt_linear_mfma_qkv) \
  X(mgpt_linear_skinny) \
  X(mgpt_linear_head_best) \
  X(mgpt_linear_decode_parts) \
  X(mgpt_sample) \
  X(mgpt_sample_advance) \
  X(mgpt_embed_scaled) \
  X(mgpt_streams_read) \
  X(mgpt_streams_write) \
  X(mgpt_streams_step) \
  X(mgpt_scale_softcap) \
  X(mgpt_rms_norm_store) \
  X(mgpt_latent_prepare) \
  X(mgpt_parallel_norm) \
  X(mgpt_token_shift) \
  X(mgpt_token_shift_keep) \
  X(mgpt_xielu) \
  X(mgpt_heads_linear) \
  X(mgpt_heads_linear_mfma) \
  X(mgpt_grouped_linear_mfma) \
  X(mgpt_gated_unit) \
  X(mgpt_expert_route) \
  X(mgpt_grouped_linear) \
  X(mgpt_expert_combine) \
  X(mgpt_gather_rows) \
  X(mgpt_linear_mfma_grouped) \
  X(mgpt_rms_norm) \
  X(mgpt_rms_post_norm) \
  X(mgpt_qk_prepare) \
  X(mgpt_decay_state) \
  X(mgpt_decay_state_chunked) \
  X(mgpt_router_topk) \
  X(mgpt_gather_scale_rows) \
  X(mgpt_gated_state) \
  X(mgpt_gated_state_chunked) \
  X(mgpt_short_conv)
