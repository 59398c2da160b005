// Gated feed-forwards and experts chosen by a table or by a router.
//
// gated unit: act[n][j] = silu(z[n][j]) * z[n][F + j], z = the joint product with the gate and up
// matrices stacked, silu(v) = v * sigmoid(v), in 32-bit.
//
// experts: a token's id picks a row of `top` experts from an integer table.  A (token, choice)
// pair is one unit of work.  The route kernel sorts the pairs by expert into slots; every expert's
// run of slots is padded to a multiple of the tile size (16 or 64 slots), so a tile of slots belongs to one expert
// (tile_expert[tile], -1 for a tile that no expert uses) and slot_token[slot] is the pair's token
// row (-1 for padding), slot_pair[slot] the pair's own index n * top + k.  The grouped product
// then multiplies each tile by its expert's matrix; rows come from, and go to, the places that the
// two index arrays name.  Every output element is one chain over k in order, whatever its slot.
#include "common.h"
#include "dtype_io.h"
#include "launchers.h"

#define EX_TILE 16
#define EX_BK 64
#define EX_MAX_EXPERTS 1024

template <typename T, bool FAST>
__global__ void gated_unit_kernel(const T* __restrict__ z, long ldz, T* __restrict__ act, long lda, long total,
                                  int hidden, int kind) {
  const long i = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long n = i / hidden;
  const int j = (int)(i - n * hidden);
  const float g = to_float<T>(z[n * ldz + j]), u = to_float<T>(z[n * ldz + hidden + j]);
  float s;
  if (kind == 1) s = fmaxf(g, 0.f);                                  // relu
  else if (kind == 2) s = FAST ? gelu_tanh_fast(g) : gelu_tanh(g);
  else s = FAST ? g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) : g / (1.0f + expf(-g));   // silu
  act[n * lda + j] = from_float<T>(s * u);
}

// the same for bfloat16 rows whose hidden size is a multiple of 8: a thread takes 8 units, 16 bytes a load
template <bool FAST>
__global__ void gated_unit_vec8_kernel(const bf16_t* __restrict__ z, long ldz, bf16_t* __restrict__ act, long lda, long total8,
                                       int hidden8, int kind) {
  const long i = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const long n = i / hidden8;
  const int j = (int)(i - n * hidden8) * 8;
  const uint4 gr = *reinterpret_cast<const uint4*>(z + n * ldz + j);
  const uint4 ur = *reinterpret_cast<const uint4*>(z + n * ldz + (long)hidden8 * 8 + j);
  const unsigned int gw[4] = {gr.x, gr.y, gr.z, gr.w}, uw[4] = {ur.x, ur.y, ur.z, ur.w};
  unsigned int out[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float r[2];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const float g = __uint_as_float(half ? (gw[e] & 0xffff0000u) : (gw[e] << 16));
      const float u = __uint_as_float(half ? (uw[e] & 0xffff0000u) : (uw[e] << 16));
      float s;
      if (kind == 1) s = fmaxf(g, 0.f);
      else if (kind == 2) s = FAST ? gelu_tanh_fast(g) : gelu_tanh(g);
      else s = FAST ? g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) : g / (1.0f + expf(-g));
      r[half] = s * u;
    }
    out[e] = pack_bf16x2(r[0], r[1]);
  }
  *reinterpret_cast<uint4*>(act + n * lda + j) = make_uint4(out[0], out[1], out[2], out[3]);
}

extern "C" int mgpt_gated_unit(const void* z, long ldz, void* act, long lda, int n_rows, int hidden, int dtype,
                               int fast, int kind, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!z || !act) return MGPT_ERR_NULL;
  if (n_rows < 0 || hidden <= 0 || ldz < 2L * hidden || lda < hidden || kind < 0 || kind > 2) return MGPT_ERR_BAD_SHAPE;
  if (dtype == MGPT_BF16 && (hidden & 7) == 0 && (ldz & 7) == 0 && (lda & 7) == 0 && (((size_t)z | (size_t)act) & 15) == 0) {
    const long total8 = (long)n_rows * (hidden / 8);
    const long blocks8 = (total8 + 255) / 256;
    if (blocks8 > 0x7fffffffL) return MGPT_ERR_TOO_LARGE;
    if (fast)
      hipLaunchKernelGGL(gated_unit_vec8_kernel<true>, dim3((unsigned)blocks8), dim3(256), 0, stream, (const bf16_t*)z, ldz,
                         (bf16_t*)act, lda, total8, hidden / 8, kind);
    else
      hipLaunchKernelGGL(gated_unit_vec8_kernel<false>, dim3((unsigned)blocks8), dim3(256), 0, stream, (const bf16_t*)z, ldz,
                         (bf16_t*)act, lda, total8, hidden / 8, kind);
    return mgpt_last_error();
  }
  const long total = (long)n_rows * hidden;
  const long blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffL) return MGPT_ERR_TOO_LARGE;
  dim3 grid((unsigned)blocks), block(256);
#define GU_LAUNCH(T, F) \
  hipLaunchKernelGGL((gated_unit_kernel<T, F>), grid, block, 0, stream, (const T*)z, ldz, (T*)act, lda, total, hidden, kind)
  if (dtype == MGPT_F32) {
    if (fast) GU_LAUNCH(float, true); else GU_LAUNCH(float, false);
  } else if (dtype == MGPT_BF16) {
    if (fast) GU_LAUNCH(bf16_t, true); else GU_LAUNCH(bf16_t, false);
  } else {
    return MGPT_ERR_BAD_DTYPE;
  }
#undef GU_LAUNCH
  return mgpt_last_error();
}

// sorted[s] = src[slot_token[s]] for every used slot: the rows of a step in the experts' order, 16 bytes a lane
__global__ void gather_rows_kernel(const uint4* __restrict__ src, long ld16, const int* __restrict__ slot_token,
                                   uint4* __restrict__ sorted, long lds16, int n_slots, int chunks) {
  const long i = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (i >= (long)n_slots * chunks) return;
  const long s = i / chunks;
  const int c = (int)(i - s * chunks);
  const int row = slot_token[s];
  if (row < 0) return;
  sorted[s * lds16 + c] = src[row * ld16 + c];
}

// bfloat16 rows of `width` (a multiple of 8) elements, 16-byte aligned
extern "C" int mgpt_gather_rows(const void* src, long ld, const int* slot_token, void* sorted, long lds, int n_slots,
                                int width, hipStream_t stream) {
  if (n_slots == 0) return MGPT_OK;
  if (!src || !slot_token || !sorted) return MGPT_ERR_NULL;
  if (n_slots < 0 || width <= 0 || (width & 7) || (ld & 7) || (lds & 7) || ld < width || lds < width ||
      (((size_t)src | (size_t)sorted) & 15))
    return MGPT_ERR_BAD_SHAPE;
  const long total = (long)n_slots * (width / 8);
  const long blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffL) return MGPT_ERR_TOO_LARGE;
  hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint4*)src, ld / 8,
                     slot_token, (uint4*)sorted, lds / 8, n_slots, width / 8);
  return mgpt_last_error();
}

// A router: scores of every expert for a token, in float32 whatever the rows' dtype, and the `top`
// largest.  logit[e] = w[e] . h; score = sigmoid(logit) (kind 0) or the logit itself (kind 1);
// chosen[n][c] is the expert with the c-th largest score (of equal scores the lower number first) and
// weight[n][c] its score.  One workgroup a token: its threads along the width in a fixed order, then the first
// wave picks the largest `top` times.
__device__ __forceinline__ float router_value(float v) { return v; }
__device__ __forceinline__ float router_value(bf16_t v) { return bf16_to_float(v); }

__device__ __forceinline__ void router_load8(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void router_load8(const bf16_t* p, float (&v)[8]) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  const unsigned words[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    v[2 * k] = __uint_as_float(words[k] << 16);
    v[2 * k + 1] = __uint_as_float(words[k] & 0xffff0000u);
  }
}

// The storage types are the kernel's parameters (a choice made load by load keeps the loads from being in flight
// together).  VEC: the width is a multiple of 8 and the rows are aligned for loads of eight elements; then thread t
// takes columns 8 t .. 8 t + 7 of every stretch of 2,048 columns for eight experts at a time, whose loads are all in
// flight together, and the sums meet through the waves in a fixed order.  Otherwise a wave takes an expert at a time.
template <typename HT, typename WT, bool VEC>
__global__ __launch_bounds__(256) void router_topk_kernel(const HT* __restrict__ h, long ldh, const WT* __restrict__ w,
                                                          const int* __restrict__ q_req, int width, int n_experts, int top,
                                                          int kind, int* __restrict__ chosen, float* __restrict__ weight) {
  __shared__ float logit[EX_MAX_EXPERTS];
  __shared__ float part[4][8];
  const int n = blockIdx.x;
  if (q_req && q_req[n] < 0) return;     // padded token
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (VEC) {
    for (int e0 = 0; e0 < n_experts; e0 += 8) {
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      for (int c = 8 * threadIdx.x; c < width; c += 8 * 256) {
        float hv[8];
        router_load8(h + (long)n * ldh + c, hv);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int e = e0 + j < n_experts ? e0 + j : n_experts - 1;     // (behind the last expert: loaded again, not used)
          float wv[8];
          router_load8(w + (long)e * width + c, wv);
#pragma unroll
          for (int k = 0; k < 8; ++k) acc[j] = fmaf(wv[k], hv[k], acc[j]);
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float sum = wave_sum(acc[j]);
        if (lane == 0) part[wave][j] = sum;
      }
      __syncthreads();
      if (threadIdx.x < 8 && e0 + threadIdx.x < n_experts)
        logit[e0 + threadIdx.x] = (part[0][threadIdx.x] + part[1][threadIdx.x]) + (part[2][threadIdx.x] + part[3][threadIdx.x]);
      __syncthreads();
    }
  } else {
    for (int e = wave; e < n_experts; e += 4) {
      float acc = 0.f;
      for (int c = lane; c < width; c += 64)
        acc = fmaf(router_value(w[(long)e * width + c]), router_value(h[(long)n * ldh + c]), acc);
      acc = wave_sum(acc);
      if (lane == 0) logit[e] = acc;
    }
    __syncthreads();
  }
  if (wave != 0) return;
  for (int c = 0; c < top; ++c) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < n_experts; e += 64) {
      const float v = logit[e];
      if (v > best) { best = v; at = e; }      // a lane's experts rise, so the lower number stays at a tie
    }
    const float all = wave_max(best);
    int cand = (best == all) ? at : 0x7fffffff;
    // the lowest number among the lanes that hold the maximum
    for (int off = 32; off > 0; off >>= 1) {
      const int other = __shfl_xor(cand, off);
      cand = other < cand ? other : cand;
    }
    if (cand == 0x7fffffff) cand = 0;          // every score is -inf or NaN
    if (lane == 0) {
      chosen[(long)n * top + c] = cand;
      weight[(long)n * top + c] = kind == 0 ? 1.0f / (1.0f + expf(-all)) : all;
    }
    if ((cand & 63) == lane) logit[cand] = -INFINITY;     // the lane that reads this expert takes it out
  }
}

// h: [n_rows, ldh] rows in `dtype`; w: dense [n_experts, width] in w_dtype; chosen: int32 [n_rows, top]; weight:
// float32 [n_rows, top].
extern "C" int mgpt_router_topk(const void* h, int dtype, long ldh, const void* w, int w_dtype, const int* q_req, int n_rows,
                                int width, int n_experts, int top, int kind, int* chosen, float* weight,
                                hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!h || !w || !chosen || !weight) return MGPT_ERR_NULL;
  if (!dtype_ok(dtype) || !dtype_ok(w_dtype)) return MGPT_ERR_BAD_DTYPE;
  if (n_rows < 0 || width <= 0 || n_experts <= 0 || n_experts > EX_MAX_EXPERTS || top <= 0 || top > n_experts ||
      (kind != 0 && kind != 1))
    return MGPT_ERR_BAD_SHAPE;
  const size_t h_size = dtype == MGPT_F32 ? 4 : 2, w_size = w_dtype == MGPT_F32 ? 4 : 2;
  const bool vec = !(width & 7) && !(((size_t)h | (size_t)(ldh * h_size)) & 15) && !((size_t)w & 15);
#define ROUTER_LAUNCH(HT, WT)                                                                                            \
  {                                                                                                                      \
    if (vec)                                                                                                             \
      hipLaunchKernelGGL((router_topk_kernel<HT, WT, true>), dim3(n_rows), dim3(256), 0, stream, (const HT*)h, ldh,      \
                         (const WT*)w, q_req, width, n_experts, top, kind, chosen, weight);                              \
    else                                                                                                                 \
      hipLaunchKernelGGL((router_topk_kernel<HT, WT, false>), dim3(n_rows), dim3(256), 0, stream, (const HT*)h, ldh,     \
                         (const WT*)w, q_req, width, n_experts, top, kind, chosen, weight);                              \
  }
  if (dtype == MGPT_F32 && w_dtype == MGPT_F32) ROUTER_LAUNCH(float, float)
  else if (dtype == MGPT_F32) ROUTER_LAUNCH(float, bf16_t)
  else if (w_dtype == MGPT_F32) ROUTER_LAUNCH(bf16_t, float)
  else ROUTER_LAUNCH(bf16_t, bf16_t)
#undef ROUTER_LAUNCH
  return mgpt_last_error();
}

// sorted[s] = pair_weight[slot_pair[s]] * src[slot_token[s]] for every used slot: the rows of a step in the
// experts' order, each scaled by its pair's weight (in float32, rounded once to the rows' dtype)
__global__ void gather_scale_rows_kernel(const void* __restrict__ src, int dtype, long ld, const int* __restrict__ slot_token,
                                         const int* __restrict__ slot_pair, const float* __restrict__ pair_weight,
                                         void* __restrict__ sorted, long lds, int n_slots, int width) {
  const long i = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (i >= (long)n_slots * width) return;
  const long s = i / width;
  const int c = (int)(i - s * width);
  const int row = slot_token[s];
  if (row < 0) return;
  store_f(sorted, dtype, s * lds + c, pair_weight[slot_pair[s]] * load_f(src, dtype, (long)row * ld + c));
}

// the same for bfloat16 rows of a multiple of 8 elements, 16-byte aligned: eight elements a lane
__global__ void gather_scale_rows_bf16x8_kernel(const uint4* __restrict__ src, long ld16, const int* __restrict__ slot_token,
                                                const int* __restrict__ slot_pair, const float* __restrict__ pair_weight,
                                                uint4* __restrict__ sorted, long lds16, int n_slots, int chunks) {
  const long i = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (i >= (long)n_slots * chunks) return;
  const long s = i / chunks;
  const int c = (int)(i - s * chunks);
  const int row = slot_token[s];
  if (row < 0) return;
  const float wgt = pair_weight[slot_pair[s]];
  uint4 v = src[row * ld16 + c];
  unsigned* words = reinterpret_cast<unsigned*>(&v);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float lo = __uint_as_float(words[k] << 16) * wgt, hi = __uint_as_float(words[k] & 0xffff0000u) * wgt;
    words[k] = (unsigned)float_to_bf16(lo) | ((unsigned)float_to_bf16(hi) << 16);
  }
  sorted[s * lds16 + c] = v;
}

extern "C" int mgpt_gather_scale_rows(const void* src, int dtype, long ld, const int* slot_token, const int* slot_pair,
                                      const float* pair_weight, void* sorted, long lds, int n_slots, int width,
                                      hipStream_t stream) {
  if (n_slots == 0) return MGPT_OK;
  if (!src || !slot_token || !slot_pair || !pair_weight || !sorted) return MGPT_ERR_NULL;
  if (!dtype_ok(dtype)) return MGPT_ERR_BAD_DTYPE;
  if (n_slots < 0 || width <= 0 || ld < width || lds < width) return MGPT_ERR_BAD_SHAPE;
  if (dtype == MGPT_BF16 && !(width & 7) && !(ld & 7) && !(lds & 7) && !(((size_t)src | (size_t)sorted) & 15)) {
    const long blocks8 = ((long)n_slots * (width / 8) + 255) / 256;
    if (blocks8 > 0x7fffffffL) return MGPT_ERR_TOO_LARGE;
    hipLaunchKernelGGL(gather_scale_rows_bf16x8_kernel, dim3((unsigned)blocks8), dim3(256), 0, stream, (const uint4*)src,
                       ld / 8, slot_token, slot_pair, pair_weight, (uint4*)sorted, lds / 8, n_slots, width / 8);
    return mgpt_last_error();
  }
  const long total = (long)n_slots * width;
  const long blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffL) return MGPT_ERR_TOO_LARGE;
  hipLaunchKernelGGL(gather_scale_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, src, dtype, ld, slot_token,
                     slot_pair, pair_weight, sorted, lds, n_slots, width);
  return mgpt_last_error();
}

// One workgroup: counts the pairs of every expert, lays the experts' runs of slots out one after
// the other (each padded to whole tiles), and deals the pairs into them.
__global__ __launch_bounds__(1024) void expert_route_kernel(
    const int* __restrict__ ids, const int* __restrict__ q_req, const int* __restrict__ table, int top,
    int n_rows, int n_experts, int* __restrict__ slot_token, int* __restrict__ slot_pair,
    int* __restrict__ pair_slot, int* __restrict__ tile_expert, int n_slots, int n_tiles, int tile_rows) {
  __shared__ int count[EX_MAX_EXPERTS];
  __shared__ int start[EX_MAX_EXPERTS];
  const int tid = threadIdx.x;
  for (int e = tid; e < n_experts; e += blockDim.x) count[e] = 0;
  for (int s = tid; s < n_slots; s += blockDim.x) slot_token[s] = -1;
  for (int t = tid; t < n_tiles; t += blockDim.x) tile_expert[t] = -1;
  __syncthreads();
  const int n_pairs = n_rows * top;
  for (int p = tid; p < n_pairs; p += blockDim.x) {
    const int n = p / top;
    if (q_req && q_req[n] < 0) continue;   // padded token
    const int e = table[(long)(ids ? ids[n] : n) * top + (p - n * top)];
    if (e >= 0 && e < n_experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int at = 0;
    for (int e = 0; e < n_experts; ++e) {
      start[e] = at;
      const int tiles = (count[e] + tile_rows - 1) / tile_rows;
      for (int t = 0; t < tiles; ++t) tile_expert[at / tile_rows + t] = e;
      at += tiles * tile_rows;
      count[e] = 0;
    }
  }
  __syncthreads();
  for (int p = tid; p < n_pairs; p += blockDim.x) {
    const int n = p / top;
    if (q_req && q_req[n] < 0) continue;
    const int e = table[(long)(ids ? ids[n] : n) * top + (p - n * top)];
    if (e < 0 || e >= n_experts) continue;
    const int s = start[e] + atomicAdd(&count[e], 1);
    slot_token[s] = n;
    slot_pair[s] = p;
    if (pair_slot) pair_slot[p] = s;
  }
}

// ids: the table's row of every token (null: the token's own number).  tile_rows: 16, 64 or 256 slots a tile; n_slots = n_tiles * tile_rows must hold n_rows * top pairs with
// every used expert's run padded to whole tiles.  pair_slot (optional, [n_rows * top]): where each pair went.
extern "C" int mgpt_expert_route(const int* ids, const int* q_req, const int* table, int top, int n_rows,
                                 int n_experts, int* slot_token, int* slot_pair, int* pair_slot, int* tile_expert,
                                 int n_slots, int n_tiles, int tile_rows, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!table || !slot_token || !slot_pair || !tile_expert) return MGPT_ERR_NULL;     // ids null: row n of the table is token n's
  if (n_rows < 0 || top <= 0 || n_experts <= 0 || n_experts > EX_MAX_EXPERTS || (tile_rows != 16 && tile_rows != 64 && tile_rows != 256) || n_slots != n_tiles * tile_rows)
    return MGPT_ERR_BAD_SHAPE;
  // every expert that is used wastes less than a tile
  const long pairs = (long)n_rows * top;
  const long worst = pairs + (n_experts < pairs ? n_experts : pairs) * (long)(tile_rows - 1);
  if ((long)n_slots < worst / tile_rows * tile_rows) return MGPT_ERR_BAD_SHAPE;
  const int threads = (long)n_rows * top > 256 ? 1024 : 256;
  hipLaunchKernelGGL(expert_route_kernel, dim3(1), dim3(threads), 0, stream, ids, q_req, table, top, n_rows, n_experts,
                     slot_token, slot_pair, pair_slot, tile_expert, n_slots, n_tiles, tile_rows);
  return mgpt_last_error();
}

template <typename T, typename OT>
__global__ __launch_bounds__(256) void grouped_linear_kernel(
    const T* __restrict__ A, long lda, const int* __restrict__ a_rows, const T* __restrict__ W, long w_stride,
    const int* __restrict__ tile_expert, const int* __restrict__ slot_token, OT* __restrict__ out, long ldo,
    const int* __restrict__ out_rows, int n_out, int k_dim, int blocks_per_tile) {
  __shared__ float As[EX_TILE][EX_BK + 1];
  __shared__ float Ws[EX_TILE][EX_BK + 1];
  const int tile = blockIdx.y;                    // 16 slots; blocks_per_tile of them share an expert
  const int e = tile_expert[tile / blocks_per_tile];
  if (e < 0) return;
  const int tid = threadIdx.x;
  const int r = tid >> 4, c = tid & 15;
  const int sk = (tid & 15) * 4;
  const int col0 = blockIdx.x * EX_TILE;
  const int slot = tile * EX_TILE + r;
  const bool a_ok = slot_token[slot] >= 0, w_ok = col0 + r < n_out;
  const long arow = a_ok ? (a_rows ? a_rows[slot] : slot) : 0;
  const T* ap = A + arow * lda + sk;
  const T* wp = W + (long)e * w_stride + (long)(col0 + r) * k_dim + sk;
  float acc = 0.f;
  for (int k0 = 0; k0 < k_dim; k0 += EX_BK) {
    const int kmax = k_dim - k0 < EX_BK ? k_dim - k0 : EX_BK;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool k_ok = sk + i < kmax;
      As[r][sk + i] = (a_ok && k_ok) ? to_float<T>(ap[k0 + i]) : 0.f;
      Ws[r][sk + i] = (w_ok && k_ok) ? to_float<T>(wp[k0 + i]) : 0.f;
    }
    __syncthreads();
    for (int kk = 0; kk < kmax; ++kk) acc = fmaf(As[r][kk], Ws[c][kk], acc);
    __syncthreads();
  }
  const int col = col0 + c;
  if (!a_ok || col >= n_out) return;
  const long orow = out_rows ? out_rows[slot] : slot;
  out[orow * ldo + col] = from_float<OT>(acc);
}

// out[out_rows[s] or s] = A[a_rows[s] or s] @ W[tile_expert[s / tile_rows]]^T for every slot s with
// slot_token[s] >= 0.  W: [experts][n_out][k_dim], w_stride elements from one expert to the next.
extern "C" int mgpt_grouped_linear(const void* a, long lda, const int* a_rows, const void* w, long w_stride,
                                   const int* tile_expert, const int* slot_token, void* out, int out_dtype,
                                   long ldo, const int* out_rows, int n_tiles, int tile_rows, int n_out, int k_dim,
                                   int dtype, hipStream_t stream) {
  if (n_tiles == 0 || n_out == 0) return MGPT_OK;
  if (!a || !w || !tile_expert || !slot_token || !out) return MGPT_ERR_NULL;
  if (n_tiles < 0 || n_out < 0 || k_dim <= 0 || lda < k_dim || ldo < n_out || (tile_rows != 16 && tile_rows != 64 && tile_rows != 256))
    return MGPT_ERR_BAD_SHAPE;
  const int blocks_per_tile = tile_rows / EX_TILE;
  if ((long)n_tiles * blocks_per_tile > 65535) return MGPT_ERR_TOO_LARGE;
  dim3 grid((n_out + EX_TILE - 1) / EX_TILE, n_tiles * blocks_per_tile), block(256);
#define GL_LAUNCH(T, OT)                                                                                     \
  hipLaunchKernelGGL((grouped_linear_kernel<T, OT>), grid, block, 0, stream, (const T*)a, lda, a_rows,       \
                     (const T*)w, w_stride, tile_expert, slot_token, (OT*)out, ldo, out_rows, n_out, k_dim,         \
                     blocks_per_tile)
  if (dtype == MGPT_F32 && out_dtype == MGPT_F32) GL_LAUNCH(float, float);
  else if (dtype == MGPT_BF16 && out_dtype == MGPT_BF16) GL_LAUNCH(bf16_t, bf16_t);
  else if (dtype == MGPT_BF16 && out_dtype == MGPT_F32) GL_LAUNCH(bf16_t, float);
  else return MGPT_ERR_BAD_DTYPE;
#undef GL_LAUNCH
  return mgpt_last_error();
}

// The grouped product in bfloat16 on the MFMA units, for tiles of 64 or 16 slots.  A workgroup owns a
// tile x 64 (or 256) columns, a wave 16 (or 64) of the columns for all of the tile's slots: per 32 k one
// (or four) slices of the expert's matrix (first operand) and four slices of gathered rows (one for a
// tile of 16 slots: a decode step's few pairs an expert), 16 bytes a lane straight from memory.
typedef __attribute__((__vector_size__(8 * sizeof(short)))) short ex_bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float ex_f32x4_t;

template <typename OT, int NJ, int NT>     // NT: slices of 16 slots a tile
__global__ __launch_bounds__(256) void grouped_linear_mfma_kernel(
    const bf16_t* __restrict__ A, long lda, const int* __restrict__ a_rows, const bf16_t* __restrict__ W,
    long w_stride, const int* __restrict__ tile_expert, const int* __restrict__ slot_token, OT* __restrict__ out,
    long ldo, const int* __restrict__ out_rows, int n_out, int k_dim) {
  // a wave owns NT * 16 slots x NJ * 16 columns: per 32 k it loads NJ slices of the matrix and NT of the
  // rows for NT * NJ MFMAs
  const int tile = blockIdx.y;
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col0 = (blockIdx.x * 4 + wave) * (NJ * 16);
  if (col0 >= n_out) return;
  const int li = lane & 15, lg = lane >> 4;
  const bf16_t* wrow[NJ];
  bool w_ok[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    w_ok[j] = col0 + j * 16 + li < n_out;
    wrow[j] = W + (long)e * w_stride + (long)(w_ok[j] ? col0 + j * 16 + li : 0) * k_dim;
  }
  const bf16_t* arow[NT];
  bool a_ok[NT];
  long orow[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int slot = tile * (16 * NT) + 16 * t + li;
    a_ok[t] = slot_token[slot] >= 0;
    arow[t] = A + (a_ok[t] ? (long)(a_rows ? a_rows[slot] : slot) : 0L) * lda;
    orow[t] = a_ok[t] ? (long)(out_rows ? out_rows[slot] : slot) : 0L;
  }
  const ex_bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  ex_f32x4_t acc[NJ][NT];
#pragma unroll
  for (int j = 0; j < NJ; ++j)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[j][t] = ex_f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < k_dim; k0 += 32) {
    const int k = k0 + lg * 8;
    const bool k_ok = k < k_dim;
    ex_bf16x8_t wf[NJ], af[NT];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      wf[j] = (w_ok[j] && k_ok) ? *reinterpret_cast<const ex_bf16x8_t*>(wrow[j] + k) : zero;
#pragma unroll
    for (int t = 0; t < NT; ++t)
      af[t] = (a_ok[t] && k_ok) ? *reinterpret_cast<const ex_bf16x8_t*>(arow[t] + k) : zero;
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int t = 0; t < NT; ++t)
        acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], af[t], acc[j][t], 0, 0, 0);
  }
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int c = col0 + j * 16 + lg * 4;
    if (c >= n_out) continue;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (!a_ok[t]) continue;
      OT* dst = out + orow[t] * ldo + c;
      if (sizeof(OT) == 4) {
        *reinterpret_cast<float4*>(dst) = make_float4(acc[j][t][0], acc[j][t][1], acc[j][t][2], acc[j][t][3]);
      } else {
        uint2 pk;
        pk.x = pack_bf16x2(acc[j][t][0], acc[j][t][1]);
        pk.y = pack_bf16x2(acc[j][t][2], acc[j][t][3]);
        *reinterpret_cast<uint2*>(dst) = pk;
      }
    }
  }
}

// bfloat16 operands, tiles of 64 or 16 slots, bfloat16 or float32 out.  Refuses (MGPT_ERR_BAD_SHAPE) inner
// sizes that are no multiple of 8, outputs that are no multiple of 4 and unaligned rows or bases;
// the caller then takes mgpt_grouped_linear.
extern "C" int mgpt_grouped_linear_mfma(const void* a, long lda, const int* a_rows, const void* w, long w_stride,
                                        const int* tile_expert, const int* slot_token, void* out, int out_dtype,
                                        long ldo, const int* out_rows, int n_tiles, int tile_rows, int n_out, int k_dim,
                                        hipStream_t stream) {
  if (n_tiles == 0 || n_out == 0) return MGPT_OK;
  if (!a || !w || !tile_expert || !slot_token || !out) return MGPT_ERR_NULL;
  if (n_tiles < 0 || n_out < 0 || k_dim <= 0 || lda < k_dim || ldo < n_out || (tile_rows != 16 && tile_rows != 64))
    return MGPT_ERR_BAD_SHAPE;
  const int out_align = out_dtype == MGPT_F32 ? 15 : 7;
  if ((k_dim & 7) || (n_out & 3) || (lda & 7) || (ldo & 3) || (w_stride & 7) || (((size_t)a | (size_t)w) & 15) ||
      (((size_t)out) & out_align))
    return MGPT_ERR_BAD_SHAPE;
  if (n_tiles > 65535) return MGPT_ERR_TOO_LARGE;
  // wide outputs: a wave takes 64 columns; narrow ones 16, so that a tile still gives several workgroups
  // ... and so do few tiles (a decode step): more workgroups then walk the inner size side by side
  const bool wide = tile_rows == 64 && n_out >= 512 && n_tiles >= 64;
  dim3 grid((n_out + (wide ? 255 : 63)) / (wide ? 256 : 64), n_tiles), block(256);
#define GM_LAUNCH(OT, NJ, NT)                                                                                 \
  hipLaunchKernelGGL((grouped_linear_mfma_kernel<OT, NJ, NT>), grid, block, 0, stream, (const bf16_t*)a, lda, \
                     a_rows, (const bf16_t*)w, w_stride, tile_expert, slot_token, (OT*)out, ldo, out_rows,    \
                     n_out, k_dim)
  if (out_dtype == MGPT_F32) {
    if (tile_rows == 16) GM_LAUNCH(float, 1, 1); else if (wide) GM_LAUNCH(float, 4, 4); else GM_LAUNCH(float, 1, 4);
  } else if (out_dtype == MGPT_BF16) {
    if (tile_rows == 16) GM_LAUNCH(bf16_t, 1, 1); else if (wide) GM_LAUNCH(bf16_t, 4, 4); else GM_LAUNCH(bf16_t, 1, 4);
  } else {
    return MGPT_ERR_BAD_DTYPE;
  }
#undef GM_LAUNCH
  return mgpt_last_error();
}

__global__ void expert_combine_kernel(const float* __restrict__ pair_out, const int* __restrict__ pair_slot,
                                      const int* __restrict__ q_req, float* __restrict__ y, long total, int width,
                                      int top, float weight) {
  const long i = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long n = i / width;
  const int c = (int)(i - n * width);
  if (q_req && q_req[n] < 0) return;   // padded token: its pairs went nowhere
  float acc = 0.f;
  for (int k = 0; k < top; ++k) {
    const long row = pair_slot ? pair_slot[n * top + k] : n * top + k;
    acc += pair_out[row * (long)width + c];
  }
  y[i] += acc * weight;
}

// the same, four columns a thread (widths in steps of 4, 16-byte aligned buffers)
__global__ void expert_combine4_kernel(const float4* __restrict__ pair_out, const int* __restrict__ pair_slot,
                                       const int* __restrict__ q_req, float4* __restrict__ y, long total, int width4,
                                       int top, float weight) {
  const long i = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long n = i / width4;
  const int c = (int)(i - n * width4);
  if (q_req && q_req[n] < 0) return;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int k = 0; k < top; ++k) {
    const long row = pair_slot ? pair_slot[n * top + k] : n * top + k;
    const float4 v = pair_out[row * (long)width4 + c];
    acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
  }
  float4 o = y[i];
  o.x += acc.x * weight; o.y += acc.y * weight; o.z += acc.z * weight; o.w += acc.w * weight;
  y[i] = o;
}

// y[n] += weight * sum_k pair_out[pair_slot[n * top + k]] (pair_slot null: row n * top + k itself)
extern "C" int mgpt_expert_combine(const float* pair_out, const int* pair_slot, const int* q_req, float* y, int n_rows,
                                   int width, int top, float weight, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!pair_out || !y) return MGPT_ERR_NULL;
  if (n_rows < 0 || width <= 0 || top <= 0) return MGPT_ERR_BAD_SHAPE;
  const bool vec = (width & 3) == 0 && ((((size_t)pair_out) | ((size_t)y)) & 15) == 0;
  const long total = (long)n_rows * (vec ? width / 4 : width);
  const long blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffL) return MGPT_ERR_TOO_LARGE;
  if (vec)
    hipLaunchKernelGGL(expert_combine4_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const float4*)pair_out,
                       pair_slot, q_req, (float4*)y, total, width / 4, top, weight);
  else
    hipLaunchKernelGGL(expert_combine_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, pair_out, pair_slot, q_req, y,
                       total, width, top, weight);
  return mgpt_last_error();
}
