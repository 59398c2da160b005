// What happens to projected queries, keys and values before attention reads them, in one pass over
// a token (one workgroup a token, its waves dealt out over the heads):
//
//  - rotation by position: channel i of a head's first `rot_dims` channels is paired with channel
//    i + rot_dims/2; the pair (u, w) becomes (u cos a - w sin a, w cos a + u sin a) with
//    a = position * freq[i].  freq is a float32 table made by the host (so base, scaling and any
//    other rule for the frequencies are the caller's); position, angle, sine and cosine are
//    float32, with the full-range sine and cosine.  The other channels pass unchanged.
//    With `rot_mag` every cosine and sine is multiplied by that number;
//  - optionally each query and key head divided by its root mean square over its `head_dim` real
//    channels (eps inside the root), after the rotation (norm_mode 0 with norm_eps >= 0);
//  - or, before the rotation, an RMS norm with weights: head by head with one weight vector [head_dim] for all
//    query heads and one for all key heads (norm_mode 1), or over all of a token's query channels at once (and
//    all of its key channels) with weights [heads * head_dim] (norm_mode 2);
//  - with `v_from_k` the values are the keys as projected (before norm and rotation), and z holds no values;
//  - optionally values mixed with those that another layer made for the same token:
//    v <- (1 - lambda) v + lambda v_other (mode 2), or kept for such layers (mode 1);
//  - queries written back in place; keys and values stored into their page (slot_mapping).
//
// Heads lie `head_stride` channels apart (a head may be padded with zero channels beyond head_dim,
// or value_dim for the values); the values kept for other layers lie value_dim apart.
#include "common.h"
#include "dtype_io.h"
#include "launchers.h"

template <typename T> __device__ __forceinline__ float qk_load(const T* p, long i) { return to_float<T>(p[i]); }
template <typename T> __device__ __forceinline__ void qk_store(T* p, long i, float v) { p[i] = from_float<T>(v); }

#define QKP_MAX_DIM 512
#define QKP_MAX_WAVES 16   // a wave a head at a time: as many waves as the token has query and key heads, up to these

// T: the storage type of z, the pools and v_other (a type known at compile time lets a lane's loads be in flight together)
template <typename T>
__global__ __launch_bounds__(1024) void qk_prepare_kernel(
    T* __restrict__ z, long ldz, int q_off, int k_off, int v_off, int n_head, int n_kv_head,
    int head_dim, int value_dim, int head_stride, const int* __restrict__ positions, const float* __restrict__ freq, int rot_dims,
    float norm_eps, const float* __restrict__ mix_lambda, T* __restrict__ v_other, long ld_other, int mix_mode,
    T* __restrict__ kpool, T* __restrict__ vpool, const int* __restrict__ slot_mapping, int page_size,
    int n_tokens, int norm_mode, const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, int v_from_k,
    float rot_mag, int stash) {
  __shared__ float cos_s[QKP_MAX_DIM / 2], sin_s[QKP_MAX_DIM / 2];
  __shared__ float red_s[2 * QKP_MAX_WAVES];
  extern __shared__ float head_s[];    // [waves][head_dim]: the head a wave is working on; with `stash` behind it
                                       // [n_head + n_kv_head][head_dim]: the token's queries and keys as loaded
  const int n = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, n_waves = blockDim.x >> 6;
  const int half = rot_dims / 2;
  if (freq) {
    const float p = (float)positions[n];
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
      const float a = p * freq[i];
      cos_s[i] = cosf(a) * rot_mag;
      sin_s[i] = sinf(a) * rot_mag;
    }
  }
  const long row = (long)n * ldz;
  float whole_q = 1.0f, whole_k = 1.0f;   // norm_mode 2: what all query (key) channels of the token are multiplied by
  if (norm_mode == 2) {
    float sq = 0.f, sk = 0.f;
    float* all_s = head_s + n_waves * head_dim;   // (used with `stash` only)
    for (int i = threadIdx.x; i < n_head * head_dim; i += blockDim.x) {
      const int hh = i / head_dim;
      const float v = qk_load<T>(z, row + q_off + (long)hh * head_stride + (i - hh * head_dim));
      if (stash) all_s[i] = v;
      sq = fmaf(v, v, sq);
    }
    for (int i = threadIdx.x; i < n_kv_head * head_dim; i += blockDim.x) {
      const int hh = i / head_dim;
      const float v = qk_load<T>(z, row + k_off + (long)hh * head_stride + (i - hh * head_dim));
      if (stash) all_s[n_head * head_dim + i] = v;
      sk = fmaf(v, v, sk);
    }
    sq = wave_sum(sq);
    sk = wave_sum(sk);
    if (lane == 0) {
      red_s[wave] = sq;
      red_s[QKP_MAX_WAVES + wave] = sk;
    }
    __syncthreads();
    sq = sk = 0.f;
    for (int w = 0; w < n_waves; ++w) {      // in wave order, the same sum in every thread
      sq += red_s[w];
      sk += red_s[QKP_MAX_WAVES + w];
    }
    whole_q = 1.0f / sqrtf(sq / (float)(n_head * head_dim) + norm_eps);
    whole_k = 1.0f / sqrtf(sk / (float)(n_kv_head * head_dim) + norm_eps);
  }
  __syncthreads();
  const int slot = slot_mapping ? slot_mapping[n] : -1;
  const long page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot - (int)page * page_size : 0;
  float* s = head_s + wave * head_dim;
  for (int hh = wave; hh < n_head + n_kv_head; hh += n_waves) {
    const bool is_q = hh < n_head;
    const int g = is_q ? hh : hh - n_head;
    if (!is_q && !kpool) continue;
    const long src = row + (is_q ? q_off : k_off) + (long)g * head_stride;
    if (stash)   // the norm's first pass has the token's queries and keys in LDS already
      for (int c = lane; c < head_dim; c += 64) s[c] = head_s[(n_waves + hh) * head_dim + c];
    else
      for (int c = lane; c < head_dim; c += 64) s[c] = qk_load<T>(z, src + c);
    __builtin_amdgcn_wave_barrier();
    const long dst = ((page * n_kv_head + g) * page_size + off) * (long)head_stride;
    if (v_from_k && !is_q && slot >= 0)   // the values are the keys as projected
      for (int c = lane; c < head_stride; c += 64) qk_store<T>(vpool, dst + c, c < head_dim ? s[c] : 0.f);
    if (norm_mode == 1) {
      float ss = 0.f;
      for (int c = lane; c < head_dim; c += 64) ss = fmaf(s[c], s[c], ss);
      const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)head_dim + norm_eps);
      const float* w = is_q ? q_norm_w : k_norm_w;
      for (int c = lane; c < head_dim; c += 64) s[c] = s[c] * inv * w[c];
      __builtin_amdgcn_wave_barrier();
    } else if (norm_mode == 2) {
      const float inv = is_q ? whole_q : whole_k;
      const float* w = (is_q ? q_norm_w : k_norm_w) + (long)g * head_dim;
      for (int c = lane; c < head_dim; c += 64) s[c] = s[c] * inv * w[c];
      __builtin_amdgcn_wave_barrier();
    }
    if (freq) {
      for (int i = lane; i < half; i += 64) {
        const float u = s[i], w = s[i + half], co = cos_s[i], si = sin_s[i];
        s[i] = u * co - w * si;
        s[i + half] = w * co + u * si;
      }
      __builtin_amdgcn_wave_barrier();
    }
    float r = 1.0f;
    if (norm_mode == 0 && norm_eps >= 0.f) {
      float ss = 0.f;
      for (int c = lane; c < head_dim; c += 64) ss = fmaf(s[c], s[c], ss);
      r = 1.0f / sqrtf(wave_sum(ss) / (float)head_dim + norm_eps);
    }
    if (is_q) {
      for (int c = lane; c < head_dim; c += 64) qk_store<T>(z, src + c, s[c] * r);
    } else if (slot >= 0) {
      for (int c = lane; c < head_stride; c += 64) qk_store<T>(kpool, dst + c, c < head_dim ? s[c] * r : 0.f);
      if (v_from_k) {
        __builtin_amdgcn_wave_barrier();
        continue;
      }
      const long vsrc = row + v_off + (long)g * head_stride;
      const long osrc = (long)n * ld_other + (long)g * value_dim;
      const float lam = mix_mode == 2 ? mix_lambda[0] : 0.f;
      for (int c = lane; c < head_stride; c += 64) {
        float v = qk_load<T>(z, vsrc + c);
        if (mix_mode == 1 && c < value_dim) qk_store<T>(v_other, osrc + c, v);
        if (mix_mode == 2 && c < value_dim) v = (1.0f - lam) * v + lam * qk_load<T>(v_other, osrc + c);
        qk_store<T>(vpool, dst + c, v);
      }
    } else if (mix_mode == 1) {
      // a token without a slot (padding of a bucket) still leaves its values: rows are independent
      const long vsrc = row + v_off + (long)g * head_stride;
      const long osrc = (long)n * ld_other + (long)g * value_dim;
      for (int c = lane; c < value_dim; c += 64) qk_store<T>(v_other, osrc + c, qk_load<T>(z, vsrc + c));
    }
    __builtin_amdgcn_wave_barrier();
  }
}

extern "C" int mgpt_qk_prepare(void* z, int dtype, long ldz, int q_off, int k_off, int v_off, int n_head, int n_kv_head,
                               int head_dim, int value_dim, int head_stride, const int* positions, const float* freq, int rot_dims,
                               float norm_eps, const float* mix_lambda, void* v_other, long ld_other, int mix_mode,
                               void* kpool, void* vpool, const int* slot_mapping, int page_size, int n_tokens,
                               int norm_mode, const float* q_norm_w, const float* k_norm_w, int v_from_k, float rot_mag,
                               hipStream_t stream) {
  if (n_tokens == 0) return MGPT_OK;
  if (!z || (freq && !positions) || (kpool && (!vpool || !slot_mapping))) return MGPT_ERR_NULL;
  if (!dtype_ok(dtype)) return MGPT_ERR_BAD_DTYPE;
  if (n_tokens < 0 || n_head <= 0 || n_kv_head <= 0 || head_dim <= 0 || head_dim > QKP_MAX_DIM || head_stride < head_dim || value_dim <= 0 || value_dim > head_stride ||
      rot_dims < 0 || (rot_dims & 1) || rot_dims > head_dim || (kpool && page_size <= 0) || mix_mode < 0 || mix_mode > 2)
    return MGPT_ERR_BAD_SHAPE;
  if (mix_mode && (!v_other || (mix_mode == 2 && !mix_lambda))) return MGPT_ERR_NULL;
  if (norm_mode < 0 || norm_mode > 2 || (norm_mode && !(norm_eps >= 0.f)) || (v_from_k && (mix_mode || value_dim != head_dim)))
    return MGPT_ERR_BAD_SHAPE;
  if (norm_mode && (!q_norm_w || !k_norm_w)) return MGPT_ERR_NULL;
  // few tokens (a decode step): a wave per head, so that a token's heads are done side by side; many tokens: four
  // waves a token, and more tokens at a time on a compute unit
  const int heads = n_head + n_kv_head;
  int waves = heads >= 8 ? 8 : 4;
  if (n_tokens < 64 && heads > 4) waves = heads < QKP_MAX_WAVES ? heads : QKP_MAX_WAVES;
  // a norm over the whole projection reads every query and key before any can be normed: they stay in LDS if they fit
  const int stash = norm_mode == 2 && (size_t)(waves + heads) * head_dim * sizeof(float) <= 48 * 1024;
#define QKP_LAUNCH(T)                                                                                                  \
  hipLaunchKernelGGL(qk_prepare_kernel<T>, dim3(n_tokens), dim3(64 * waves), (waves + (stash ? heads : 0)) * head_dim * sizeof(float), \
                     stream, (T*)z, ldz, q_off, k_off, v_off, n_head, n_kv_head, head_dim, value_dim, head_stride, positions,  \
                     rot_dims ? freq : nullptr, rot_dims, norm_eps, mix_lambda, (T*)v_other, ld_other, mix_mode, (T*)kpool,    \
                     (T*)vpool, slot_mapping, page_size, n_tokens, norm_mode, q_norm_w, k_norm_w, v_from_k, rot_mag, stash)
  if (dtype == MGPT_F32) QKP_LAUNCH(float);
  else QKP_LAUNCH(bf16_t);
#undef QKP_LAUNCH
  return mgpt_last_error();
}
