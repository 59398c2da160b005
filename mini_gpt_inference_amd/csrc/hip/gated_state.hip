// Linear attention whose decay is made from the token: a mixer whose memory is one float32 matrix
// per request and head, as in decay_state.hip, but with a decay that differs from token to token.
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T      (S: [D, E], zero before a request's first token)
//   o_t = S_t^T q_t (+ skip_h v_t)
//
// Two ways to make a_t, both in float32 from a number that a projection left in the compute dtype:
//   mode 0 (a decay per key channel): a_t[d] = sigmoid(u_t[h][d])^(1/tau) = exp(-softplus(-u) / tau),
//           q is multiplied by q_scale;
//   mode 1 (a decay per head, the discretised state-space form): dt = softplus(u_t[h] + dt_bias[h]),
//           a_t[d] = exp(-exp(a_log[h]) dt) for every d, k is multiplied by dt.
// Heads may share queries and keys in groups (head h reads group h / heads_per_group), values are
// per head.  q, k, v lie in rows of `z`, the decay's source in rows of `a`.
//
// One workgroup per (request, head, block of EB value channels) walks the request's tokens of this
// step in order, whatever their number, from the state the step before left in the request's slot.
// The columns of S are independent, so the value channels of a head are dealt out over workgroups
// until the grid fills the chip.  The state lives in registers: thread (dg, e) owns S[d][e] for
// d = dg, dg + NG, ...; q, k, a, v of eight tokens are staged through LDS at a time, and the partial
// sums over dg meet there once per eight tokens, in the order of dg.
#include "common.h"
#include "dtype_io.h"
#include "launchers.h"

#define GS_MAX 256  // largest D and E
#define GS_TC 8     // tokens staged at once
#define GS_NT 256   // threads a workgroup

__device__ __forceinline__ float gs_softplus(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

template <int R>     // state values a thread
__global__ __launch_bounds__(GS_NT) void gated_state_kernel(
    const void* __restrict__ z, int dtype, long ldz, int q_off, int k_off, int v_off, int n_head, int heads_per_group,
    int D, int E, int EB, const void* __restrict__ a, int a_dtype, long lda, int a_off, int mode, float q_scale,
    float inv_tau, const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ skip,
    float* __restrict__ state, long ld_state, const int* __restrict__ state_slots, const int* __restrict__ cu_q,
    const int* __restrict__ positions, float* __restrict__ out, long ldo) {
  __shared__ float q_s[GS_TC][GS_MAX], k_s[GS_TC][GS_MAX], a_s[GS_TC][GS_MAX], v_s[GS_TC][64], red[GS_TC][GS_NT];
  __shared__ float dt_s[GS_TC];
  const int r = blockIdx.x, h = blockIdx.y, e0 = blockIdx.z * EB, tid = threadIdx.x;
  const int slot = state_slots[r];
  const int t_begin = cu_q[r], t_end = cu_q[r + 1];
  if (slot < 0 || t_end <= t_begin) return;     // a request of the padding
  const int eb = E - e0 < EB ? E - e0 : EB;     // value channels of this workgroup
  const int NG = GS_NT / EB < D ? GS_NT / EB : D;
  const int ec = tid % EB, dg = tid / EB;
  const bool owner = dg < NG && ec < eb;
  const int count = owner ? (D - dg + NG - 1) / NG : 0;
  const int group = h / heads_per_group;
  float S[R];
  float* st = state + (long)slot * ld_state + (long)h * D * E;
  const bool fresh = positions[t_begin] == 0;   // the request's first token: its state starts at zero
#pragma unroll
  for (int j = 0; j < R; ++j) S[j] = (j < count && !fresh) ? st[(long)(dg + j * NG) * E + e0 + ec] : 0.f;
  const float rate = mode == 1 ? expf(a_log[h]) : 0.f;
  const float bias = mode == 1 ? dt_bias[h] : 0.f;
  const float sk = skip ? skip[h] : 0.f;

  for (int t0 = t_begin; t0 < t_end; t0 += GS_TC) {
    const int nt = t_end - t0 < GS_TC ? t_end - t0 : GS_TC;
    __syncthreads();     // the chunk before is read
    if (mode == 1 && tid < nt)
      dt_s[tid] = gs_softplus(load_f(a, a_dtype, (long)(t0 + tid) * lda + a_off + h) + bias);
    __syncthreads();
    for (int i = tid; i < nt * D; i += GS_NT) {
      const int tt = i / D, d = i - tt * D;
      const long row = (long)(t0 + tt) * ldz + (long)group * D + d;
      const float qv = load_f(z, dtype, row + q_off), kv = load_f(z, dtype, row + k_off);
      if (mode == 0) {
        const float u = load_f(a, a_dtype, (long)(t0 + tt) * lda + a_off + (long)h * D + d);
        q_s[tt][d] = qv * q_scale;
        k_s[tt][d] = kv;
        a_s[tt][d] = expf(-gs_softplus(-u) * inv_tau);
      } else {
        const float dt = dt_s[tt];
        q_s[tt][d] = qv;
        k_s[tt][d] = kv * dt;
        a_s[tt][d] = expf(-rate * dt);
      }
    }
    for (int i = tid; i < nt * eb; i += GS_NT) {
      const int tt = i / eb, c = i - tt * eb;
      v_s[tt][c] = load_f(z, dtype, (long)(t0 + tt) * ldz + v_off + (long)h * E + e0 + c);
    }
    __syncthreads();
    if (owner) {
      for (int tt = 0; tt < nt; ++tt) {
        const float ve = v_s[tt][ec];
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
          if (j < count) {
            const int d = dg + j * NG;
            S[j] = fmaf(a_s[tt][d], S[j], k_s[tt][d] * ve);
            acc = fmaf(S[j], q_s[tt][d], acc);
          }
        }
        red[tt][tid] = acc;
      }
    }
    __syncthreads();
    // the sums over dg in order, the skip, the store
    for (int i = tid; i < nt * eb; i += GS_NT) {
      const int tt = i / eb, c = i - tt * eb;
      float o = 0.f;
      for (int g = 0; g < NG; ++g) o += red[tt][g * EB + c];
      if (skip) o = fmaf(sk, v_s[tt][c], o);
      out[(long)(t0 + tt) * ldo + (long)h * E + e0 + c] = o;
    }
  }
#pragma unroll
  for (int j = 0; j < R; ++j)
    if (j < count) st[(long)(dg + j * NG) * E + e0 + ec] = S[j];
}

// z: [n_tokens, ldz] rows in `dtype`; q at q_off and k at k_off, group by group (D channels each), v at v_off head by
// head (E channels each).  a: rows in a_dtype, the decay's source at a_off (mode 0: [heads, D], mode 1: [heads]).
// state: rows of ld_state floats, a request's [heads, D, E] at the row of its slot; state_slots[r] the slot of
// request r (-1: none), cu_q its tokens.  out: float32 rows of all heads' values.
extern "C" int mgpt_gated_state(const void* z, int dtype, long ldz, int q_off, int k_off, int v_off, int n_head,
                                int n_group, int head_dim, int value_dim, const void* a, int a_dtype, long lda, int a_off,
                                int mode, float q_scale, float inv_tau, const float* dt_bias, const float* a_log,
                                const float* skip, float* state, long ld_state, const int* state_slots, const int* cu_q,
                                int n_req, const int* positions, float* out, long ldo, hipStream_t stream) {
  if (n_req == 0) return MGPT_OK;
  if (!z || !a || !positions || !state || !state_slots || !cu_q || !out) return MGPT_ERR_NULL;
  if (mode == 1 && (!dt_bias || !a_log)) return MGPT_ERR_NULL;
  if (!dtype_ok(dtype) || !dtype_ok(a_dtype)) return MGPT_ERR_BAD_DTYPE;
  const int D = head_dim, E = value_dim;
  if (n_req < 0 || n_head <= 0 || n_group <= 0 || n_head % n_group || D <= 0 || E <= 0 || D > GS_MAX || E > GS_MAX ||
      (mode != 0 && mode != 1) || ld_state < (long)n_head * D * E)
    return MGPT_ERR_BAD_SHAPE;
  if (n_head > 65535) return MGPT_ERR_TOO_LARGE;
  // value channels a workgroup: halved while a block would be mostly empty or the grid would not fill the chip
  int EB = 64;
  while (EB > 8 && (EB >= 2 * E || (long)n_req * n_head * ((E + EB - 1) / EB) < 512)) EB >>= 1;
  const int NG = GS_NT / EB < D ? GS_NT / EB : D;
  const int per_thread = (D + NG - 1) / NG;
  dim3 grid(n_req, n_head, (E + EB - 1) / EB);
#define GS_LAUNCH(R)                                                                                                    \
  hipLaunchKernelGGL((gated_state_kernel<R>), grid, dim3(GS_NT), 0, stream, z, dtype, ldz, q_off, k_off, v_off, n_head, \
                     n_head / n_group, D, E, EB, a, a_dtype, lda, a_off, mode, q_scale, inv_tau, dt_bias, a_log, skip,  \
                     state, ld_state, state_slots, cu_q, positions, out, ldo)
  if (per_thread <= 2) GS_LAUNCH(2);
  else if (per_thread <= 4) GS_LAUNCH(4);
  else if (per_thread <= 8) GS_LAUNCH(8);
  else if (per_thread <= 16) GS_LAUNCH(16);
  else if (per_thread <= 32) GS_LAUNCH(32);
  else if (per_thread <= 64) GS_LAUNCH(64);
  else return MGPT_ERR_BAD_SHAPE;
#undef GS_LAUNCH
  return mgpt_last_error();
}
