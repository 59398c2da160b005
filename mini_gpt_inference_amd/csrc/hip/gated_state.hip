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

// ---------------------------------------------------------------------------------------------
// Prompt portions: the same recurrence a chunk of 32 tokens at a time, as matrix products on the
// float32 matrix cores (v_mfma_f32_16x16x4_f32: true 32-bit products and sums).  With g_t[d] the
// base-2 logarithm of a_t[d] and L_i[d] = g_0[d] + ... + g_i[d] over a chunk's tokens i = 0 .. n-1:
//   P[i][j] = sum_d q_i[d] k_j[d] 2^(L_i[d] - L_j[d]) for j <= i, else 0
//   o_i     = sum_j P[i][j] v_j + S^T (q_i * 2^L_i) (+ skip v_i)
//   S      <- diag(2^L_(n-1)) S + sum_j (k_j * 2^(L_(n-1) - L_j)) v_j^T
// No exponent is ever positive: where i and j lie in different halves of the chunk, the decay between
// them is split at the border m between the halves, (q_i * 2^(L_i - L_m)) . (k_j * 2^(L_m - L_j)), and the
// product runs on the matrix cores; inside a half each pair (i, j) with j < i is summed over d by one
// thread with the exact decay of every channel.  With one decay for a whole head the decay leaves the
// sum over d, and those tiles are matrix products too.
// A workgroup owns (request, head, 32 or 16 value channels); queries, keys and logarithms come ready
// as float32, head by head, from gated_state_inputs_kernel.

#define GC_C 32        // tokens a chunk
#define GC_DMAX 128    // largest head size of this path
#define GC_LDP (GC_C + 4)
#define GC_MILD 96.f   // a half chunk's decay, in powers of two, up to which 2^(L_start - L_j) is safely finite

typedef float gs_f32x4 __attribute__((ext_vector_type(4)));

#define GS_LOG2E 1.4426950408889634f

// qkg: [n_tokens][3][heads * D]: q (scaled), k (times dt in mode 1), log2 of the decay, channel by channel
__global__ __launch_bounds__(256) void gated_state_inputs_kernel(
    const void* __restrict__ z, int dtype, long ldz, int q_off, int k_off, int n_head, int heads_per_group, int D,
    const void* __restrict__ a, int a_dtype, long lda, int a_off, int mode, float q_scale, float inv_tau,
    const float* __restrict__ dt_bias, const float* __restrict__ a_log, float* __restrict__ qkg) {
  const int n = blockIdx.x, HD = n_head * D;
  float* dst = qkg + (long)n * 3 * HD;
  for (int i = threadIdx.x; i < HD; i += 256) {
    const int h = i / D, d = i - h * D;
    if (mode == 0) {
      const float u = load_f(a, a_dtype, (long)n * lda + a_off + i);
      dst[i] = load_f(z, dtype, (long)n * ldz + q_off + i) * q_scale;
      dst[HD + i] = load_f(z, dtype, (long)n * ldz + k_off + i);
      dst[2 * HD + i] = -gs_softplus(-u) * inv_tau * GS_LOG2E;
    } else {
      const long at = (long)n * ldz + (long)(h / heads_per_group) * D + d;
      const float dt = gs_softplus(load_f(a, a_dtype, (long)n * lda + a_off + h) + dt_bias[h]);
      dst[i] = load_f(z, dtype, at + q_off);
      dst[HD + i] = load_f(z, dtype, at + k_off) * dt;
      dst[2 * HD + i] = -expf(a_log[h]) * dt * GS_LOG2E;
    }
  }
}

__device__ __forceinline__ float gs_exp2(float v) { return __builtin_amdgcn_exp2f(v); }

template <int EB, bool SCALAR>     // value channels a workgroup; one decay for all channels of a head
__global__ __launch_bounds__(256) void gated_state_chunk_kernel(
    const float* __restrict__ qkg, const void* __restrict__ z, int dtype, long ldz, int v_off, int n_head, int D, int E,
    const float* __restrict__ skip, const int* __restrict__ positions, float* __restrict__ state, long ld_state,
    const int* __restrict__ state_slots, const int* __restrict__ cu_q, float* __restrict__ out, long ldo) {
  constexpr int NJ = EB / 16;     // column tiles of the workgroup's value channels
  // queries, keys and summed logarithms [token][d]; the state and the values transposed, [value channel][d] and
  // [value channel][token]; P [token][token].  Every product's index of summation runs along a row, so that a
  // lane's operands of four matrix instructions are one 16-byte read.
  extern __shared__ __attribute__((aligned(16))) float gc_lds[];
  const int Dp = (D + 15) & ~15;                // rows of S and steps along d, padded with zeros
  const int ld = Dp + 4;
  float* Qs = gc_lds;                           // [GC_C][ld]
  float* Ks = Qs + GC_C * ld;                   // [GC_C][ld]
  float* Ls = Ks + GC_C * ld;                   // [GC_C][ld]
  float* St = Ls + GC_C * ld;                   // [EB][ld]
  float* Vt = St + EB * ld;                     // [EB][GC_LDP]
  float* Ps = Vt + EB * GC_LDP;                 // [GC_C][GC_LDP]
  const int r = blockIdx.x, h = blockIdx.y, e0 = blockIdx.z * EB, tid = threadIdx.x;
  const int slot = state_slots[r];
  const int t_begin = cu_q[r], t_end = cu_q[r + 1];
  if (slot < 0 || t_end <= t_begin) return;     // a request of the padding
  const int wave = tid >> 6, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
  const int HD = n_head * D;
  const float sk = skip ? skip[h] : 0.f;
  float* st = state + (long)slot * ld_state + (long)h * D * E;
  const bool fresh = positions[t_begin] == 0;
  for (int i = tid; i < Dp * EB; i += 256) {
    const int d = i / EB, c = i - d * EB;
    St[c * ld + d] = (!fresh && d < D && e0 + c < E) ? st[(long)d * E + e0 + c] : 0.f;
  }
  const int ti = wave >> 1, tj = wave & 1;      // this wave's 16 x 16 tile of P
  // the pair (pi, pj), pj < pi, of a half of the chunk that this thread sums over d (240 pairs in both halves)
  int pi = 0, pj = 0;
  const bool has_pair = !SCALAR && tid < 240;
  if (has_pair) {
    const int idx = tid % 120;
    int i = 1;
    while ((i + 1) * i / 2 <= idx) ++i;
    pi = (tid / 120) * 16 + i;
    pj = (tid / 120) * 16 + idx - i * (i - 1) / 2;
  }

  // A chunk's rows travel from memory into registers while the chunk before is multiplied: thread tid holds
  // elements tid, tid + 256, ... of the chunk's [32, Dp] queries, keys and logarithms and of its [32, EB] values.
  constexpr int QK_PT = GC_C * GC_DMAX / 256, V_PT = GC_C * EB / 256;
  float q_r[QK_PT], k_r[QK_PT], g_r[QK_PT], v_r[V_PT];
  auto fetch = [&](int t0) {
    const int nt = t_end - t0 < GC_C ? t_end - t0 : GC_C;      // may be <= 0
#pragma unroll
    for (int u = 0; u < QK_PT; ++u) {
      const int i = tid + u * 256, tt = i / Dp, d = i - tt * Dp;
      const bool ok = i < GC_C * Dp && tt < nt && d < D;
      const long at = (long)(t0 + tt) * 3 * HD + (long)h * D + d;
      q_r[u] = ok ? qkg[at] : 0.f;
      k_r[u] = ok ? qkg[at + HD] : 0.f;
      g_r[u] = ok ? qkg[at + 2 * HD] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < V_PT; ++u) {
      const int i = tid + u * 256, tt = i / EB, c = i - tt * EB;
      v_r[u] = (tt < nt && e0 + c < E) ? load_f(z, dtype, (long)(t0 + tt) * ldz + v_off + (long)h * E + e0 + c) : 0.f;
    }
  };
  fetch(t_begin);

  for (int t0 = t_begin; t0 < t_end; t0 += GC_C) {
    const int nt = t_end - t0 < GC_C ? t_end - t0 : GC_C;
    __syncthreads();     // the chunk before is done with the staged rows; S is whole
#pragma unroll
    for (int u = 0; u < QK_PT; ++u) {
      const int i = tid + u * 256, tt = i / Dp, d = i - tt * Dp;
      if (i < GC_C * Dp) {
        Qs[tt * ld + d] = q_r[u];
        Ks[tt * ld + d] = k_r[u];
        Ls[tt * ld + d] = g_r[u];
      }
    }
#pragma unroll
    for (int u = 0; u < V_PT; ++u) {
      const int i = tid + u * 256;
      Vt[(i % EB) * GC_LDP + i / EB] = v_r[u];
    }
    __syncthreads();
    fetch(t0 + GC_C);     // (behind the last chunk: no token is left, nothing is loaded)
    // ---- L: the logarithms summed over the chunk's tokens, each half by one thread per channel, then the first
    // half's total onto the second.  (Rows behind the chunk's last token hold zeros: L stays what it was there.)
    int mild;
    {
      const int d = tid & 127, half = tid >> 7;
      float run[16] = {};
      if (d < Dp) {
#pragma unroll
        for (int i = 0; i < 16; ++i) run[i] = Ls[(half * 16 + i) * ld + d];
#pragma unroll
        for (int i = 1; i < 16; ++i) run[i] += run[i - 1];
        if (half == 0) {
#pragma unroll
          for (int i = 0; i < 16; ++i) Ls[i * ld + d] = run[i];
        }
      }
      // do all channels keep at least 2^-GC_MILD of their size over each half?  Then the decay inside a half can be
      // split at the half's start as well, without overflow on the key's side
      mild = __syncthreads_and(SCALAR || d >= Dp || run[15] > -GC_MILD);
      if (d < Dp && half == 1) {
        const float first = Ls[15 * ld + d];
#pragma unroll
        for (int i = 0; i < 16; ++i) Ls[(16 + i) * ld + d] = run[i] + first;
      }
    }
    __syncthreads();
    // ---- P
    if (tj <= ti) {
      gs_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
      const float* qrow = Qs + (ti * 16 + r16) * ld;
      const float* krow = Ks + (tj * 16 + r16) * ld;
      if (ti != tj) {
        // the lower left tile: the decay split at the last token of the first half
        const float* lq = Ls + (ti * 16 + r16) * ld;
        const float* lk = Ls + (tj * 16 + r16) * ld;
        const float* lm = Ls + 15 * ld;
#pragma unroll 2
        for (int k0 = 0; k0 < Dp; k0 += 16) {
          const int c = k0 + 4 * g;
          gs_f32x4 a = *reinterpret_cast<const gs_f32x4*>(qrow + c), b = *reinterpret_cast<const gs_f32x4*>(krow + c);
          const gs_f32x4 la = *reinterpret_cast<const gs_f32x4*>(lq + c), lb = *reinterpret_cast<const gs_f32x4*>(lk + c);
          const gs_f32x4 mid = *reinterpret_cast<const gs_f32x4*>(lm + c);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            a[e] *= gs_exp2(la[e] - mid[e]);
            b[e] *= gs_exp2(mid[e] - lb[e]);
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], acc, 0, 0, 0);
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) Ps[(ti * 16 + 4 * g + v) * GC_LDP + tj * 16 + r16] = acc[v];
      } else if (!SCALAR && mild) {
        // a tile on the diagonal whose decays are mild: split at the start of the half (L = 0 before the chunk)
        const float* lq = Ls + (ti * 16 + r16) * ld;
        const float* lm = Ls + 15 * ld;
#pragma unroll 2
        for (int k0 = 0; k0 < Dp; k0 += 16) {
          const int c = k0 + 4 * g;
          gs_f32x4 a = *reinterpret_cast<const gs_f32x4*>(qrow + c), b = *reinterpret_cast<const gs_f32x4*>(krow + c);
          const gs_f32x4 la = *reinterpret_cast<const gs_f32x4*>(lq + c);
          gs_f32x4 mid = {0.f, 0.f, 0.f, 0.f};
          if (ti) mid = *reinterpret_cast<const gs_f32x4*>(lm + c);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float w = gs_exp2(la[e] - mid[e]);     // (a tile on the diagonal: q's row and k's row are the same)
            a[e] *= w;
            b[e] *= __builtin_amdgcn_rcpf(w);
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], acc, 0, 0, 0);
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int i = ti * 16 + 4 * g + v, j = tj * 16 + r16;
          Ps[i * GC_LDP + j] = j <= i ? acc[v] : 0.f;
        }
      } else {
        // a tile on the diagonal: q . k without decay, which is what its diagonal needs; below it, with one decay a
        // head, the decay of the distance multiplies the sum; with a decay per channel the pairs' own threads fill in
#pragma unroll 2
        for (int k0 = 0; k0 < Dp; k0 += 16) {
          const gs_f32x4 a = *reinterpret_cast<const gs_f32x4*>(qrow + k0 + 4 * g);
          const gs_f32x4 b = *reinterpret_cast<const gs_f32x4*>(krow + k0 + 4 * g);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], acc, 0, 0, 0);
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int i = ti * 16 + 4 * g + v, j = tj * 16 + r16;
          if (SCALAR)
            Ps[i * GC_LDP + j] = j <= i ? acc[v] * gs_exp2(Ls[i * ld] - Ls[j * ld]) : 0.f;
          else if (j >= i)
            Ps[i * GC_LDP + j] = j == i ? acc[v] : 0.f;
        }
      }
    } else {
      // the upper right tile is empty
#pragma unroll
      for (int v = 0; v < 4; ++v) Ps[(ti * 16 + 4 * g + v) * GC_LDP + tj * 16 + r16] = 0.f;
    }
    if (has_pair && !mild) {
      const float* qrow = Qs + pi * ld;
      const float* krow = Ks + pj * ld;
      const float* lq = Ls + pi * ld;
      const float* lk = Ls + pj * ld;
      float acc = 0.f;
#pragma unroll 2
      for (int c = 0; c < Dp; c += 4) {
        const gs_f32x4 a = *reinterpret_cast<const gs_f32x4*>(qrow + c), b = *reinterpret_cast<const gs_f32x4*>(krow + c);
        const gs_f32x4 la = *reinterpret_cast<const gs_f32x4*>(lq + c), lb = *reinterpret_cast<const gs_f32x4*>(lk + c);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = fmaf(a[e] * b[e], gs_exp2(la[e] - lb[e]), acc);
      }
      Ps[pi * GC_LDP + pj] = acc;
    }
    __syncthreads();
    // ---- o = P V + (Q * 2^L) S: the tiles (oi, oj) of the chunk's [32, EB] outputs
    for (int t = wave; t < 2 * NJ; t += 4) {
      const int oi = t / NJ, oj = t - oi * NJ;
      gs_f32x4 a1 = {0.f, 0.f, 0.f, 0.f}, a2 = {0.f, 0.f, 0.f, 0.f};
      for (int k0 = 0; k0 < (oi + 1) * 16; k0 += 16) {
        const gs_f32x4 a = *reinterpret_cast<const gs_f32x4*>(Ps + (oi * 16 + r16) * GC_LDP + k0 + 4 * g);
        const gs_f32x4 b = *reinterpret_cast<const gs_f32x4*>(Vt + (oj * 16 + r16) * GC_LDP + k0 + 4 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) a1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], a1, 0, 0, 0);
      }
#pragma unroll 2
      for (int k0 = 0; k0 < Dp; k0 += 16) {
        const int c = k0 + 4 * g;
        gs_f32x4 a = *reinterpret_cast<const gs_f32x4*>(Qs + (oi * 16 + r16) * ld + c);
        const gs_f32x4 la = *reinterpret_cast<const gs_f32x4*>(Ls + (oi * 16 + r16) * ld + c);
        const gs_f32x4 b = *reinterpret_cast<const gs_f32x4*>(St + (oj * 16 + r16) * ld + c);
#pragma unroll
        for (int e = 0; e < 4; ++e) a[e] *= gs_exp2(la[e]);
#pragma unroll
        for (int e = 0; e < 4; ++e) a2 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], a2, 0, 0, 0);
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int i = oi * 16 + 4 * g + v, c = oj * 16 + r16;
        if (i < nt && e0 + c < E) {
          float o = a1[v] + a2[v];
          if (skip) o = fmaf(sk, Vt[c * GC_LDP + i], o);
          out[(long)(t0 + i) * ldo + (long)h * E + e0 + c] = o;
        }
      }
    }
    __syncthreads();     // every wave has read the old S
    // ---- S <- diag(2^L_last) S + sum_t (k_t * 2^(L_last - L_t)) v_t^T: the tiles (di, sj) of the [Dp, EB] state
    const float* last = Ls + (GC_C - 1) * ld;
    for (int t = wave; t < (Dp >> 4) * NJ; t += 4) {
      const int di = t / NJ, sj = t - di * NJ;
      gs_f32x4* mine = reinterpret_cast<gs_f32x4*>(St + (sj * 16 + r16) * ld + di * 16 + 4 * g);     // rows d = 4 g + v of column r16
      gs_f32x4 acc = *mine;
      const gs_f32x4 fall = *reinterpret_cast<const gs_f32x4*>(last + di * 16 + 4 * g);
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[v] *= gs_exp2(fall[v]);
      const float mine_last = last[di * 16 + r16];
#pragma unroll
      for (int k0 = 0; k0 < GC_C; k0 += 16) {
        const gs_f32x4 b = *reinterpret_cast<const gs_f32x4*>(Vt + (sj * 16 + r16) * GC_LDP + k0 + 4 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int tk = k0 + 4 * g + e;
          const float w = gs_exp2(mine_last - Ls[tk * ld + di * 16 + r16]);
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(Ks[tk * ld + di * 16 + r16] * w, b[e], acc, 0, 0, 0);
        }
      }
      *mine = acc;
    }
  }
  __syncthreads();
  for (int i = tid; i < D * EB; i += 256) {
    const int d = i / EB, c = i - d * EB;
    if (e0 + c < E) st[(long)d * E + e0 + c] = St[c * ld + d];
  }
}

// The chunked form for steps with prompt portions: the arguments of mgpt_gated_state, and qkg, float32 scratch
// [n_tokens, 3 * n_head * head_dim].  Head sizes up to 128 (value sizes up to 256); others are refused with
// MGPT_ERR_BAD_SHAPE and nothing launched.
extern "C" int mgpt_gated_state_chunked(const void* z, int dtype, long ldz, int q_off, int k_off, int v_off, int n_head,
                                        int n_group, int head_dim, int value_dim, const void* a, int a_dtype, long lda,
                                        int a_off, int mode, float q_scale, float inv_tau, const float* dt_bias,
                                        const float* a_log, const float* skip, float* state, long ld_state,
                                        const int* state_slots, const int* cu_q, int n_req, int n_tokens,
                                        const int* positions, float* qkg, float* out, long ldo, hipStream_t stream) {
  if (n_req == 0 || n_tokens == 0) return MGPT_OK;
  if (!z || !a || !positions || !state || !state_slots || !cu_q || !out || !qkg) return MGPT_ERR_NULL;
  if (mode == 1 && (!dt_bias || !a_log)) return MGPT_ERR_NULL;
  if (!dtype_ok(dtype) || !dtype_ok(a_dtype)) return MGPT_ERR_BAD_DTYPE;
  const int D = head_dim, E = value_dim;
  if (n_req < 0 || n_tokens < 0 || n_head <= 0 || n_group <= 0 || n_head % n_group || D <= 0 || E <= 0 || D > GC_DMAX ||
      E > GS_MAX || (mode != 0 && mode != 1) || ld_state < (long)n_head * D * E)
    return MGPT_ERR_BAD_SHAPE;
  if (n_head > 65535) return MGPT_ERR_TOO_LARGE;
  hipLaunchKernelGGL(gated_state_inputs_kernel, dim3(n_tokens), dim3(256), 0, stream, z, dtype, ldz, q_off, k_off, n_head,
                     n_head / n_group, D, a, a_dtype, lda, a_off, mode, q_scale, inv_tau, dt_bias, a_log, qkg);
  const int ld = ((D + 15) & ~15) + 4;
#define GC_LAUNCH(EB, SC)                                                                                               \
  {                                                                                                                     \
    const int lds_bytes = (int)sizeof(float) * (3 * GC_C * ld + EB * ld + EB * GC_LDP + GC_C * GC_LDP);                \
    static int allowed = 0; /* more LDS than a kernel gets without asking */                                            \
    if (allowed < lds_bytes) {                                                                                          \
      const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(gated_state_chunk_kernel<EB, SC>),      \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);               \
      if (err != hipSuccess) return (int)err;                                                                           \
      allowed = lds_bytes;                                                                                              \
    }                                                                                                                   \
    hipLaunchKernelGGL((gated_state_chunk_kernel<EB, SC>), dim3(n_req, n_head, (E + EB - 1) / EB), dim3(256), lds_bytes, \
                       stream, qkg, z, dtype, ldz, v_off, n_head, D, E, skip, positions, state, ld_state, state_slots, \
                       cu_q, out, ldo);                                                                                 \
  }
  // 32 value channels a workgroup; 16 where that many workgroups would leave compute units idle
  const bool wide = (long)n_req * n_head * ((E + 31) / 32) >= 256;
  if (mode == 1) {
    if (wide) GC_LAUNCH(32, true) else GC_LAUNCH(16, true)
  } else {
    if (wide) GC_LAUNCH(32, false) else GC_LAUNCH(16, false)
  }
#undef GC_LAUNCH
  return mgpt_last_error();
}
