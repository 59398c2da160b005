// A short causal convolution over time, channel by channel, for steps of any shape:
//
//   y_t[c] = act(sum_j w[c][j] u_(t - J + 1 + j)[c] (+ b[c])),   j = 0 .. J-1
//
// with zeros before a request's first token: the last tap multiplies the current token.  u are
// columns of the step's rows (a projection's output); the J - 1 inputs that precede the step's first
// token come from the request's slot of a float32 state pool, [J - 1][C] in the order of time, which a
// second kernel brings up to date with the step's last inputs afterwards.  Which taps reach back
// before position 0 is decided from the token's position, so a slot that another request used needs
// no clearing.  The sum runs over j in order, in float32, whatever the step's shape.
#include "common.h"
#include "dtype_io.h"
#include "launchers.h"

#define SC_MAX_TAPS 9

// A thread a (token, channel): steps of few tokens a request (decode steps), where a run of tokens would be a chain
// of dependent loads of one request's data after the other.
template <typename UT, typename OT>
__global__ __launch_bounds__(256) void short_conv_token_kernel(
    const UT* __restrict__ u, long ldu, int u_off, const float* __restrict__ w, const float* __restrict__ bias,
    int act, const float* __restrict__ state, long ld_state, const int* __restrict__ state_slots,
    const int* __restrict__ cu_q, const int* __restrict__ q_req, const int* __restrict__ positions, OT* __restrict__ out,
    long ldo, int o_off, int C, int J) {
  const int n = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  const int r = q_req[n];
  if (r < 0 || c >= C) return;      // a token of the padding
  const int start = cu_q[r], p = positions[n], slot = state_slots[r];
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < J; ++j) {
    const int back = J - 1 - j;
    if (p - back < 0) continue;     // before the sequence's start
    const int s = n - back;
    float val;
    if (s >= start) val = to_float<UT>(u[(long)s * ldu + u_off + c]);
    else if (slot >= 0) val = state[(long)slot * ld_state + (long)((J - 1) - (start - s)) * C + c];
    else val = 0.f;
    acc = fmaf(w[(long)c * J + j], val, acc);
  }
  if (act == 1) acc = acc / (1.0f + expf(-acc));
  out[(long)n * ldo + o_off + c] = from_float<OT>(acc);
}

#define SC_TB 16     // tokens a workgroup

// A workgroup takes SC_TB consecutive tokens of the step and 256 channels, a thread one channel: it loads its
// channel's inputs of those tokens and of the SC_MAX_TAPS - 1 rows before them once, all loads in flight
// together (the storage types are the kernel's parameters for that), into its own column of an LDS array (which
// only serves as an array that a thread can index at run time: no thread reads another's column), and then goes
// through the tokens.  Where a token's request starts in this step, the token's position and the request's slot
// are the same for the whole workgroup: sixteen threads fetch them first, all at once.
template <typename UT, typename OT>
__global__ __launch_bounds__(256) void short_conv_kernel(
    const UT* __restrict__ u, long ldu, int u_off, const float* __restrict__ w, const float* __restrict__ bias,
    int act, const float* __restrict__ state, long ld_state, const int* __restrict__ state_slots,
    const int* __restrict__ cu_q, const int* __restrict__ q_req, const int* __restrict__ positions, OT* __restrict__ out,
    long ldo, int o_off, int C, int J, int n_tokens) {
  constexpr int LEAD = SC_MAX_TAPS - 1;
  __shared__ float win[SC_TB + LEAD][256];
  __shared__ int meta[3][SC_TB];     // per token: where its request's rows start (-1: padding), its position, its slot
  const int n0 = blockIdx.x * SC_TB, tid = threadIdx.x;
  const int c = blockIdx.y * 256 + tid;
  if (tid < SC_TB) {
    const int n = n0 + tid;
    const int r = n < n_tokens ? q_req[n] : -1;
    meta[0][tid] = r >= 0 ? cu_q[r] : -1;
    meta[1][tid] = r >= 0 ? positions[n] : 0;
    meta[2][tid] = r >= 0 ? state_slots[r] : -1;
  }
  __syncthreads();
  if (c >= C) return;
#pragma unroll
  for (int i = 0; i < SC_TB + LEAD; ++i) {
    const int s = n0 - LEAD + i;
    win[i][tid] = (s >= 0 && s < n_tokens) ? to_float<UT>(u[(long)s * ldu + u_off + c]) : 0.f;
  }
  float wv[SC_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < SC_MAX_TAPS; ++j) wv[j] = j < J ? w[(long)c * J + j] : 0.f;
  const float b = bias ? bias[c] : 0.f;
  for (int i = 0; i < SC_TB && n0 + i < n_tokens; ++i) {
    const int n = n0 + i;
    const int start = meta[0][i], p = meta[1][i], slot = meta[2][i];
    if (start < 0) continue;      // a token of the padding
    float acc = b;
#pragma unroll
    for (int j = 0; j < SC_MAX_TAPS; ++j) {
      const int back = J - 1 - j;
      if (j >= J || p - back < 0) continue;     // no such tap; before the sequence's start
      const int s = n - back;
      float val;
      if (s >= start) val = win[i + LEAD - back][tid];
      else if (slot >= 0) val = state[(long)slot * ld_state + (long)((J - 1) - (start - s)) * C + c];
      else val = 0.f;
      acc = fmaf(wv[j], val, acc);
    }
    if (act == 1) acc = acc / (1.0f + expf(-acc));
    out[(long)n * ldo + o_off + c] = from_float<OT>(acc);
  }
}

// the request's last J - 1 inputs after this step: from the step's rows, or moved up inside the state
__global__ __launch_bounds__(256) void short_conv_state_kernel(
    const void* __restrict__ u, int dtype, long ldu, int u_off, float* __restrict__ state, long ld_state,
    const int* __restrict__ state_slots, const int* __restrict__ cu_q, int C, int J) {
  const int r = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  const int slot = state_slots[r];
  const int start = cu_q[r], end = cu_q[r + 1], len = end - start;
  if (slot < 0 || len <= 0 || c >= C) return;
  float* st = state + (long)slot * ld_state;
  float keep[SC_MAX_TAPS - 1];
#pragma unroll
  for (int i = 0; i < SC_MAX_TAPS - 1; ++i) {
    if (i < J - 1) {
      const int s = end - (J - 1) + i;
      if (s >= start) keep[i] = load_f(u, dtype, (long)s * ldu + u_off + c);
      else keep[i] = st[(long)(i + len) * C + c];      // i + len < J - 1: an input of an earlier step
    }
  }
#pragma unroll
  for (int i = 0; i < SC_MAX_TAPS - 1; ++i)
    if (i < J - 1) st[(long)i * C + c] = keep[i];
}

// u: rows in `dtype`, the C channels at u_off; w: float32 [C][J]; bias: float32 [C] or null; act: 0 none, 1 silu.
// state: rows of ld_state floats, (J - 1) * C of them used (with one tap none: it may be null).  out: rows in out_dtype, the C channels at o_off
// (not the rows of u: a token reads the inputs of the tokens before it).
extern "C" int mgpt_short_conv(const void* u, int dtype, long ldu, int u_off, const float* w, const float* bias, int act,
                               float* state, long ld_state, const int* state_slots, const int* cu_q, const int* q_req,
                               const int* positions, int n_req, void* out, int out_dtype, long ldo, int o_off,
                               int n_tokens, int channels, int taps, hipStream_t stream) {
  if (n_tokens == 0 || n_req == 0) return MGPT_OK;
  if (!u || !w || (!state && taps > 1) || !state_slots || !cu_q || !q_req || !positions || !out) return MGPT_ERR_NULL;
  if (!dtype_ok(dtype) || !dtype_ok(out_dtype)) return MGPT_ERR_BAD_DTYPE;
  if (n_tokens < 0 || n_req < 0 || channels <= 0 || taps < 1 || taps > SC_MAX_TAPS || (act != 0 && act != 1) ||
      ld_state < (long)(taps - 1) * channels || u == out)
    return MGPT_ERR_BAD_SHAPE;
  const int cb = (channels + 255) / 256;
  if (cb > 65535) return MGPT_ERR_TOO_LARGE;
  // steps with runs of tokens (prompt portions): a workgroup a run of SC_TB tokens; few tokens a request: a token
  const bool runs = n_tokens >= 4 * n_req && n_tokens >= 64;
#define SC_LAUNCH(UT, OT)                                                                                                 \
  {                                                                                                                       \
    if (runs)                                                                                                             \
      hipLaunchKernelGGL((short_conv_kernel<UT, OT>), dim3((n_tokens + SC_TB - 1) / SC_TB, cb), dim3(256), 0, stream,     \
                         (const UT*)u, ldu, u_off, w, bias, act, state, ld_state, state_slots, cu_q, q_req, positions,    \
                         (OT*)out, ldo, o_off, channels, taps, n_tokens);                                                 \
    else                                                                                                                  \
      hipLaunchKernelGGL((short_conv_token_kernel<UT, OT>), dim3(n_tokens, cb), dim3(256), 0, stream, (const UT*)u, ldu,  \
                         u_off, w, bias, act, state, ld_state, state_slots, cu_q, q_req, positions, (OT*)out, ldo, o_off, \
                         channels, taps);                                                                                 \
  }
  if (dtype == MGPT_F32 && out_dtype == MGPT_F32) SC_LAUNCH(float, float)
  else if (dtype == MGPT_F32) SC_LAUNCH(float, bf16_t)
  else if (out_dtype == MGPT_F32) SC_LAUNCH(bf16_t, float)
  else SC_LAUNCH(bf16_t, bf16_t)
#undef SC_LAUNCH
  if (taps > 1)
    hipLaunchKernelGGL(short_conv_state_kernel, dim3(n_req, cb), dim3(256), 0, stream, u, dtype, ldu, u_off, state, ld_state,
                       state_slots, cu_q, channels, taps);
  return mgpt_last_error();
}
