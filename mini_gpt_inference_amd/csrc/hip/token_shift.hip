// The step between two layers whose sublayers all read one norm of the residual and whose mixer reads that norm
// blended with the previous token's (a token shift), and the activation of such a layer's feed-forward.
//
//   x <- x + mult * y          (y: the float32 sum of the previous layer's sublayers; cleared afterwards)
//   h  = x / sqrt(mean(x^2) + eps) * (offset + gain)
//   hs = h + (h' - h) * shift  (channel by channel; h' the h of the token before in the same sequence, zeros at
//                               position 0)
//
// h' of a request's first token of a step is what the request's row of the state pool holds: the h of its last
// token so far, as float32 of the rounded value that the step's own rows hold, so that a sequence cut anywhere
// computes with the same numbers.  Three kernels, one workgroup a row each:
//   parallel_norm_kernel   the addition, the norm and, in a step whose requests bring one token each, also the
//                          shift and the new state (a row then reads and writes only its own request's state);
//   token_shift_kernel     the shift in a step with prompt portions: a request's first row reads the state, the
//                          others the row before;
//   token_shift_keep_kernel  afterwards, a workgroup a request: the last row's h into the state.
// Sums of squares are float32 in a fixed order (thread-strided, across the wave, across the waves in order).
//
// xielu: for z > 0  a_p z^2 + z / 2;  for z <= 0  a_n (exp(z) - 1 - z) + z / 2, with the two coefficients read from
// a float32 pair (the host applies whatever maps stored parameters to them).
#include "common.h"
#include "dtype_io.h"
#include "launchers.h"

__device__ __forceinline__ float ts_block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  return (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
}

__global__ __launch_bounds__(256) void parallel_norm_kernel(
    float* __restrict__ x, float* __restrict__ y, float mult, const float* __restrict__ gain, float offset, float eps,
    void* __restrict__ h, void* __restrict__ hs, int dtype, const float* __restrict__ shift, float* __restrict__ state,
    long ld_state, const int* __restrict__ state_slots, const int* __restrict__ q_req, const int* __restrict__ positions,
    int width) {
  __shared__ float scratch[4];
  const long row = (long)blockIdx.x * width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    float v = x[row + c];
    if (y) {
      v = fmaf(mult, y[row + c], v);
      x[row + c] = v;
      y[row + c] = 0.f;
    }
    ss = fmaf(v, v, ss);
  }
  if (!h) return;   // the addition only
  const float inv = 1.0f / sqrtf(ts_block_sum(ss, scratch) / (float)width + eps);
  const float* prev = nullptr;
  float* keep = nullptr;
  if (hs) {
    const int r = q_req[blockIdx.x];
    if (r >= 0) {   // not a row of the padding
      keep = state + (long)state_slots[r] * ld_state;
      if (positions[blockIdx.x] > 0) prev = keep;
    }
  }
  for (int c = threadIdx.x; c < width; c += 256) {
    const float v = x[row + c] * inv * (offset + gain[c]);
    store_f(h, dtype, row + c, v);
    if (hs) {
      const float hv = load_f(h, dtype, row + c);   // as the other sublayers read it
      const float pv = prev ? prev[c] : 0.f;
      store_f(hs, dtype, row + c, hv + (pv - hv) * shift[c]);
      if (keep) keep[c] = hv;
    }
  }
}

// x [n_rows, width] float32 in place; y: float32 [n_rows, width] or null; h, hs: rows in `dtype` (hs null: no shift
// in this kernel; h null: only the addition).  With hs every request of the step brings exactly one token.
extern "C" int mgpt_parallel_norm(float* x, float* y, float mult, const float* gain, float offset, float eps, void* h,
                                  void* hs, int dtype, const float* shift, float* state, long ld_state,
                                  const int* state_slots, const int* q_req, const int* positions, int n_rows, int width,
                                  hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!x || (h && !gain) || (hs && (!h || !shift || !state || !state_slots || !q_req || !positions))) return MGPT_ERR_NULL;
  if (n_rows < 0 || width <= 0 || (hs && ld_state < width)) return MGPT_ERR_BAD_SHAPE;
  if (h && !dtype_ok(dtype)) return MGPT_ERR_BAD_DTYPE;
  if (!h && !y) return MGPT_OK;
  hipLaunchKernelGGL(parallel_norm_kernel, dim3(n_rows), dim3(256), 0, stream, x, y, mult, gain, offset, eps, h, hs, dtype,
                     shift, state, ld_state, state_slots, q_req, positions, width);
  return mgpt_last_error();
}

__global__ __launch_bounds__(256) void token_shift_kernel(
    const void* __restrict__ h, void* __restrict__ hs, int dtype, const float* __restrict__ shift,
    const float* __restrict__ state, long ld_state, const int* __restrict__ state_slots, const int* __restrict__ q_req,
    const int* __restrict__ cu_q, const int* __restrict__ positions, int width) {
  const int n = blockIdx.x;
  const long row = (long)n * width;
  const int r = q_req[n];
  const float* kept = nullptr;
  bool before = false;   // the token before is a row of this step
  if (r >= 0) {
    if (n > cu_q[r]) before = true;
    else if (positions[n] > 0) kept = state + (long)state_slots[r] * ld_state;
  }
  for (int c = threadIdx.x; c < width; c += 256) {
    const float hv = load_f(h, dtype, row + c);
    const float pv = before ? load_f(h, dtype, row - width + c) : (kept ? kept[c] : 0.f);
    store_f(hs, dtype, row + c, hv + (pv - hv) * shift[c]);
  }
}

extern "C" int mgpt_token_shift(const void* h, void* hs, int dtype, const float* shift, const float* state,
                                long ld_state, const int* state_slots, const int* q_req, const int* cu_q,
                                const int* positions, int n_rows, int width, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!h || !hs || !shift || !state || !state_slots || !q_req || !cu_q || !positions) return MGPT_ERR_NULL;
  if (n_rows < 0 || width <= 0 || ld_state < width) return MGPT_ERR_BAD_SHAPE;
  if (!dtype_ok(dtype)) return MGPT_ERR_BAD_DTYPE;
  hipLaunchKernelGGL(token_shift_kernel, dim3(n_rows), dim3(256), 0, stream, h, hs, dtype, shift, state, ld_state,
                     state_slots, q_req, cu_q, positions, width);
  return mgpt_last_error();
}

__global__ __launch_bounds__(256) void token_shift_keep_kernel(
    const void* __restrict__ h, int dtype, float* __restrict__ state, long ld_state, const int* __restrict__ state_slots,
    const int* __restrict__ cu_q, int width) {
  const int r = blockIdx.x;
  const int last = cu_q[r + 1] - 1;
  if (last < cu_q[r]) return;   // a request of the padding brings no token
  float* keep = state + (long)state_slots[r] * ld_state;
  for (int c = threadIdx.x; c < width; c += 256) keep[c] = load_f(h, dtype, (long)last * width + c);
}

extern "C" int mgpt_token_shift_keep(const void* h, int dtype, float* state, long ld_state, const int* state_slots,
                                     const int* cu_q, int n_req, int width, hipStream_t stream) {
  if (n_req == 0) return MGPT_OK;
  if (!h || !state || !state_slots || !cu_q) return MGPT_ERR_NULL;
  if (n_req < 0 || width <= 0 || ld_state < width) return MGPT_ERR_BAD_SHAPE;
  if (!dtype_ok(dtype)) return MGPT_ERR_BAD_DTYPE;
  hipLaunchKernelGGL(token_shift_keep_kernel, dim3(n_req), dim3(256), 0, stream, h, dtype, state, ld_state, state_slots,
                     cu_q, width);
  return mgpt_last_error();
}

template <bool FAST>
__global__ __launch_bounds__(256) void xielu_kernel(const void* __restrict__ z, long ldz, void* __restrict__ out, long ldo,
                                                    int dtype, const float* __restrict__ coef, int n_rows, int hidden) {
  const float a_p = coef[0], a_n = coef[1];
  const long total = (long)n_rows * hidden;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    const long row = i / hidden;
    const int c = (int)(i - row * hidden);
    const float v = load_f(z, dtype, row * ldz + c);
    const float r = v > 0.f ? fmaf(a_p * v, v, 0.5f * v)
                            : fmaf(a_n, (FAST ? __expf(v) - 1.0f : expm1f(v)) - v, 0.5f * v);
    store_f(out, dtype, row * ldo + c, r);
  }
}

// z, out: rows in `dtype` (out may be z); coef: float32 [2], the coefficients of the two branches.
extern "C" int mgpt_xielu(const void* z, long ldz, void* out, long ldo, int dtype, const float* coef, int n_rows,
                          int hidden, int fast, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!z || !out || !coef) return MGPT_ERR_NULL;
  if (n_rows < 0 || hidden <= 0 || ldz < hidden || ldo < hidden) return MGPT_ERR_BAD_SHAPE;
  if (!dtype_ok(dtype)) return MGPT_ERR_BAD_DTYPE;
  const long total = (long)n_rows * hidden;
  const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  if (fast)
    hipLaunchKernelGGL(xielu_kernel<true>, dim3(blocks), dim3(256), 0, stream, z, ldz, out, ldo, dtype, coef, n_rows, hidden);
  else
    hipLaunchKernelGGL(xielu_kernel<false>, dim3(blocks), dim3(256), 0, stream, z, ldz, out, ldo, dtype, coef, n_rows, hidden);
  return mgpt_last_error();
}
