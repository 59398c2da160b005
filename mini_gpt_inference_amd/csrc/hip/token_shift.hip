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

// Four neighbouring values of a row in `dtype`: one 16-byte (float32) or 8-byte (bfloat16) access.
template <typename T> __device__ __forceinline__ float4 ts_load4(const T* p);
template <> __device__ __forceinline__ float4 ts_load4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 ts_load4<bf16_t>(const bf16_t* p) {
  const uint2 r = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u), __uint_as_float(r.y << 16),
                     __uint_as_float(r.y & 0xffff0000u));
}
template <typename T> __device__ __forceinline__ void ts_store4(T* p, float4 v);
template <> __device__ __forceinline__ void ts_store4<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <> __device__ __forceinline__ void ts_store4<bf16_t>(bf16_t* p, float4 v) {
  uint2 r;
  r.x = pack_bf16x2(v.x, v.y);
  r.y = pack_bf16x2(v.z, v.w);
  *reinterpret_cast<uint2*>(p) = r;
}
// the values as the stored row holds them
template <typename T> __device__ __forceinline__ float4 ts_rounded(float4 v);
template <> __device__ __forceinline__ float4 ts_rounded<float>(float4 v) { return v; }
template <> __device__ __forceinline__ float4 ts_rounded<bf16_t>(float4 v) {
  return make_float4(bf16_to_float(float_to_bf16(v.x)), bf16_to_float(float_to_bf16(v.y)), bf16_to_float(float_to_bf16(v.z)),
                     bf16_to_float(float_to_bf16(v.w)));
}

// The same as parallel_norm_kernel for rows of up to 1,024 PT values (a multiple of 4) with 16-byte aligned rows:
// a thread keeps its PT groups of four values in registers between the two passes, and everything the second
// pass needs (gain, shift, the kept row) is sent for before the sum of squares is put together.
template <typename T, int PT>
__global__ __launch_bounds__(256) void parallel_norm_row_kernel(
    float* __restrict__ x, float* __restrict__ y, float mult, const float* __restrict__ gain, float offset, float eps,
    T* __restrict__ h, T* __restrict__ hs, const float* __restrict__ shift, float* __restrict__ state, long ld_state,
    const int* __restrict__ state_slots, const int* __restrict__ q_req, const int* __restrict__ positions, int width) {
  __shared__ float scratch[4];
  const long row = (long)blockIdx.x * width;
  const float* prev = nullptr;
  float* keep = nullptr;
  if (hs) {
    const int r = q_req[blockIdx.x];
    if (r >= 0) {   // not a row of the padding
      keep = state + (long)state_slots[r] * ld_state;
      if (positions[blockIdx.x] > 0) prev = keep;
    }
  }
  float4 xv[PT], gv[PT], sv[PT], pv[PT];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const int c = (i * 256 + threadIdx.x) * 4;
    if (c < width) {
      xv[i] = *reinterpret_cast<const float4*>(x + row + c);
      float4 yv = make_float4(0.f, 0.f, 0.f, 0.f);
      if (y) yv = *reinterpret_cast<const float4*>(y + row + c);
      if (h) gv[i] = *reinterpret_cast<const float4*>(gain + c);
      if (hs) {
        sv[i] = *reinterpret_cast<const float4*>(shift + c);
        pv[i] = prev ? *reinterpret_cast<const float4*>(prev + c) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
      if (y) {
        xv[i] = make_float4(fmaf(mult, yv.x, xv[i].x), fmaf(mult, yv.y, xv[i].y), fmaf(mult, yv.z, xv[i].z),
                            fmaf(mult, yv.w, xv[i].w));
        *reinterpret_cast<float4*>(x + row + c) = xv[i];
        *reinterpret_cast<float4*>(y + row + c) = make_float4(0.f, 0.f, 0.f, 0.f);
      }
      ss = fmaf(xv[i].x, xv[i].x, ss);
      ss = fmaf(xv[i].y, xv[i].y, ss);
      ss = fmaf(xv[i].z, xv[i].z, ss);
      ss = fmaf(xv[i].w, xv[i].w, ss);
    }
  }
  if (!h) return;   // the addition only
  const float inv = 1.0f / sqrtf(ts_block_sum(ss, scratch) / (float)width + eps);
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const int c = (i * 256 + threadIdx.x) * 4;
    if (c < width) {
      const float4 v = make_float4(xv[i].x * inv * (offset + gv[i].x), xv[i].y * inv * (offset + gv[i].y),
                                   xv[i].z * inv * (offset + gv[i].z), xv[i].w * inv * (offset + gv[i].w));
      ts_store4<T>(h + row + c, v);
      if (hs) {
        const float4 hv = ts_rounded<T>(v);   // as the other sublayers read it
        ts_store4<T>(hs + row + c, make_float4(hv.x + (pv[i].x - hv.x) * sv[i].x, hv.y + (pv[i].y - hv.y) * sv[i].y,
                                               hv.z + (pv[i].z - hv.z) * sv[i].z, hv.w + (pv[i].w - hv.w) * sv[i].w));
        if (keep) *reinterpret_cast<float4*>(keep + c) = hv;
      }
    }
  }
}

template <typename T>
static void parallel_norm_row_launch(int pt, int n_rows, hipStream_t stream, float* x, float* y, float mult, const float* gain,
                                     float offset, float eps, void* h, void* hs, const float* shift, float* state,
                                     long ld_state, const int* state_slots, const int* q_req, const int* positions, int width) {
#define PN_LAUNCH(PT)                                                                                                 \
  hipLaunchKernelGGL((parallel_norm_row_kernel<T, PT>), dim3(n_rows), dim3(256), 0, stream, x, y, mult, gain, offset, \
                     eps, (T*)h, (T*)hs, shift, state, ld_state, state_slots, q_req, positions, width)
  if (pt <= 1) PN_LAUNCH(1);
  else if (pt == 2) PN_LAUNCH(2);
  else PN_LAUNCH(4);
#undef PN_LAUNCH
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
  const size_t align = (size_t)x | (size_t)y | (size_t)gain | (size_t)h | (size_t)hs | (size_t)shift | (size_t)state;
  if (width % 4 == 0 && width <= 4096 && (align & 15) == 0 && (!hs || ld_state % 4 == 0)) {
    const int pt = (width + 1023) / 1024;
    if (h && dtype == MGPT_BF16)
      parallel_norm_row_launch<bf16_t>(pt, n_rows, stream, x, y, mult, gain, offset, eps, h, hs, shift, state, ld_state,
                                       state_slots, q_req, positions, width);
    else
      parallel_norm_row_launch<float>(pt, n_rows, stream, x, y, mult, gain, offset, eps, h, hs, shift, state, ld_state,
                                      state_slots, q_req, positions, width);
    return mgpt_last_error();
  }
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

// the same, four values a thread (rows of a multiple of four values, 16-byte aligned state rows)
template <typename T>
__global__ __launch_bounds__(256) void token_shift_vec_kernel(
    const T* __restrict__ h, T* __restrict__ hs, const float* __restrict__ shift, const float* __restrict__ state,
    long ld_state, const int* __restrict__ state_slots, const int* __restrict__ q_req, const int* __restrict__ cu_q,
    const int* __restrict__ positions, int width) {
  const int n = blockIdx.x;
  const int c = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (c >= width) return;
  const long row = (long)n * width;
  const int r = q_req[n];
  const float* kept = nullptr;
  bool before = false;
  if (r >= 0) {
    if (n > cu_q[r]) before = true;
    else if (positions[n] > 0) kept = state + (long)state_slots[r] * ld_state;
  }
  const float4 hv = ts_load4<T>(h + row + c), sv = *reinterpret_cast<const float4*>(shift + c);
  float4 pv = make_float4(0.f, 0.f, 0.f, 0.f);
  if (before) pv = ts_load4<T>(h + row - width + c);
  else if (kept) pv = *reinterpret_cast<const float4*>(kept + c);
  ts_store4<T>(hs + row + c, make_float4(hv.x + (pv.x - hv.x) * sv.x, hv.y + (pv.y - hv.y) * sv.y,
                                         hv.z + (pv.z - hv.z) * sv.z, hv.w + (pv.w - hv.w) * sv.w));
}

extern "C" int mgpt_token_shift(const void* h, void* hs, int dtype, const float* shift, const float* state,
                                long ld_state, const int* state_slots, const int* q_req, const int* cu_q,
                                const int* positions, int n_rows, int width, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!h || !hs || !shift || !state || !state_slots || !q_req || !cu_q || !positions) return MGPT_ERR_NULL;
  if (n_rows < 0 || width <= 0 || ld_state < width) return MGPT_ERR_BAD_SHAPE;
  if (!dtype_ok(dtype)) return MGPT_ERR_BAD_DTYPE;
  if (width % 4 == 0 && ld_state % 4 == 0 && (((size_t)h | (size_t)hs | (size_t)shift | (size_t)state) & 15) == 0) {
    const dim3 grid(n_rows, (width + 1023) / 1024);
    if (dtype == MGPT_BF16)
      hipLaunchKernelGGL(token_shift_vec_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)h, (bf16_t*)hs, shift, state,
                         ld_state, state_slots, q_req, cu_q, positions, width);
    else
      hipLaunchKernelGGL(token_shift_vec_kernel<float>, grid, dim3(256), 0, stream, (const float*)h, (float*)hs, shift, state,
                         ld_state, state_slots, q_req, cu_q, positions, width);
    return mgpt_last_error();
  }
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

__device__ __forceinline__ float xielu_fast(float v, float a_p, float a_n) {
  return v > 0.f ? fmaf(a_p * v, v, 0.5f * v) : fmaf(a_n, (__expf(v) - 1.0f) - v, 0.5f * v);
}

// bfloat16 rows whose starts and lengths are multiples of 8 values: 16 bytes a thread
__global__ __launch_bounds__(256) void xielu_vec8_kernel(const bf16_t* __restrict__ z, long ldz, bf16_t* __restrict__ out, long ldo,
                                                         const float* __restrict__ coef, long total8, int hidden8) {
  const float a_p = coef[0], a_n = coef[1];
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total8; i += (long)gridDim.x * 256) {
    const long row = i / hidden8;
    const int c = (int)(i - row * hidden8) * 8;
    const uint4 raw = *reinterpret_cast<const uint4*>(z + row * ldz + c);
    const unsigned int w[4] = {raw.x, raw.y, raw.z, raw.w};
    unsigned int o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      o[e] = pack_bf16x2(xielu_fast(__uint_as_float(w[e] << 16), a_p, a_n), xielu_fast(__uint_as_float(w[e] & 0xffff0000u), a_p, a_n));
    *reinterpret_cast<uint4*>(out + row * ldo + c) = make_uint4(o[0], o[1], o[2], o[3]);
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
  if (fast && dtype == MGPT_BF16 && hidden % 8 == 0 && ldz % 8 == 0 && ldo % 8 == 0 && (((size_t)z | (size_t)out) & 15) == 0) {
    const long total8 = total / 8;
    const int blocks8 = (int)((total8 + 255) / 256 < 8192 ? (total8 + 255) / 256 : 8192);
    hipLaunchKernelGGL(xielu_vec8_kernel, dim3(blocks8), dim3(256), 0, stream, (const bf16_t*)z, ldz, (bf16_t*)out, ldo, coef,
                       total8, hidden / 8);
    return mgpt_last_error();
  }
  const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  if (fast)
    hipLaunchKernelGGL(xielu_kernel<true>, dim3(blocks), dim3(256), 0, stream, z, ldz, out, ldo, dtype, coef, n_rows, hidden);
  else
    hipLaunchKernelGGL(xielu_kernel<false>, dim3(blocks), dim3(256), 0, stream, z, ldz, out, ldo, dtype, coef, n_rows, hidden);
  return mgpt_last_error();
}
