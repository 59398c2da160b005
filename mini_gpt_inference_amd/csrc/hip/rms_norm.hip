// Root-mean-square norms over float32 statistics.
//
//   unit(x) = x / sqrt(mean(x^2) + eps)
//
// rms_norm: out = [out +] mult * unit(x) * (offset + gain) [* act(gate)] (or, with the gate in front of the norm,
// unit(x * silu(gate)) in place of unit(x) and no gate behind), per segment: a row holds
// `groups` segments of `width` values (one for a norm over the row, one per head for a norm per
// head).  gain may be absent (a norm without a weight), offset is 1 for a gain stored as its
// distance from one.  Rows may be gathered (`rows`), and a second buffer may be cleared on the way
// (the buffer the next sublayer adds its output into).
//
// rms_post_norm: the step between two sublayers of a layer whose sublayers are normed on both
// sides, one workgroup a row:
//   y = sum_b coef * unit(y_b) * gain_b          (only with several branches; else y = y_0;
//                                                 join_unit = 0: sum_b coef * y_b * gain_b, a weighted sum)
//   x += mult * unit(y) * (offset + gain_post) (* scale_post, a scale per channel)
//   h = unit(x) * (offset + gain_next)           (if there is a next norm)
//   y_b = 0                                       (ready for the next sublayer's additions)
// Sums of squares are taken in float32 in a fixed order (lane-strided, then across the wave, then
// across the waves in order), so a row's result does not depend on the other rows of the step.
#include "common.h"
#include "dtype_io.h"
#include "launchers.h"

#define RMS_ACT_NONE 0
#define RMS_ACT_SILU 1
#define RMS_ACT_SIGMOID 2
#define RMS_ACT_SILU_FIRST 3      // the input is multiplied by silu(gate) before its root mean square is taken

__device__ __forceinline__ float rms_gate_act(float g, int act) {
  if (act == RMS_ACT_SILU) return g / (1.0f + expf(-g));
  if (act == RMS_ACT_SIGMOID) return 1.0f / (1.0f + expf(-g));
  return g;
}

// sum over the workgroup's threads (1, 2 or 4 waves), the same value in every thread; waves are added in order
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  if (blockDim.x == 64) return v;
  const int wave = threadIdx.x >> 6;
  __syncthreads();      // the scratch's readers of the call before are done
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  return blockDim.x == 128 ? scratch[0] + scratch[1] : (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
}

// one workgroup per segment: a wave for a narrow one (a head), four for a wide one (a row of the model's width).
// PT > 0: a thread keeps its PT values of the segment in registers between the two passes (segments of up to
// PT * threads values); PT = 0: the second pass reads them again.
template <int PT>
__global__ __launch_bounds__(256) void rms_norm_kernel(
    const void* x, int x_dtype, long ldx, const int* __restrict__ rows,      // (out may be x: the norm in place)
    const float* __restrict__ gain, float offset, float eps, float mult, const void* __restrict__ gate,
    int gate_dtype, long ldg, int gate_act, void* out, int out_dtype, long ldo, int accumulate,
    float* __restrict__ zero, long ldz, int zero_width, int n_rows, int groups, int x_gstride, int o_gstride,
    int width) {
  __shared__ float scratch[4];
  const long seg = blockIdx.x;
  const int row = (int)(seg / groups), g = (int)(seg - (long)row * groups);
  const int src = rows ? rows[row] : row;
  const long xb = (long)src * ldx + (long)g * x_gstride;
  const int step = blockDim.x;
  const long ob = (long)row * ldo + (long)g * o_gstride;
  const long gb = (long)row * ldg + (long)g * o_gstride;
  const bool gate_first = gate && gate_act == RMS_ACT_SILU_FIRST;
  auto input = [&](int c) {
    float v = load_f(x, x_dtype, xb + c);
    if (gate_first) v *= rms_gate_act(load_f(gate, gate_dtype, gb + c), RMS_ACT_SILU);
    return v;
  };
  float xv[PT > 0 ? PT : 1];
  float ss = 0.f;
  if (PT > 0) {
#pragma unroll
    for (int u = 0; u < PT; ++u) {
      const int c = threadIdx.x + u * step;
      xv[u] = c < width ? input(c) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < PT; ++u) ss = fmaf(xv[u], xv[u], ss);
  } else {
    for (int c = threadIdx.x; c < width; c += step) {
      const float v = input(c);
      ss = fmaf(v, v, ss);
    }
  }
  ss = block_sum(ss, scratch);
  const float r = mult / sqrtf(ss / (float)width + eps);
  auto finish = [&](int c, float v) {
    v *= r;
    if (gain) v *= offset + gain[(long)g * width + c];
    if (gate && !gate_first) v *= rms_gate_act(load_f(gate, gate_dtype, gb + c), gate_act);
    if (accumulate) v += load_f(out, out_dtype, ob + c);
    store_f(out, out_dtype, ob + c, v);
  };
  if (PT > 0) {
#pragma unroll
    for (int u = 0; u < PT; ++u) {
      const int c = threadIdx.x + u * step;
      if (c < width) finish(c, xv[u]);
    }
  } else {
    for (int c = threadIdx.x; c < width; c += step) finish(c, input(c));
  }
  if (zero && g == 0)
    for (int c = threadIdx.x; c < zero_width; c += step) zero[(long)row * ldz + c] = 0.f;
}

extern "C" int mgpt_rms_norm(const void* x, int x_dtype, long ldx, const int* rows, const float* gain, float offset,
                             float eps, float mult, const void* gate, int gate_dtype, long ldg, int gate_act,
                             void* out, int out_dtype, long ldo, int accumulate, float* zero, long ldz,
                             int zero_width, int n_rows, int groups, int x_gstride, int o_gstride, int width,
                             hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!x || !out) return MGPT_ERR_NULL;
  if (n_rows < 0 || groups <= 0 || width <= 0 || zero_width < 0) return MGPT_ERR_BAD_SHAPE;
  if (!dtype_ok(x_dtype) || !dtype_ok(out_dtype) || (gate && !dtype_ok(gate_dtype))) return MGPT_ERR_BAD_DTYPE;
  const long segs = (long)n_rows * groups;
  if (segs > 0x7fffffffL) return MGPT_ERR_TOO_LARGE;
  const int threads = width <= 256 ? 64 : (width <= 512 ? 128 : 256);
#define RN_LAUNCH(PT)                                                                                              \
  hipLaunchKernelGGL(rms_norm_kernel<PT>, dim3((unsigned)segs), dim3(threads), 0, stream, x, x_dtype, ldx, rows, gain,  \
                     offset, eps, mult, gate, gate_dtype, ldg, gate_act, out, out_dtype, ldo, accumulate, zero, ldz,   \
                     zero_width, n_rows, groups, x_gstride, o_gstride, width)
  const int per_thread = (width + threads - 1) / threads;
  if (per_thread <= 4) RN_LAUNCH(4);
  else if (per_thread <= 16) RN_LAUNCH(16);
  else RN_LAUNCH(0);
#undef RN_LAUNCH
  return mgpt_last_error();
}

// sum over the workgroup's 256 threads, the same value in every thread; waves are added in order
__device__ __forceinline__ float block_sum_256(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();      // the scratch's readers of the call before are done
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  return (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
}

#define RMS_MAX_BRANCHES 4

struct RmsBranches {
  float* y[RMS_MAX_BRANCHES];
  const float* gain[RMS_MAX_BRANCHES];
};

__global__ __launch_bounds__(256) void rms_post_norm_kernel(RmsBranches br, int n_branches, float coef, int join_unit,
                                                            float* __restrict__ x, const float* __restrict__ gain_post,
                                                            const float* __restrict__ scale_post, float offset, float eps,
                                                            float mult, const float* __restrict__ gain_next,
                                                            void* __restrict__ h, int h_dtype, int n_rows, int width) {
  __shared__ float scratch[4];
  const int row = blockIdx.x;
  if (row >= n_rows) return;
  const long base = (long)row * width;
  float* y0 = br.y[0] + base;
  if (n_branches > 1) {
    // the branches' outputs, each normed with its own plain gain, averaged into the first one's buffer
    float r[RMS_MAX_BRANCHES];
    for (int b = 0; b < n_branches; ++b) {
      const float* yb = br.y[b] + base;
      float ss = 0.f;
      if (join_unit)
        for (int c = threadIdx.x; c < width; c += 256) ss = fmaf(yb[c], yb[c], ss);
      r[b] = join_unit ? coef / sqrtf(block_sum_256(ss, scratch) / (float)width + eps) : coef;
    }
    for (int c = threadIdx.x; c < width; c += 256) {
      float v = 0.f;
      for (int b = 0; b < n_branches; ++b) {
        v = fmaf(br.y[b][base + c] * r[b], br.gain[b][c], v);
        if (b) br.y[b][base + c] = 0.f;
      }
      y0[c] = v;      // read again below by the thread that wrote it
    }
  }
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) ss = fmaf(y0[c], y0[c], ss);
  const float ry = mult / sqrtf(block_sum_256(ss, scratch) / (float)width + eps);
  float sx = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    const float v = x[base + c] + y0[c] * ry * (offset + gain_post[c]) * (scale_post ? scale_post[c] : 1.0f);
    x[base + c] = v;
    y0[c] = 0.f;
    sx = fmaf(v, v, sx);
  }
  if (!gain_next) return;
  const float rx = 1.0f / sqrtf(block_sum_256(sx, scratch) / (float)width + eps);
  for (int c = threadIdx.x; c < width; c += 256)
    store_f(h, h_dtype, base + c, x[base + c] * rx * (offset + gain_next[c]));
}

// The same step for one or two branches and rows of up to 256 * PT values: every value is loaded once (the row,
// the sublayers' outputs and all gains are in registers before the first sum), one trip to memory instead of
// three or five.
template <int PT, int NB>
__global__ __launch_bounds__(256) void rms_post_norm_row_kernel(RmsBranches br, float coef, int join_unit, float* __restrict__ x,
                                                                const float* __restrict__ gain_post,
                                                                const float* __restrict__ scale_post, float offset, float eps,
                                                                float mult, const float* __restrict__ gain_next,
                                                                void* __restrict__ h, int h_dtype, int n_rows, int width) {
  __shared__ float scratch[4];
  const long base = (long)blockIdx.x * width;
  float yv[NB][PT], jg[NB][PT], xv[PT], gp[PT], gn[PT];
#pragma unroll
  for (int u = 0; u < PT; ++u) {
    const int c = threadIdx.x + u * 256;
    const bool ok = c < width;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      yv[b][u] = ok ? br.y[b][base + c] : 0.f;
      jg[b][u] = (ok && NB > 1) ? br.gain[b][c] : 1.f;
    }
    xv[u] = ok ? x[base + c] : 0.f;
    gp[u] = ok ? (offset + gain_post[c]) * (scale_post ? scale_post[c] : 1.0f) : 0.f;
    gn[u] = (ok && gain_next) ? gain_next[c] : 0.f;
  }
  if (NB > 1) {
    // the branches' outputs, each normed with its own plain gain, averaged
    float r[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      float ss = 0.f;
#pragma unroll
      for (int u = 0; u < PT; ++u) ss = fmaf(yv[b][u], yv[b][u], ss);
      r[b] = join_unit ? coef / sqrtf(block_sum_256(ss, scratch) / (float)width + eps) : coef;
    }
#pragma unroll
    for (int u = 0; u < PT; ++u) {
      float v = 0.f;
#pragma unroll
      for (int b = 0; b < NB; ++b) v = fmaf(yv[b][u] * r[b], jg[b][u], v);
      yv[0][u] = v;
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < PT; ++u) ss = fmaf(yv[0][u], yv[0][u], ss);
  const float ry = mult / sqrtf(block_sum_256(ss, scratch) / (float)width + eps);
  float sx = 0.f;
#pragma unroll
  for (int u = 0; u < PT; ++u) {
    const int c = threadIdx.x + u * 256;
    xv[u] = xv[u] + yv[0][u] * ry * gp[u];
    if (c < width) {
      x[base + c] = xv[u];
#pragma unroll
      for (int b = 0; b < NB; ++b) br.y[b][base + c] = 0.f;
      sx = fmaf(xv[u], xv[u], sx);
    }
  }
  if (!gain_next) return;
  const float rx = 1.0f / sqrtf(block_sum_256(sx, scratch) / (float)width + eps);
#pragma unroll
  for (int u = 0; u < PT; ++u) {
    const int c = threadIdx.x + u * 256;
    if (c < width) store_f(h, h_dtype, base + c, xv[u] * rx * (offset + gn[u]));
  }
}

// y_ptrs / gain_ptrs: n_branches device pointers each (float32 [n_rows, width] buffers; [width] gains, unused
// with one branch).  x, y: contiguous float32 rows.
extern "C" int mgpt_rms_post_norm(float* y0, float* y1, float* y2, float* y3, const float* g0, const float* g1,
                                  const float* g2, const float* g3, int n_branches, float coef, int join_unit, float* x,
                                  const float* gain_post, const float* scale_post, float offset, float eps, float mult,
                                  const float* gain_next,
                                  void* h, int h_dtype, int n_rows, int width, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!x || !y0 || !gain_post || (gain_next && !h)) return MGPT_ERR_NULL;
  if (n_rows < 0 || width <= 0 || n_branches < 1 || n_branches > RMS_MAX_BRANCHES) return MGPT_ERR_BAD_SHAPE;
  if (gain_next && !dtype_ok(h_dtype)) return MGPT_ERR_BAD_DTYPE;
  RmsBranches br = {{y0, y1, y2, y3}, {g0, g1, g2, g3}};
  for (int b = 0; b < n_branches; ++b)
    if (!br.y[b] || (n_branches > 1 && !br.gain[b])) return MGPT_ERR_NULL;
#define RPN_ROW(PT, NB)                                                                                              \
  hipLaunchKernelGGL((rms_post_norm_row_kernel<PT, NB>), dim3(n_rows), dim3(256), 0, stream, br, coef, join_unit, x, gain_post, \
                     scale_post, offset, eps, mult, gain_next, h, h_dtype, n_rows, width)
  if (n_branches == 1 && width <= 256 * 4) RPN_ROW(4, 1);
  else if (n_branches == 1 && width <= 256 * 8) RPN_ROW(8, 1);
  else if (n_branches == 1 && width <= 256 * 16) RPN_ROW(16, 1);
  else if (n_branches == 2 && width <= 256 * 4) RPN_ROW(4, 2);
  else if (n_branches == 2 && width <= 256 * 8) RPN_ROW(8, 2);
  else
    hipLaunchKernelGGL(rms_post_norm_kernel, dim3(n_rows), dim3(256), 0, stream, br, n_branches, coef, join_unit, x, gain_post,
                       scale_post, offset, eps, mult, gain_next, h, h_dtype, n_rows, width);
#undef RPN_ROW
  return mgpt_last_error();
}
