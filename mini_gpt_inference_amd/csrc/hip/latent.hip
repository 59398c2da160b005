// Latent attention's own steps: the RMS-normed latent stored into its pages, and the products
// that every head makes with a matrix of its own (queries folded onto the latent basis before
// attention, the attended latents unfolded into the head's values after it).
//
// A latent pool is [pages][1][page_size][rank]: one row per cached token, keys and values both
// come from it, so slot s lies at s * rank.
#include "common.h"
#include "launchers.h"

// c = v / sqrt(mean(v^2) + eps) * gain, statistics and product in 32-bit; one wave per token
template <typename T>
__global__ void rms_norm_store_kernel(const T* __restrict__ src, long ld, const float* __restrict__ gain,
                                      float eps, T* __restrict__ pool, const int* __restrict__ slot_mapping,
                                      int n_tokens, int rank) {
  const int lane = threadIdx.x & (MGPT_WAVE - 1);
  const int row = blockIdx.x * (blockDim.x / MGPT_WAVE) + (threadIdx.x / MGPT_WAVE);
  if (row >= n_tokens) return;
  const int slot = slot_mapping[row];
  if (slot < 0) return;  // padded row
  const T* r = src + (long)row * ld;
  float ss = 0.f;
  for (int c = lane; c < rank; c += MGPT_WAVE) {
    const float v = to_float<T>(r[c]);
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
  T* dst = pool + (long)slot * rank;
  for (int c = lane; c < rank; c += MGPT_WAVE) dst[c] = from_float<T>(to_float<T>(r[c]) * inv * gain[c]);
}

// src: [n_tokens, rank] with row stride ld (already offset to the latent's columns); pool: the
// latent pages, same dtype.
extern "C" int mgpt_rms_norm_store(const void* src, int dtype, long ld, const float* gain, float eps, void* pool,
                                   const int* slot_mapping, int n_tokens, int rank, hipStream_t stream) {
  if (n_tokens == 0) return MGPT_OK;
  if (!src || !gain || !pool || !slot_mapping) return MGPT_ERR_NULL;
  if (n_tokens < 0 || rank <= 0 || ld < rank) return MGPT_ERR_BAD_SHAPE;
  dim3 grid((n_tokens + 3) / 4), block(4 * MGPT_WAVE);
  if (dtype == MGPT_F32)
    hipLaunchKernelGGL(rms_norm_store_kernel<float>, grid, block, 0, stream, (const float*)src, ld, gain, eps,
                       (float*)pool, slot_mapping, n_tokens, rank);
  else if (dtype == MGPT_BF16)
    hipLaunchKernelGGL(rms_norm_store_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)src, ld, gain, eps,
                       (bf16_t*)pool, slot_mapping, n_tokens, rank);
  else
    return MGPT_ERR_BAD_DTYPE;
  return mgpt_last_error();
}

// A latent with a rotated part.  A cached row is [c: rank | kr: rot_dim | zeros up to row_width]: c as above,
// kr one key part that all heads share, rotated by the token's position; a query head is [plain: head_dim |
// rotated: rot_dim] and its rotated part is rotated in place.  Rotation of pairs (i, i + rot_dim / 2) by the angle
// position * freq[i], cosine and sine both times rot_mag, in 32-bit.  One workgroup a token.  Without a pool
// (a layer that reads another layer's latents) only the queries are rotated.
#define LP_MAX_HALF 256
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    T* __restrict__ z, long ldz, int q_off, int n_head, int head_dim, int rot_dim, int c_off, int rank,
    const float* __restrict__ gain, float eps, const int* __restrict__ positions, const float* __restrict__ freq,
    float rot_mag, T* __restrict__ pool, int row_width, const int* __restrict__ slot_mapping, int n_tokens) {
  __shared__ float cos_s[LP_MAX_HALF], sin_s[LP_MAX_HALF];
  __shared__ float red_s[4];
  const int n = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = rot_dim / 2;
  const float p = (float)positions[n];
  for (int i = tid; i < half; i += 256) {
    const float a = p * freq[i];
    cos_s[i] = cosf(a) * rot_mag;
    sin_s[i] = sinf(a) * rot_mag;
  }
  T* row = z + (long)n * ldz;
  const int slot = pool ? slot_mapping[n] : -1;
  float ss = 0.f;
  if (slot >= 0)
    for (int c = tid; c < rank; c += 256) {
      const float v = to_float<T>(row[c_off + c]);
      ss = fmaf(v, v, ss);
    }
  ss = wave_sum(ss);
  if (lane == 0) red_s[wave] = ss;
  __syncthreads();
  for (int idx = tid; idx < n_head * half; idx += 256) {
    const int h = idx / half, i = idx - h * half;
    T* at = row + q_off + (long)h * (head_dim + rot_dim) + head_dim;
    const float u = to_float<T>(at[i]), w = to_float<T>(at[i + half]);
    at[i] = from_float<T>(u * cos_s[i] - w * sin_s[i]);
    at[i + half] = from_float<T>(w * cos_s[i] + u * sin_s[i]);
  }
  if (slot < 0) return;
  const float inv = 1.0f / sqrtf(((red_s[0] + red_s[1]) + (red_s[2] + red_s[3])) / (float)rank + eps);
  T* dst = pool + (long)slot * row_width;
  for (int c = tid; c < rank; c += 256) dst[c] = from_float<T>(to_float<T>(row[c_off + c]) * inv * gain[c]);
  for (int i = tid; i < half; i += 256) {
    const float u = to_float<T>(row[c_off + rank + i]), w = to_float<T>(row[c_off + rank + i + half]);
    dst[rank + i] = from_float<T>(u * cos_s[i] - w * sin_s[i]);
    dst[rank + i + half] = from_float<T>(w * cos_s[i] + u * sin_s[i]);
  }
  for (int c = rank + rot_dim + tid; c < row_width; c += 256) dst[c] = from_float<T>(0.f);
}

// z: the step's projected rows (queries at q_off, n_head heads of head_dim + rot_dim; the latent's rank + rot_dim
// columns at c_off); pool: the latent pages with rows of row_width >= rank + rot_dim values, or null.
extern "C" int mgpt_latent_prepare(void* z, int dtype, long ldz, int q_off, int n_head, int head_dim, int rot_dim,
                                   int c_off, int rank, const float* gain, float eps, const int* positions,
                                   const float* freq, float rot_mag, void* pool, int row_width,
                                   const int* slot_mapping, int n_tokens, hipStream_t stream) {
  if (n_tokens == 0) return MGPT_OK;
  if (!z || !positions || !freq || (pool && (!gain || !slot_mapping))) return MGPT_ERR_NULL;
  if (n_tokens < 0 || n_head <= 0 || head_dim < 0 || rot_dim <= 0 || (rot_dim & 1) || rot_dim / 2 > LP_MAX_HALF ||
      q_off < 0 || ldz < q_off + (long)n_head * (head_dim + rot_dim) ||
      (pool && (rank <= 0 || row_width < rank + rot_dim || c_off < 0 || ldz < c_off + rank + rot_dim)))
    return MGPT_ERR_BAD_SHAPE;
  if (dtype == MGPT_F32)
    hipLaunchKernelGGL(latent_prepare_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, (float*)z, ldz, q_off, n_head,
                       head_dim, rot_dim, c_off, rank, gain, eps, positions, freq, rot_mag, (float*)pool, row_width,
                       slot_mapping, n_tokens);
  else if (dtype == MGPT_BF16)
    hipLaunchKernelGGL(latent_prepare_kernel<bf16_t>, dim3(n_tokens), dim3(256), 0, stream, (bf16_t*)z, ldz, q_off, n_head,
                       head_dim, rot_dim, c_off, rank, gain, eps, positions, freq, rot_mag, (bf16_t*)pool, row_width,
                       slot_mapping, n_tokens);
  else
    return MGPT_ERR_BAD_DTYPE;
  return mgpt_last_error();
}

// out[n][h][o] = sum_i a[n][h][i] * w[h][o][i], optionally times sigmoid(gate[n][h][o]).
// A workgroup owns 16 rows x 16 columns of one head, one element a thread; k runs 0..K-1 in order
// for every element, so a row's result does not depend on the other rows of the launch.
#define HL_TILE 16
#define HL_BK 64

template <typename T, bool FAST>
__global__ __launch_bounds__(256) void heads_linear_kernel(
    const T* __restrict__ A, long lda, const T* __restrict__ W, T* __restrict__ out, long ldo,
    const T* __restrict__ gate, long ldg, int n_rows, int n_out, int k_dim) {
  __shared__ float As[HL_TILE][HL_BK + 1];
  __shared__ float Ws[HL_TILE][HL_BK + 1];
  const int tid = threadIdx.x, head = blockIdx.z;
  const int r = tid >> 4, c = tid & 15;
  const int sk = (tid & 15) * 4;
  const int row0 = blockIdx.y * HL_TILE, col0 = blockIdx.x * HL_TILE;
  const bool a_ok = row0 + r < n_rows, w_ok = col0 + r < n_out;
  const T* ap = A + (long)(row0 + r) * lda + (long)head * k_dim + sk;
  const T* wp = W + ((long)head * n_out + col0 + r) * (long)k_dim + sk;
  float acc = 0.f;
  for (int k0 = 0; k0 < k_dim; k0 += HL_BK) {
    const int kmax = k_dim - k0 < HL_BK ? k_dim - k0 : HL_BK;
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
  const int row = row0 + r, col = col0 + c;
  if (row >= n_rows || col >= n_out) return;
  float v = acc;
  if (gate) {
    const float g = to_float<T>(gate[(long)row * ldg + (long)head * n_out + col]);
    v *= FAST ? __builtin_amdgcn_rcpf(1.0f + __expf(-g)) : 1.0f / (1.0f + expf(-g));
  }
  out[(long)row * ldo + (long)head * n_out + col] = from_float<T>(v);
}

extern "C" int mgpt_heads_linear(const void* a, long lda, const void* w, void* out, long ldo, const void* gate,
                                 long ldg, int n_rows, int n_head, int n_out, int k_dim, int dtype, int fast,
                                 hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!a || !w || !out) return MGPT_ERR_NULL;
  if (n_rows < 0 || n_head <= 0 || n_out <= 0 || k_dim <= 0 || lda < (long)n_head * k_dim ||
      ldo < (long)n_head * n_out || (gate && ldg < (long)n_head * n_out))
    return MGPT_ERR_BAD_SHAPE;
  if (n_head > 65535 || (n_rows + HL_TILE - 1) / HL_TILE > 65535) return MGPT_ERR_TOO_LARGE;
  dim3 grid((n_out + HL_TILE - 1) / HL_TILE, (n_rows + HL_TILE - 1) / HL_TILE, n_head), block(256);
#define HL_LAUNCH(T, F)                                                                                   \
  hipLaunchKernelGGL((heads_linear_kernel<T, F>), grid, block, 0, stream, (const T*)a, lda, (const T*)w,  \
                     (T*)out, ldo, (const T*)gate, ldg, n_rows, n_out, k_dim)
  if (dtype == MGPT_F32) {
    if (fast) HL_LAUNCH(float, true); else HL_LAUNCH(float, false);
  } else if (dtype == MGPT_BF16) {
    if (fast) HL_LAUNCH(bf16_t, true); else HL_LAUNCH(bf16_t, false);
  } else {
    return MGPT_ERR_BAD_DTYPE;
  }
#undef HL_LAUNCH
  return mgpt_last_error();
}

// The same products in bfloat16 on the MFMA units.  A wave owns 64 rows x up to 128 columns of one
// head (a workgroup, four waves, 256 rows): per 32 k it loads the slices of the head's matrix for
// its columns (the first MFMA operand, 16 bytes a lane straight from memory; a head's matrix is a
// few KB and stays in the cache) and four slices of the rows, and a lane ends up with four
// neighbouring columns of one row in each result.  Inner sizes in steps of 8, outputs in steps of 4.
typedef __attribute__((__vector_size__(8 * sizeof(short)))) short hl_bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float hl_f32x4_t;

template <int NJ>
__global__ __launch_bounds__(256) void heads_linear_mfma_kernel(
    const bf16_t* __restrict__ A, long lda, const bf16_t* __restrict__ W, bf16_t* __restrict__ out, long ldo,
    const bf16_t* __restrict__ gate, long ldg, int n_rows, int n_out, int k_dim) {
  // a wave owns 64 rows x NJ * 16 columns of one head: the rows are read once for all those columns
  const int head = blockIdx.z, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row0 = (blockIdx.y * 4 + wave) * 64, col0 = blockIdx.x * (NJ * 16);
  if (row0 >= n_rows) return;   // the whole wave; the kernel has no barrier
  const int li = lane & 15, lg = lane >> 4;
  const bf16_t* wrow[NJ];
  bool w_ok[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    w_ok[j] = col0 + j * 16 + li < n_out;
    wrow[j] = W + ((long)head * n_out + (w_ok[j] ? col0 + j * 16 + li : 0)) * (long)k_dim;
  }
  const bf16_t* arow[4];
  bool a_ok[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int r = row0 + 16 * t + li;
    a_ok[t] = r < n_rows;
    arow[t] = A + (long)(a_ok[t] ? r : 0) * lda + (long)head * k_dim;
  }
  const hl_bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  hl_f32x4_t acc[NJ][4];
#pragma unroll
  for (int j = 0; j < NJ; ++j)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[j][t] = hl_f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < k_dim; k0 += 32) {
    const int k = k0 + lg * 8;
    const bool k_ok = k < k_dim;
    hl_bf16x8_t wf[NJ], af[4];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      wf[j] = (w_ok[j] && k_ok) ? *reinterpret_cast<const hl_bf16x8_t*>(wrow[j] + k) : zero;
#pragma unroll
    for (int t = 0; t < 4; ++t)
      af[t] = (a_ok[t] && k_ok) ? *reinterpret_cast<const hl_bf16x8_t*>(arow[t] + k) : zero;
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], af[t], acc[j][t], 0, 0, 0);
  }
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int c = col0 + j * 16 + lg * 4;   // this lane's four columns, of row 16 t + li
    if (c >= n_out) continue;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int r = row0 + 16 * t + li;
      if (r >= n_rows) continue;
      float v[4] = {acc[j][t][0], acc[j][t][1], acc[j][t][2], acc[j][t][3]};
      if (gate) {
        const uint2 g = *reinterpret_cast<const uint2*>(gate + (long)r * ldg + (long)head * n_out + c);
        const float gv[4] = {bf16_to_float((bf16_t)(g.x & 0xffff)), bf16_to_float((bf16_t)(g.x >> 16)),
                             bf16_to_float((bf16_t)(g.y & 0xffff)), bf16_to_float((bf16_t)(g.y >> 16))};
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] *= __builtin_amdgcn_rcpf(1.0f + __expf(-gv[i]));
      }
      uint2 pk;
      pk.x = pack_bf16x2(v[0], v[1]);
      pk.y = pack_bf16x2(v[2], v[3]);
      *reinterpret_cast<uint2*>(out + (long)r * ldo + (long)head * n_out + c) = pk;
    }
  }
}

// bfloat16 only.  Refuses (MGPT_ERR_BAD_SHAPE) inner sizes that are no multiple of 8, outputs
// that are no multiple of 4 and rows or bases that are not aligned for 16-byte loads and 8-byte
// stores; the caller then takes mgpt_heads_linear.
extern "C" int mgpt_heads_linear_mfma(const void* a, long lda, const void* w, void* out, long ldo, const void* gate,
                                      long ldg, int n_rows, int n_head, int n_out, int k_dim, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!a || !w || !out) return MGPT_ERR_NULL;
  if (n_rows < 0 || n_head <= 0 || n_out <= 0 || k_dim <= 0 || lda < (long)n_head * k_dim ||
      ldo < (long)n_head * n_out || (gate && ldg < (long)n_head * n_out))
    return MGPT_ERR_BAD_SHAPE;
  if ((k_dim & 7) || (n_out & 3) || (lda & 7) || (ldo & 3) || (gate && (ldg & 3)) || (((size_t)a | (size_t)w) & 15) ||
      (((size_t)out | (size_t)gate) & 7))
    return MGPT_ERR_BAD_SHAPE;
  if (n_head > 65535 || (n_rows + 255) / 256 > 65535) return MGPT_ERR_TOO_LARGE;
  // columns a wave, in sixteens: as many as still leave about a thousand waves (a wave's rows are read
  // once for all of its columns), one sixteen where the rows are few
  int nj = 8;
  while (nj > 1 && (nj * 16 > n_out + 15 ||
                    (long)((n_rows + 63) / 64) * ((n_out + nj * 16 - 1) / (nj * 16)) * n_head < 1024))
    nj >>= 1;
  dim3 grid((n_out + nj * 16 - 1) / (nj * 16), (n_rows + 255) / 256, n_head), block(256);
#define HM_LAUNCH(NJ)                                                                                        \
  hipLaunchKernelGGL(heads_linear_mfma_kernel<NJ>, grid, block, 0, stream, (const bf16_t*)a, lda,            \
                     (const bf16_t*)w, (bf16_t*)out, ldo, (const bf16_t*)gate, ldg, n_rows, n_out, k_dim)
  if (nj == 1) HM_LAUNCH(1);
  else if (nj == 2) HM_LAUNCH(2);
  else if (nj == 4) HM_LAUNCH(4);
  else HM_LAUNCH(8);
#undef HM_LAUNCH
  return mgpt_last_error();
}
