// Kernels of decoders that normalise a sublayer's OUTPUT only and average over the depth:
//     x <- x + w * rms(f(x))          (the sublayer reads the residual row itself; w = 1 + the stored weight, given as fp32)
//     after layer i:  X_(i+1) = x,    x <- sum_(j <= i+1) coef[j] * X_j      (X_0 = the embedding output)
//  * ssd_embed_hist         token rows of the embedding table -> fp32 residual rows, level 0 of the history, GEMM-input rows
//  * ssd_postnorm_tail      (routed mix ->) output norm + residual sum (-> history level + depth average) -> the next sublayer's input
//                           rows (the residual row in the element type), one launch
//  * ssd_rmsnorm_w32_rows   y = w * x / sqrt(mean(x^2) + eps) with fp32 weights, optional row gather (the model's last norm)
//  * ssd_rope_rows          rotary positions in place on column blocks of fp32 projection rows (q and k of a recurrent mixer)
//  * ssd_gate_rows          out = o * sigmoid(g) element by element, fp32 rows in, GEMM-input rows out
// All reductions and sums are fp32, one workgroup per row, a fixed order per row (independent of the batch): 256 threads, or 1024 for
// rows of >= 2048 entries in batches of <= 64 rows (changes the fp32 summation ORDER only).
// `f32` selects the element type of the embedding table and of GEMM-input rows: 0 = bf16, 1 = fp32.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }

template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < NT / 256; ++q) s += (red[4 * q] + red[4 * q + 1]) + (red[4 * q + 2] + red[4 * q + 3]);
  return s;
}

template <typename T>
__global__ void __launch_bounds__(256)
embed_hist_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table, float* __restrict__ x, float* __restrict__ hist0,
                  T* __restrict__ rows, int W, long vocab) {
  const size_t t = blockIdx.x;
  const long id = ids[t];
  const bool ok = id >= 0 && id < vocab;
  const T* src = table + (size_t)(ok ? id : 0) * W;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < W; c += 256 * gridDim.y) {
    const float v = ok ? ldf<T>(src + c) : 0.f;
    x[t * W + c] = v;
    if (hist0) hist0[t * W + c] = v;
    if (rows) stf<T>(rows + t * W + c, v);
  }
}

// One token row per workgroup.  v = the sublayer's fp32 output row, or the routed mix sum_j wt[t][j] * ydn[inv[t * top + j]] in slot
// order (kept in registers between the statistic and the sum for rows of up to 16 entries per thread, else computed twice with the
// same arithmetic);  x += w * v / sqrt(mean(v^2) + eps).
// With a history: level n - 1 receives x and x becomes sum_(j < n) coef[j] * level_j (j ascending; the newest level from registers).
template <typename T, int NT>
__global__ void __launch_bounds__(NT)
postnorm_tail_kernel(const float* __restrict__ y, const float* __restrict__ ydn, const int32_t* __restrict__ inv,
                     const float* __restrict__ wt, int top, const float* __restrict__ w, float eps, float* __restrict__ x,
                     float* __restrict__ hist, long hist_stride, int n, const float* __restrict__ coef, T* __restrict__ next_out, int W) {
  __shared__ float red[NT / 64];
  const size_t t = blockIdx.x;
  float* xr = x + t * W;
  auto val = [&](int c) -> float {
    if (y) return y[t * W + c];
    float v = 0.f;
    for (int j = 0; j < top; ++j) v = fmaf(wt[t * top + j], ydn[(size_t)inv[t * top + j] * W + c], v);
    return v;
  };
  constexpr int KEEP = 16;
  const bool kept = W <= KEEP * NT;
  float vk[KEEP];
  float ss = 0.f;
  if (kept) {
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      const int c = threadIdx.x + k * NT;
      vk[k] = c < W ? val(c) : 0.f;
      ss += vk[k] * vk[k];
    }
  } else {
    for (int c = threadIdx.x; c < W; c += NT) { const float v = val(c); ss += v * v; }
  }
  ss = block_sum<NT>(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  auto finish = [&](int c, float yv) {
    float v = xr[c] + yv * r * w[c];
    if (hist) {
      hist[(size_t)(n - 1) * hist_stride + t * W + c] = v;
      float a = 0.f;
      for (int j = 0; j + 1 < n; ++j) a = fmaf(coef[j], hist[(size_t)j * hist_stride + t * W + c], a);
      v = fmaf(coef[n - 1], v, a);
    }
    xr[c] = v;
    if (next_out) stf<T>(next_out + t * W + c, v);
  };
  if (kept) {
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      const int c = threadIdx.x + k * NT;
      if (c < W) finish(c, vk[k]);
    }
  } else {
    for (int c = threadIdx.x; c < W; c += NT) finish(c, val(c));
  }
}

template <typename T, int NT>
__global__ void __launch_bounds__(NT)
rmsnorm_w32_kernel(const float* __restrict__ x, const float* __restrict__ w, float eps, T* __restrict__ out,
                   const int32_t* __restrict__ gather, int W) {
  __shared__ float red[NT / 64];
  const size_t ro = blockIdx.x;
  const size_t ri = gather ? (size_t)gather[ro] : ro;
  const float* xr = x + ri * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) { const float v = xr[c]; ss += v * v; }
  ss = block_sum<NT>(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) stf<T>(out + ro * W + c, xr[c] * r * w[c]);
}

// Blocks of `heads` heads of D entries at columns off_a and off_b (off_b < 0: one block) of fp32 rows: the first rot_dims entries of a
// head turn (entry i pairs with i + rot_dims / 2) by positions[t] * freqs[i], then the whole head is multiplied by the block's scale.
__global__ void __launch_bounds__(256)
rope_rows_kernel(float* __restrict__ rows, long ld, const int64_t* __restrict__ positions, const float* __restrict__ freqs, int rot_dims,
                 int heads, int D, int off_a, float scale_a, int off_b, float scale_b) {
  const size_t t = blockIdx.x;
  const float pos = (float)positions[t];
  const int half = rot_dims >> 1, per = D - half;          // work items of a head: `half` pairs, then the entries that do not turn
  const int nblk = off_b >= 0 ? 2 : 1;
  for (int u = blockIdx.y * 256 + threadIdx.x; u < nblk * heads * per; u += 256 * gridDim.y) {
    const int blk = u / (heads * per), h = (u / per) % heads, i = u % per;
    float* p = rows + t * ld + (blk ? off_b : off_a) + h * D;
    const float sc = blk ? scale_b : scale_a;
    if (i < half) {
      float s, c;
      sincosf(pos * freqs[i], &s, &c);
      const float a = p[i], b = p[i + half];
      p[i] = (a * c - b * s) * sc;
      p[i + half] = (b * c + a * s) * sc;
    } else {
      p[i + half] *= sc;
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
gate_rows_kernel(const float* __restrict__ o, long ldo, const float* __restrict__ g, long ldg, T* __restrict__ out, int N) {
  const size_t t = blockIdx.x;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < N; c += 256 * gridDim.y)
    stf<T>(out + t * N + c, o[t * ldo + c] / (1.0f + expf(-g[t * ldg + c])));
}

inline int col_blocks(int rows, int cols) { return rows < 64 ? (cols + 255) / 256 > 64 ? 64 : (cols + 255) / 256 : 1; }

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_embed_hist(const int64_t* ids, const void* table, void* x_out, void* hist0, void* rows_out, int T, int W, long vocab,
                              int f32, void* stream) {
  if (!ids || !table || !x_out) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0 || vocab <= 0) return SSD_ERR_SHAPE;
  const dim3 grid(T, col_blocks(T, W));
  if (f32)
    hipLaunchKernelGGL(embed_hist_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, ids, (const float*)table, (float*)x_out,
                       (float*)hist0, (float*)rows_out, W, vocab);
  else
    hipLaunchKernelGGL(embed_hist_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, ids, (const bf16_t*)table, (float*)x_out,
                       (float*)hist0, (bf16_t*)rows_out, W, vocab);
  return LAUNCH_OK();
}

extern "C" int ssd_postnorm_tail(const void* y_rows, const void* ydn_rows, const int32_t* inv, const float* weights, int top,
                                 const float* post_weight, float eps, void* x, void* hist, long hist_stride, int hist_levels,
                                 const float* coef, void* next_out, int T, int W, int f32, void* stream) {
  if (!post_weight || !x) return SSD_ERR_ARG;
  if (!y_rows && (!ydn_rows || !inv || !weights || top <= 0)) return SSD_ERR_ARG;
  if (hist && (!coef || hist_levels < 1 || hist_stride < (long)T * W)) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0) return SSD_ERR_SHAPE;
#define POSTNORM(TY, NT)                                                                                                          \
  hipLaunchKernelGGL((postnorm_tail_kernel<TY, NT>), dim3(T), dim3(NT), 0, (hipStream_t)stream, (const float*)y_rows,             \
                     (const float*)ydn_rows, inv, weights, top, post_weight, eps, (float*)x, (float*)hist, hist_stride,           \
                     hist_levels, coef, (TY*)next_out, W)
  if (T <= 64 && W >= 2048) {
    if (f32) POSTNORM(float, 1024); else POSTNORM(bf16_t, 1024);
  } else {
    if (f32) POSTNORM(float, 256); else POSTNORM(bf16_t, 256);
  }
#undef POSTNORM
  return LAUNCH_OK();
}

extern "C" int ssd_rmsnorm_w32_rows(const void* x, const float* weight, float eps, void* out_rows, const int32_t* gather, int T, int W,
                                    int f32, void* stream) {
  if (!x || !weight || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0) return SSD_ERR_SHAPE;
#define NORM32(TY, NT)                                                                                                            \
  hipLaunchKernelGGL((rmsnorm_w32_kernel<TY, NT>), dim3(T), dim3(NT), 0, (hipStream_t)stream, (const float*)x, weight, eps,       \
                     (TY*)out_rows, gather, W)
  if (T <= 64 && W >= 2048) {
    if (f32) NORM32(float, 1024); else NORM32(bf16_t, 1024);
  } else {
    if (f32) NORM32(float, 256); else NORM32(bf16_t, 256);
  }
#undef NORM32
  return LAUNCH_OK();
}

extern "C" int ssd_rope_rows(void* rows, long ld, const int64_t* positions, const float* freqs, int rot_dims, int heads, int D, int off_a,
                             float scale_a, int off_b, float scale_b, int T, void* stream) {
  if (!rows || !positions || (rot_dims > 0 && !freqs)) return SSD_ERR_ARG;
  if (T <= 0 || heads <= 0 || D <= 0 || rot_dims < 0 || rot_dims > D || (rot_dims & 1) || off_a < 0 ||
      ld < (long)(off_a > off_b ? off_a : off_b) + (long)heads * D)
    return SSD_ERR_SHAPE;
  const int items = (off_b >= 0 ? 2 : 1) * heads * (D - rot_dims / 2);
  hipLaunchKernelGGL(rope_rows_kernel, dim3(T, col_blocks(T, items)), dim3(256), 0, (hipStream_t)stream, (float*)rows, ld, positions,
                     freqs, rot_dims, heads, D, off_a, scale_a, off_b, scale_b);
  return LAUNCH_OK();
}

extern "C" int ssd_gate_rows(const void* o_rows, long ldo, const void* gate_rows, long ldg, void* out_rows, int T, int N, int f32,
                             void* stream) {
  if (!o_rows || !gate_rows || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || N <= 0 || ldo < N || ldg < N) return SSD_ERR_SHAPE;
  const dim3 grid(T, col_blocks(T, N));
  if (f32)
    hipLaunchKernelGGL(gate_rows_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)o_rows, ldo,
                       (const float*)gate_rows, ldg, (float*)out_rows, N);
  else
    hipLaunchKernelGGL(gate_rows_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)o_rows, ldo,
                       (const float*)gate_rows, ldg, (bf16_t*)out_rows, N);
  return LAUNCH_OK();
}
