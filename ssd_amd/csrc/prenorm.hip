// Kernels of pre-norm decoders over an fp32 residual stream:   x <- x + f(w * rms(x))
//  * ssd_embed_pos_res32   x = table[id] + pos_table[position] (a learned position vector, unscaled) as fp32 residual rows, and the first
//                          sublayer's norm of it in the same launch
//  * ssd_prenorm_tail      x += y (a sublayer's fp32 output rows, or the routed feed-forward's sum over a token's expert rows) and the
//                          NEXT sublayer's norm w_next * rms(x) as GEMM-input rows, one launch
//  * ssd_polynorm_rows     act(z) = a rms(z) + b rms(z^2) + c rms(z^3) + e over a token's row of feed-forward values (powers element by
//                          element, every power divided by its own root mean square)
//  * ssd_glu_clamp_rows    clamped swish-GLU rows  g = min(s zg, limit), u = clamp(s zu, -limit, limit), out = g sigmoid(alpha g) (u + 1);
//                          s = a per-row factor (a routing weight that multiplies the expert's INPUT: the products are linear in it, so it
//                          is applied to their fp32 results)
//  * ssd_logits_cap_rows   z <- cap * tanh(scale * z / cap) in place on fp32 logit rows (cap <= 0: only the scale)
// All reductions are fp32, one workgroup per row: 256 threads, or 1024 for rows of >= 2048 entries in batches of <= 64 rows (a
// dispatch that depends on the batch and changes the fp32 summation ORDER only).
// `f32` selects the element type of weights and of GEMM-input rows: 0 = bf16, 1 = fp32.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }

// sum over the workgroup's NT threads (a multiple of 256): waves summed in groups of four, the groups in order
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
// few rows: a row is a latency chain, so it gets 1024 threads (the summation order then differs from the 256-thread form's: the
// choice depends on the batch, the inputs and roundings do not)
static inline bool wide_rows(int T, int W) { return T <= 64 && W >= 2048; }

template <typename T, int NT>
__global__ void __launch_bounds__(NT)
embed_pos_kernel(const int64_t* __restrict__ ids, const int64_t* __restrict__ positions, const T* __restrict__ table,
                 const T* __restrict__ pos_table, float* __restrict__ x, const T* __restrict__ w, float eps, T* __restrict__ out, int W,
                 long vocab, long max_pos) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  const long id = ids[t], p = positions[t];
  const bool ok = id >= 0 && id < vocab && p >= 0 && p < max_pos;
  const T* src = table + (size_t)(ok ? id : 0) * W;
  const T* ps = pos_table + (size_t)(ok ? p : 0) * W;
  float* xr = x + (size_t)t * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) {
    const float v = ok ? ldf<T>(src + c) + ldf<T>(ps + c) : 0.f;
    xr[c] = v;
    ss += v * v;
  }
  if (!w) return;
  ss = block_sum<NT>(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) stf<T>(out + (size_t)t * W + c, xr[c] * r * ldf<T>(w + c));
}

template <typename T, int NT>
__global__ void __launch_bounds__(NT)
prenorm_tail_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ ydn, const int32_t* __restrict__ inv,
                    const float* __restrict__ wt, int top, float eps, const T* __restrict__ w_next, T* __restrict__ next_out, int W) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) {
    float v;
    if (y) {
      v = y[(size_t)t * W + c];
    } else {
      v = 0.f;
      for (int j = 0; j < top; ++j) {
        const float e = ydn[(size_t)inv[(size_t)t * top + j] * W + c];
        v = wt ? fmaf(wt[(size_t)t * top + j], e, v) : v + e;
      }
    }
    v += xr[c];
    xr[c] = v;
    ss += v * v;
  }
  if (!w_next) return;
  ss = block_sum<NT>(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) stf<T>(next_out + (size_t)t * W + c, xr[c] * r * ldf<T>(w_next + c));
}

template <typename T, int NT>
__global__ void __launch_bounds__(NT)
polynorm_kernel(const float* __restrict__ z, const float* __restrict__ coef, float eps, T* __restrict__ out, int F) {
  __shared__ float red[3][NT / 64];
  const float* zr = z + (size_t)blockIdx.x * F;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int c = threadIdx.x; c < F; c += NT) {
    const float v = zr[c], v2 = v * v, v3 = v2 * v;
    s1 += v2; s2 += v2 * v2; s3 += v3 * v3;
  }
  s1 = wave_sum(s1); s2 = wave_sum(s2); s3 = wave_sum(s3);
  if ((threadIdx.x & 63) == 0) { red[0][threadIdx.x >> 6] = s1; red[1][threadIdx.x >> 6] = s2; red[2][threadIdx.x >> 6] = s3; }
  __syncthreads();
  s1 = s2 = s3 = 0.f;
#pragma unroll
  for (int q = 0; q < NT / 256; ++q) {
    s1 += (red[0][4 * q] + red[0][4 * q + 1]) + (red[0][4 * q + 2] + red[0][4 * q + 3]);
    s2 += (red[1][4 * q] + red[1][4 * q + 1]) + (red[1][4 * q + 2] + red[1][4 * q + 3]);
    s3 += (red[2][4 * q] + red[2][4 * q + 1]) + (red[2][4 * q + 2] + red[2][4 * q + 3]);
  }
  const float r1 = coef[0] / sqrtf(s1 / (float)F + eps), r2 = coef[1] / sqrtf(s2 / (float)F + eps),
              r3 = coef[2] / sqrtf(s3 / (float)F + eps), e = coef[3];
  for (int c = threadIdx.x; c < F; c += NT) {
    const float v = zr[c], v2 = v * v;
    stf<T>(out + (size_t)blockIdx.x * F + c, v * r1 + v2 * r2 + v2 * v * r3 + e);
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
glu_clamp_kernel(const float* __restrict__ ab, const float* __restrict__ row_scale, const int32_t* __restrict__ perm,
                 T* __restrict__ out, int F, float limit, float alpha) {
  const size_t r = blockIdx.x;
  const float s = row_scale ? row_scale[perm ? perm[r] : r] : 1.0f;
  const float* row = ab + r * 2 * F;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < F; c += 256 * gridDim.y) {
    const float g = fminf(s * row[c], limit);
    const float u = fminf(fmaxf(s * row[F + c], -limit), limit);
    stf<T>(out + r * F + c, g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
  }
}

__global__ void __launch_bounds__(256)
logits_cap_kernel(float* __restrict__ z, int V, long ld, float scale, float cap) {
  float* row = z + (size_t)blockIdx.x * ld;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < V; c += 256 * gridDim.y) {
    const float v = row[c] * scale;
    row[c] = cap > 0.f ? cap * tanhf(v / cap) : v;
  }
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_embed_pos_res32(const int64_t* ids, const int64_t* positions, const void* table, const void* pos_table, void* x_out,
                                   const void* norm_weight, float eps, void* norm_out, int T, int W, long vocab, long max_pos, int f32,
                                   void* stream) {
  if (!ids || !positions || !table || !pos_table || !x_out || ((norm_weight == nullptr) != (norm_out == nullptr))) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0 || vocab <= 0 || max_pos <= 0) return SSD_ERR_SHAPE;
#define EMBED_POS(TY, NT)                                                                                                       \
  hipLaunchKernelGGL((embed_pos_kernel<TY, NT>), dim3(T), dim3(NT), 0, (hipStream_t)stream, ids, positions, (const TY*)table, \
                     (const TY*)pos_table, (float*)x_out, (const TY*)norm_weight, eps, (TY*)norm_out, W, vocab, max_pos)
  if (wide_rows(T, W)) { if (f32) EMBED_POS(float, 1024); else EMBED_POS(bf16_t, 1024); }
  else { if (f32) EMBED_POS(float, 256); else EMBED_POS(bf16_t, 256); }
#undef EMBED_POS
  return LAUNCH_OK();
}

extern "C" int ssd_prenorm_tail(void* x, const void* y_rows, const void* ydn_rows, const int32_t* inv, const float* weights, int top,
                                float eps, const void* next_weight, void* next_out, int T, int W, int f32, void* stream) {
  if (!x || ((next_weight == nullptr) != (next_out == nullptr))) return SSD_ERR_ARG;
  if (!y_rows && (!ydn_rows || !inv || top <= 0)) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0) return SSD_ERR_SHAPE;
#define PRENORM_TAIL(TY, NT)                                                                                                        \
  hipLaunchKernelGGL((prenorm_tail_kernel<TY, NT>), dim3(T), dim3(NT), 0, (hipStream_t)stream, (float*)x, (const float*)y_rows,   \
                     (const float*)ydn_rows, inv, weights, top, eps, (const TY*)next_weight, (TY*)next_out, W)
  if (wide_rows(T, W)) { if (f32) PRENORM_TAIL(float, 1024); else PRENORM_TAIL(bf16_t, 1024); }
  else { if (f32) PRENORM_TAIL(float, 256); else PRENORM_TAIL(bf16_t, 256); }
#undef PRENORM_TAIL
  return LAUNCH_OK();
}

extern "C" int ssd_polynorm_rows(const void* z_rows, const float* coef, float eps, void* out_rows, int T, int F, int f32, void* stream) {
  if (!z_rows || !coef || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || F <= 0) return SSD_ERR_SHAPE;
#define POLYNORM(TY, NT)                                                                                                      \
  hipLaunchKernelGGL((polynorm_kernel<TY, NT>), dim3(T), dim3(NT), 0, (hipStream_t)stream, (const float*)z_rows, coef, eps, \
                     (TY*)out_rows, F)
  if (wide_rows(T, F)) { if (f32) POLYNORM(float, 1024); else POLYNORM(bf16_t, 1024); }
  else { if (f32) POLYNORM(float, 256); else POLYNORM(bf16_t, 256); }
#undef POLYNORM
  return LAUNCH_OK();
}

extern "C" int ssd_glu_clamp_rows(const void* ab_rows, const float* row_scale, const int32_t* perm, void* out_rows, int rows, int F,
                                  float limit, float alpha, int f32, void* stream) {
  if (!ab_rows || !out_rows || (perm && !row_scale)) return SSD_ERR_ARG;
  if (rows <= 0 || F <= 0 || !(limit > 0.f)) return SSD_ERR_SHAPE;
  const dim3 grid(rows, rows < 64 ? (F + 255) / 256 : 1);
  if (f32)
    hipLaunchKernelGGL(glu_clamp_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)ab_rows, row_scale, perm,
                       (float*)out_rows, F, limit, alpha);
  else
    hipLaunchKernelGGL(glu_clamp_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)ab_rows, row_scale, perm,
                       (bf16_t*)out_rows, F, limit, alpha);
  return LAUNCH_OK();
}

extern "C" int ssd_logits_cap_rows(void* logits, int rows, int V, long ld, float scale, float cap, void* stream) {
  if (!logits) return SSD_ERR_ARG;
  if (rows <= 0 || V <= 0 || ld < V) return SSD_ERR_SHAPE;
  hipLaunchKernelGGL(logits_cap_kernel, dim3(rows, (V + 2047) / 2048), dim3(256), 0, (hipStream_t)stream, (float*)logits, V, ld, scale, cap);
  return LAUNCH_OK();
}
