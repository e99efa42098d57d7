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
// All reductions are fp32, one workgroup of 256 threads per row, a fixed summation order per row (independent of the batch).
// `f32` selects the element type of weights and of GEMM-input rows: 0 = bf16, 1 = fp32.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }

__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

template <typename T>
__global__ void __launch_bounds__(256)
embed_pos_kernel(const int64_t* __restrict__ ids, const int64_t* __restrict__ positions, const T* __restrict__ table,
                 const T* __restrict__ pos_table, float* __restrict__ x, const T* __restrict__ w, float eps, T* __restrict__ out, int W,
                 long vocab, long max_pos) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const long id = ids[t], p = positions[t];
  const bool ok = id >= 0 && id < vocab && p >= 0 && p < max_pos;
  const T* src = table + (size_t)(ok ? id : 0) * W;
  const T* ps = pos_table + (size_t)(ok ? p : 0) * W;
  float* xr = x + (size_t)t * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = ok ? ldf<T>(src + c) + ldf<T>(ps + c) : 0.f;
    xr[c] = v;
    ss += v * v;
  }
  if (!w) return;
  ss = block_sum_256(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += 256) stf<T>(out + (size_t)t * W + c, xr[c] * r * ldf<T>(w + c));
}

template <typename T>
__global__ void __launch_bounds__(256)
prenorm_tail_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ ydn, const int32_t* __restrict__ inv,
                    const float* __restrict__ wt, int top, float eps, const T* __restrict__ w_next, T* __restrict__ next_out, int W) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
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
  ss = block_sum_256(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += 256) stf<T>(next_out + (size_t)t * W + c, xr[c] * r * ldf<T>(w_next + c));
}

template <typename T>
__global__ void __launch_bounds__(256)
polynorm_kernel(const float* __restrict__ z, const float* __restrict__ coef, float eps, T* __restrict__ out, int F) {
  __shared__ float red[4];
  const float* zr = z + (size_t)blockIdx.x * F;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int c = threadIdx.x; c < F; c += 256) {
    const float v = zr[c], v2 = v * v, v3 = v2 * v;
    s1 += v2; s2 += v2 * v2; s3 += v3 * v3;
  }
  s1 = block_sum_256(s1, red);
  s2 = block_sum_256(s2, red);
  s3 = block_sum_256(s3, red);
  const float r1 = coef[0] / sqrtf(s1 / (float)F + eps), r2 = coef[1] / sqrtf(s2 / (float)F + eps),
              r3 = coef[2] / sqrtf(s3 / (float)F + eps), e = coef[3];
  for (int c = threadIdx.x; c < F; c += 256) {
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
  if (f32)
    hipLaunchKernelGGL(embed_pos_kernel<float>, dim3(T), dim3(256), 0, (hipStream_t)stream, ids, positions, (const float*)table,
                       (const float*)pos_table, (float*)x_out, (const float*)norm_weight, eps, (float*)norm_out, W, vocab, max_pos);
  else
    hipLaunchKernelGGL(embed_pos_kernel<bf16_t>, dim3(T), dim3(256), 0, (hipStream_t)stream, ids, positions, (const bf16_t*)table,
                       (const bf16_t*)pos_table, (float*)x_out, (const bf16_t*)norm_weight, eps, (bf16_t*)norm_out, W, vocab, max_pos);
  return LAUNCH_OK();
}

extern "C" int ssd_prenorm_tail(void* x, const void* y_rows, const void* ydn_rows, const int32_t* inv, const float* weights, int top,
                                float eps, const void* next_weight, void* next_out, int T, int W, int f32, void* stream) {
  if (!x || ((next_weight == nullptr) != (next_out == nullptr))) return SSD_ERR_ARG;
  if (!y_rows && (!ydn_rows || !inv || top <= 0)) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(prenorm_tail_kernel<float>, dim3(T), dim3(256), 0, (hipStream_t)stream, (float*)x, (const float*)y_rows,
                       (const float*)ydn_rows, inv, weights, top, eps, (const float*)next_weight, (float*)next_out, W);
  else
    hipLaunchKernelGGL(prenorm_tail_kernel<bf16_t>, dim3(T), dim3(256), 0, (hipStream_t)stream, (float*)x, (const float*)y_rows,
                       (const float*)ydn_rows, inv, weights, top, eps, (const bf16_t*)next_weight, (bf16_t*)next_out, W);
  return LAUNCH_OK();
}

extern "C" int ssd_polynorm_rows(const void* z_rows, const float* coef, float eps, void* out_rows, int T, int F, int f32, void* stream) {
  if (!z_rows || !coef || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || F <= 0) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(polynorm_kernel<float>, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)z_rows, coef, eps,
                       (float*)out_rows, F);
  else
    hipLaunchKernelGGL(polynorm_kernel<bf16_t>, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)z_rows, coef, eps,
                       (bf16_t*)out_rows, F);
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
