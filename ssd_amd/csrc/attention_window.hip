// Sliding-window attention over the paged KV cache with unit-RMS queries and keys, capped scores, a per-head linear distance penalty
// and a softmax sink:
//     s_ij = cap * tanh(scale * <q_i, k_j> / cap) - slope_h * (i - j)          for  0 <= i - j < window  (window 0: every earlier key)
//     p_ij = exp(s_ij) / (sum_j' exp(s_ij') + exp(sink_h)),   o_i = sum_j p_ij v_j
// q and k are divided by their root mean square over the head's D entries (no weight); the sink has no key and no value and only joins
// the denominator; there is no rotation -- positions enter through the penalty and the window only.  Grouped key / value heads (query
// head h reads kv head h / (H / G)); query / key size D and value size Dv are independent (any D, Dv <= 512); element type bf16 or fp32.
//   cache layout per layer: K [blocks][G][block_size][D] (normalised), V TRANSPOSED per page [blocks][G][Dv][block_size]
//   * ssd_winattn_store   from the fused projection's fp32 rows [q | k | v]: norm q -> q_out, norm k -> K cache at slots[t], v -> V cache.
//   * ssd_winattn_paged   scalar form: one workgroup per (token, head); its 4 waves take 64-key tiles round-robin, the tiles START at
//                         the window's first key (so a row's summation order is a function of its own position only); a lane owns a
//                         KEY for the scores and a VALUE COLUMN for the sums; partial (max, sum, accumulator) triples merge in LDS in
//                         wave order, then the sink joins the denominator.
//                         MFMA form (bf16, D % 32 == 0, D <= 256, Dv % 16 == 0, Dv <= 256, block_size % 32 == 0): see below.
//   Scores, weights, sums and norms are fp32 whatever the element type.  A token's position and sequence come from positions[] and
//   cu_q[] (varlen batches: prompt portions beside single tokens) or q_per_seq (fixed rows per sequence).
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }

constexpr int WA_MAXV = 8;      // value columns per lane: Dv <= 512

template <typename T>
__global__ void __launch_bounds__(256)
winattn_store_kernel(const float* __restrict__ qkv, long ld, float eps, const int32_t* __restrict__ slots, T* __restrict__ q_out,
                     T* __restrict__ kc, T* __restrict__ vc, int H, int G, int D, int Dv, int bs) {
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int Nq = H * D, Nk = G * D, Nv = G * Dv;
  const float* row = qkv + (size_t)t * ld;
  const int slot = slots[t];
  const long blk = slot >= 0 ? slot / bs : 0;
  const int off = slot >= 0 ? slot % bs : 0;
  // one wave per head vector (q heads, then k heads); grid.y cuts the units so that a single decoding token spreads over workgroups
  for (int u = blockIdx.y * 4 + wave; u < H + G; u += 4 * gridDim.y) {
    const bool isq = u < H;
    const float* src = row + (size_t)u * D;            // k heads follow the q heads in the row
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) { const float v = src[d]; ss += v * v; }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)D + eps);
    if (isq) {
      T* dst = q_out + (size_t)t * Nq + (size_t)u * D;
      for (int d = lane; d < D; d += 64) stf<T>(dst + d, src[d] * r);
    } else if (slot >= 0) {
      T* dst = kc + (((size_t)blk * G + (u - H)) * bs + off) * D;
      for (int d = lane; d < D; d += 64) stf<T>(dst + d, src[d] * r);
    }
  }
  if (slot >= 0) {
    for (int c = blockIdx.y * 256 + threadIdx.x; c < Nv; c += 256 * gridDim.y) {
      const int g = c / Dv, d = c % Dv;
      stf<T>(vc + (((size_t)blk * G + g) * Dv + d) * bs + off, row[Nq + Nk + c]);
    }
  }
}

__device__ __forceinline__ int seq_of_row(const int32_t* cu_q, int q_per_seq, int B, int t) {
  if (!cu_q) return t / q_per_seq;
  int lo = 0, hi = B;
  while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (cu_q[mid] <= t) lo = mid; else hi = mid; }
  return lo;
}

template <typename T>
__global__ void __launch_bounds__(256)
winattn_paged_kernel(const T* __restrict__ q, const T* __restrict__ kc, const T* __restrict__ vc, const float* __restrict__ slopes,
                     const float* __restrict__ sinks, const int32_t* __restrict__ bt, int max_blocks,
                     const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_q, int q_per_seq, int B, int H, int G, int D,
                     int Dv, int bs, int window, float scale, float cap, T* __restrict__ out) {
  extern __shared__ float smem[];
  const int t = blockIdx.x, h = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = h / (H / G);
  float* sq = smem;                          // [D]
  float* sp = sq + D + (D & 1);              // [4 waves][64] weights of the current tile
  long* srow = reinterpret_cast<long*>(sp + 4 * 64);       // [4 waves][64] V^T address of every key of the tile
  float* sacc = reinterpret_cast<float*>(srow + 4 * 64);   // [4 waves][Dv]
  float* sml = sacc + 4 * Dv;                // [4 waves][2]

  const int b = seq_of_row(cu_q, q_per_seq, B, t);
  const int pos = (int)positions[t];
  const int first = window > 0 && pos + 1 > window ? pos + 1 - window : 0;
  const int nkeys = pos + 1 - first;
  const int32_t* table = bt + (size_t)b * max_blocks;
  const float slope = slopes ? slopes[h] : 0.f;

  const T* qrow = q + ((size_t)t * H + h) * D;
  for (int d = threadIdx.x; d < D; d += 256) sq[d] = ldf<T>(qrow + d);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float a[WA_MAXV];
#pragma unroll
  for (int i = 0; i < WA_MAXV; ++i) a[i] = 0.f;
  float* pw = sp + wave * 64;
  long* rowp = srow + wave * 64;
  const int ntiles = (nkeys + 63) >> 6;
  for (int kt = wave; kt < ntiles; kt += 4) {
    const int j = first + kt * 64 + lane;
    float s = -INFINITY;
    long crow = 0;
    if (j <= pos) {
      const long pg = (long)table[j / bs] * G + g;
      crow = pg * Dv * bs + (j % bs);
      const T* kr = kc + (size_t)(pg * bs + (j % bs)) * D;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(sq[d], ldf<T>(kr + d), dot);
      s = dot * scale;
      if (cap > 0.f) s = cap * tanhf(s / cap);
      s -= slope * (float)(pos - j);
    }
    const float n = fmaxf(m, wave_max(s));
    const float c = expf(m - n);                  // first tile: exp(-inf) = 0
    const float e = j <= pos ? expf(s - n) : 0.f;
    l = l * c + wave_sum(e);
    m = n;
    pw[lane] = e; rowp[lane] = crow;
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);           // lgkmcnt(0): this wave's LDS writes have landed
    const int cnt = min(64, nkeys - kt * 64);
#pragma unroll
    for (int i = 0; i < WA_MAXV; ++i) a[i] *= c;
    for (int jj = 0; jj < cnt; ++jj) {
      const float w = pw[jj];
      const T* vr = vc + (size_t)rowp[jj];
#pragma unroll
      for (int i = 0; i < WA_MAXV; ++i) {
        const int d = lane + i * 64;
        if (d < Dv) a[i] = fmaf(w, ldf<T>(vr + (size_t)d * bs), a[i]);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
#pragma unroll
  for (int i = 0; i < WA_MAXV; ++i) {
    const int d = lane + i * 64;
    if (d < Dv) sacc[wave * Dv + d] = a[i];
  }
  if (lane == 0) { sml[wave * 2] = m; sml[wave * 2 + 1] = l; }
  __syncthreads();
  const float sink = sinks ? sinks[h] : -INFINITY;
  float M = sink;
  for (int w = 0; w < 4; ++w) M = fmaxf(M, sml[w * 2]);
  float L = sinks ? expf(sink - M) : 0.f, f[4];
  for (int w = 0; w < 4; ++w) {
    f[w] = sml[w * 2 + 1] > 0.f ? expf(sml[w * 2] - M) : 0.f;
    L += sml[w * 2 + 1] * f[w];
  }
  for (int d = threadIdx.x; d < Dv; d += 256) {
    float s = 0.f;
    for (int w = 0; w < 4; ++w) s += sacc[w * Dv + d] * f[w];
    stf<T>(out + ((size_t)t * H + h) * Dv + d, s / L);
  }
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_winattn_store(const void* qkv_rows, long ld, float eps, const int32_t* slots, void* q_out, void* k_cache,
                                 void* v_cache, int T, int H, int G, int D, int Dv, int block_size, int f32, void* stream) {
  if (!qkv_rows || !slots || !q_out || !k_cache || !v_cache) return SSD_ERR_ARG;
  if (T <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || block_size <= 0 || ld < (long)(H + G) * D + (long)G * Dv)
    return SSD_ERR_SHAPE;
  const int units = (H + G + 3) / 4;
  const dim3 grid(T, T >= 256 ? 1 : (units < 16 ? units : 16));
  if (f32)
    hipLaunchKernelGGL(winattn_store_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)qkv_rows, ld, eps, slots,
                       (float*)q_out, (float*)k_cache, (float*)v_cache, H, G, D, Dv, block_size);
  else
    hipLaunchKernelGGL(winattn_store_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)qkv_rows, ld, eps, slots,
                       (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, H, G, D, Dv, block_size);
  return LAUNCH_OK();
}

extern "C" int ssd_winattn_paged(const void* q_rows, const void* k_cache, const void* v_cache, const float* slopes, const float* sinks,
                                 const int32_t* block_tables, int max_blocks, const int64_t* positions, const int32_t* cu_q,
                                 int q_per_seq, int B, int T, int H, int G, int D, int Dv, int block_size, int window, float scale,
                                 float cap, void* out_rows, int f32, void* stream) {
  if (!q_rows || !k_cache || !v_cache || !block_tables || !positions || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || B <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || Dv > 64 * WA_MAXV || block_size <= 0 || window < 0 ||
      max_blocks <= 0 || (!cu_q && q_per_seq <= 0) || H > 65535)
    return SSD_ERR_SHAPE;
  const size_t bytes = ((size_t)D + (D & 1) + 4 * 64 + 2 * 4 * 64 + 4 * (size_t)Dv + 8) * sizeof(float);
  if (bytes > 64 * 1024) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(winattn_paged_kernel<float>, dim3(T, H), dim3(256), bytes, (hipStream_t)stream, (const float*)q_rows,
                       (const float*)k_cache, (const float*)v_cache, slopes, sinks, block_tables, max_blocks, positions, cu_q, q_per_seq,
                       B, H, G, D, Dv, block_size, window, scale, cap, (float*)out_rows);
  else
    hipLaunchKernelGGL(winattn_paged_kernel<bf16_t>, dim3(T, H), dim3(256), bytes, (hipStream_t)stream, (const bf16_t*)q_rows,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, slopes, sinks, block_tables, max_blocks, positions, cu_q,
                       q_per_seq, B, H, G, D, Dv, block_size, window, scale, cap, (bf16_t*)out_rows);
  return LAUNCH_OK();
}
