// Row-major GEMM for ANY M, N, K, in bf16 (MFMA 16x16x32, fp32 accumulation) or in true fp32 (FMA), dense or grouped:
//   y[m][n] = sum_k x[row(m)][k] * w[g(m)][n][k]
// The skinny / prefill GEMMs of gemm.hip and gemm_pf.hip need fragment-major operands with N % 16 == 0 and K % 32 == 0; models whose
// sizes do not meet that, grouped (per-expert) products over gathered token rows, and the fp32 arithmetic mode use this kernel.
// Few token rows in bf16 take the skinny weight-streaming form below; otherwise a 256-thread workgroup owns a 64 x 64 output tile; a K step of 32 is staged through LDS with bounds guards (rows or columns past
// the edge read as zero), so no operand needs padding.  Wave w multiplies token rows 16w..16w+15 by the tile's four 16-feature
// groups.  Every output element is the sum over k in ascending 32-wide steps, whatever M, the tile or the group is: a row's result does not
// depend on which other rows share its launch.
//   grouped: offsets[E+1] cuts the (sorted) rows into E runs, run e multiplies by w + e * N * K; row_idx (optional) names the x row
//   of every sorted row as row_idx[r] / idx_div; tiles never straddle two runs (blockIdx.y walks a list of at most
//   ceil(rows / 64) + E tiles, found by a scan of offsets).
//   batched: G independent products in one launch (blockIdx.z / blockIdx.y = g): x + g * gsx with row stride ldx, w + g * N * K,
//   y + g * gsy with row stride ldy -- per-head products whose operands are column slices of token-major rows.
#include "common.h"

namespace {

constexpr int BM = 64, BN = 64, BK = 32;

template <typename T> struct Elem;
template <> struct Elem<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct Elem<bf16_t> {
  static __device__ __forceinline__ float ld(const bf16_t* p) { return bf2f(*p); }
  static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }
};

// Stage a [64][32] tile of `src` (row stride ld elements) into LDS (row stride LDT elements); rows >= nrows and columns >= K are zero.
// 16-byte loads when the row stride and base allow, element loads otherwise.
template <typename T, int LDT>
__device__ __forceinline__ void stage_tile(T* lds, const T* __restrict__ src, const int* __restrict__ rowmap, int idx_div, int row0,
                                           int nrows, int k0, int K, long ld, bool vec_ok) {
  constexpr int VEC = 16 / sizeof(T);            // elements per 16 bytes
  constexpr int CPR = BK / VEC;                  // chunks per row
  for (int c = threadIdx.x; c < 64 * CPR; c += 256) {
    const int r = c / CPR, kc = (c % CPR) * VEC;
    const int gr = row0 + r;
    T tmp[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) tmp[i] = T(0);
    if (gr < nrows) {
      const long srow = rowmap ? (long)(rowmap[gr] / idx_div) : (long)gr;
      const T* p = src + srow * ld + k0 + kc;
      if (vec_ok && k0 + kc + VEC <= K) {
        *reinterpret_cast<u32x4_t*>(tmp) = *reinterpret_cast<const u32x4_t*>(p);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i)
          if (k0 + kc + i < K) tmp[i] = p[i];
      }
    }
    *reinterpret_cast<u32x4_t*>(lds + r * LDT + kc) = *reinterpret_cast<u32x4_t*>(tmp);
  }
}

// epilogue 0: fp32 rows; 1: relu(v)^2 as element-type rows; 2: element-type rows; 5: tanh(v) as element-type rows (3, 4: see glu_act)
template <typename T>
__device__ __forceinline__ void store_out(void* y, long row, long ldy, long n, float v, int epi) {
  if (epi == 0) {
    reinterpret_cast<float*>(y)[row * ldy + n] = v;
  } else {
    if (epi == 1) { v = v > 0.f ? v : 0.f; v = v * v; }
    if (epi == 5) v = tanhf(v);
    Elem<T>::st(reinterpret_cast<T*>(y) + row * ldy + n, v);
  }
}

// epilogues 3 / 4 (bf16 forms only): the weight rows come in (gate, up) pairs -- row 2i = gate_i, row 2i + 1 = up_i -- and the output is
// act(gate) * up as element-type rows [M][N / 2], act = silu (3) or tanh-form gelu (4).  A lane's accumulators hold both halves of a pair.
// epilogue 6 (ssd_gemm_rows_grouped_glu_clamp): the clamped swish-GLU of experts whose routing weight multiplies their INPUT -- both
// halves of a pair are scaled by the row's factor s = row_scale[row_idx[m]] (the products are linear in it), then g = min(s z, limit),
// u = clamp(s u, -limit, limit), out = g sigmoid(alpha g) (u + 1).
struct GluClamp { const float* row_scale; float limit, alpha; };
__host__ __device__ __forceinline__ bool epi_pairs(int epi) { return epi == 3 || epi == 4 || epi == 6; }
__device__ __forceinline__ float glu_act(float z, float u, int epi, float s = 1.0f, float limit = 0.f, float alpha = 0.f) {
  if (epi == 6) {
    const float g = fminf(s * z, limit);
    return g / (1.0f + expf(-alpha * g)) * (fminf(fmaxf(s * u, -limit), limit) + 1.0f);
  }
  const float g = epi == 3 ? z / (1.0f + expf(-z)) : 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return g * u;
}

template <typename T>
__global__ void __launch_bounds__(256)
gemm_rows_kernel(const T* __restrict__ x, const T* __restrict__ w, void* __restrict__ y, int M, int N, int K, int epi,
                 const int* __restrict__ offsets, int E, const int* __restrict__ row_idx, int idx_div, bool vec_ok, long ldx, long ldy,
                 long gsx, long gsy, GluClamp gc) {
  constexpr int PAD = 16 / sizeof(T);
  constexpr int LDT = BK + PAD;
  __shared__ __attribute__((aligned(16))) T sx[BM * LDT];
  __shared__ __attribute__((aligned(16))) T sw[BN * LDT];
  int row0 = blockIdx.y * BM, row_end = M;
  const T* wg = w + (size_t)blockIdx.z * N * K;
  x += (size_t)blockIdx.z * gsx;
  const long ycol = (long)blockIdx.z * gsy;
  if (offsets) {           // grouped: find the run and the tile inside it that this workgroup owns
    int tile = blockIdx.y, e = 0;
    for (; e < E; ++e) {
      const int cnt = offsets[e + 1] - offsets[e];
      const int nt = (cnt + BM - 1) / BM;
      if (tile < nt) break;
      tile -= nt;
    }
    if (e >= E) return;
    row0 = offsets[e] + tile * BM;
    row_end = offsets[e + 1];
    wg = w + (size_t)e * N * K;
  }
  const int n0 = blockIdx.x * BN;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;

  if constexpr (sizeof(T) == 2) {
    f32x4_t acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += BK) {
      stage_tile<T, LDT>(sx, x, row_idx, idx_div, row0, row_end, k0, K, ldx, vec_ok);
      stage_tile<T, LDT>(sw, wg, nullptr, 1, n0, N, k0, K, K, vec_ok);
      __syncthreads();
      const u32x4_t b = *reinterpret_cast<const u32x4_t*>(sx + (wave * 16 + (lane & 15)) * LDT + (lane >> 4) * 8);
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const u32x4_t a = *reinterpret_cast<const u32x4_t*>(sw + (nt * 16 + (lane & 15)) * LDT + (lane >> 4) * 8);
        acc[nt] = mfma16(a, b, acc[nt]);
      }
      __syncthreads();
    }
    const int m = row0 + wave * 16 + (lane & 15);
    if (m < row_end && epi_pairs(epi)) {
      const float rs = epi == 6 && gc.row_scale ? gc.row_scale[row_idx ? row_idx[m] : m] : 1.0f;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int r = 0; r < 4; r += 2) {
          const int n = n0 + nt * 16 + (lane >> 4) * 4 + r;
          if (n + 1 < N)
            Elem<T>::st(reinterpret_cast<T*>(y) + (long)m * ldy + ycol + (n >> 1),
                        glu_act(acc[nt][r], acc[nt][r + 1], epi, rs, gc.limit, gc.alpha));
        }
    } else if (m < row_end) {
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int n = n0 + nt * 16 + (lane >> 4) * 4 + r;
          if (n < N) store_out<T>(y, m, ldy, ycol + n, acc[nt][r], epi);
        }
    }
  } else {
    // fp32: thread (tm, tn) owns token rows tm*4..+3 and features tn*4..+3 of the tile; plain FMA chains in ascending k
    const int tm = threadIdx.x >> 4, tn = threadIdx.x & 15;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < K; k0 += BK) {
      stage_tile<T, LDT>(sx, x, row_idx, idx_div, row0, row_end, k0, K, ldx, vec_ok);
      stage_tile<T, LDT>(sw, wg, nullptr, 1, n0, N, k0, K, K, vec_ok);
      __syncthreads();
#pragma unroll 8
      for (int k = 0; k < BK; ++k) {
        float a[4], b[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = (float)sx[(tm * 4 + i) * LDT + k];
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = (float)sw[(tn + 16 * j) * LDT + k];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
      }
      __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = row0 + tm * 4 + i;
      if (m >= row_end) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + tn + 16 * j;
        if (n < N) store_out<T>(y, m, ldy, ycol + n, acc[i][j], epi);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// Skinny form (bf16, K % 8 == 0, few token rows: decoding): a weight-streaming product.  A workgroup owns 16 features; its NW waves take
// the 32-wide k-tiles round-robin in runs of U, so the workgroup as a whole walks its 16 weight rows linearly; both MFMA operands are
// 16-byte loads straight from the row-major matrices (lane = (row & 15) + 16 * (k chunk)); the waves' partial tiles are summed through
// LDS in wave order.  Grouped: blockIdx.y is the group; a group with no rows exits at once, one with more than 16 rows loops over
// 16-row chunks.
// ---------------------------------------------------------------------------------------------------------------------
template <int NW>
__global__ void __launch_bounds__(NW * 64)
gemm_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ y, int M, int N, int K, int epi,
                   const int* __restrict__ offsets, const int* __restrict__ row_idx, int idx_div, long ldx, long ldy, long gsx,
                   long gsy, GluClamp gc) {
  constexpr int U = 8;
  __shared__ f32x4_t red[NW * 64];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, qd = lane >> 4;
  const int n0 = blockIdx.x * 16;
  int m_begin = 0, m_end = M;
  const bf16_t* wg = w;
  long ycol = 0;
  if (!offsets) {          // batched (or a single product: blockIdx.y == 0)
    wg = w + (size_t)blockIdx.y * N * K;
    x += (size_t)blockIdx.y * gsx;
    ycol = (long)blockIdx.y * gsy;
  }
  if (offsets) {
    m_begin = offsets[blockIdx.y];
    m_end = offsets[blockIdx.y + 1];
    if (m_begin >= m_end) return;
    wg = w + (size_t)blockIdx.y * N * K;
  }
  const int nrow = min(n0 + r, N - 1);
  const bf16_t* wp = wg + (size_t)nrow * K + qd * 8;
  const int KT = (K + 31) >> 5;
  for (int m0 = m_begin; m0 < m_end; m0 += 16) {
    const int mrow = m0 + r;
    const bool mvalid = mrow < m_end;
    const long xrow = mvalid ? (row_idx ? (long)(row_idx[mrow] / idx_div) : (long)mrow) : 0;
    const bf16_t* xp = x + xrow * ldx + qd * 8;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int kt0 = wave * U; kt0 < KT; kt0 += NW * U) {
      u32x4_t a[U], b[U];
#pragma unroll
      for (int i = 0; i < U; ++i) {
        const int kt = kt0 + i;
        const bool ok = kt < KT && kt * 32 + qd * 8 < K;
        a[i] = u32x4_t{0u, 0u, 0u, 0u};
        b[i] = u32x4_t{0u, 0u, 0u, 0u};
        if (ok) a[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(wp + kt * 32));
        if (ok && mvalid) b[i] = *reinterpret_cast<const u32x4_t*>(xp + kt * 32);
      }
#pragma unroll
      for (int i = 0; i < U; ++i) acc = mfma16(a[i], b[i], acc);
    }
    red[wave * 64 + lane] = acc;
    __syncthreads();
    if (wave == 0) {
      f32x4_t sum = red[lane];
#pragma unroll
      for (int wv = 1; wv < NW; ++wv) sum += red[wv * 64 + lane];
      if (mvalid && epi_pairs(epi)) {
        const float rs = epi == 6 && gc.row_scale ? gc.row_scale[row_idx ? row_idx[mrow] : mrow] : 1.0f;
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
          const int n = n0 + qd * 4 + e;
          if (n + 1 < N)
            reinterpret_cast<bf16_t*>(y)[(long)mrow * ldy + ycol + (n >> 1)] =
                (bf16_t)f2bf(glu_act(sum[e], sum[e + 1], epi, rs, gc.limit, gc.alpha));
        }
      } else if (mvalid) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int n = n0 + qd * 4 + e;
          if (n < N) store_out<bf16_t>(y, mrow, ldy, ycol + n, sum[e], epi);
        }
      }
    }
    __syncthreads();
  }
}

constexpr int SKINNY_MAX_ROWS = 16, SKINNY_MAX_GROUPED_ROWS = 64;

int launch(const void* x, const void* w, void* y, int M, int N, int K, int epi, const int* offsets, int E, const int* row_idx,
           int idx_div, int f32, void* stream, int G = 1, long ldx = 0, long gsx = 0, long ldy = 0, long gsy = 0,
           GluClamp gc = GluClamp{nullptr, 0.f, 0.f}) {
  if (!x || !w || !y) return SSD_ERR_ARG;
  if (M <= 0 || N <= 0 || K <= 0 || epi < 0 || epi > 6) return SSD_ERR_SHAPE;
  if (epi_pairs(epi) && (f32 || (N & 1))) return SSD_ERR_SHAPE;        // the paired epilogues exist in the bf16 forms only
  if (offsets && E <= 0) return SSD_ERR_SHAPE;
  if (G < 1 || G > 65535 || (G > 1 && offsets)) return SSD_ERR_SHAPE;
  if (ldx == 0) ldx = K;
  if (ldy == 0) ldy = epi_pairs(epi) ? N / 2 : N;
  if (ldx < K || ldy < (epi_pairs(epi) ? N / 2 : N)) return SSD_ERR_SHAPE;
  const int esz0 = f32 ? 4 : 2;
  const bool x_vec = ((size_t)ldx * esz0) % 16 == 0 && ((size_t)gsx * esz0) % 16 == 0 && (uintptr_t)x % 16 == 0;
  if (!f32 && K % 8 == 0 && x_vec && (uintptr_t)w % 16 == 0 &&
      M <= (offsets ? SKINNY_MAX_GROUPED_ROWS : SKINNY_MAX_ROWS)) {
    const int groups = (N + 15) / 16;
    const dim3 sg(groups, offsets ? E : G);
    const int id = idx_div < 1 ? 1 : idx_div;
    const long wgs = (long)groups * (offsets ? (M < E ? M : E) : G);          // workgroups that have rows
    // few workgroups: more waves each (a CU pulls from HBM what its waves have in flight), as long as every wave gets k-tiles
    const int kt = (K + 31) / 32;
    if (wgs < 256 && kt >= 64)
      hipLaunchKernelGGL(gemm_skinny_kernel<16>, sg, dim3(1024), 0, (hipStream_t)stream, (const bf16_t*)x, (const bf16_t*)w, y, M, N, K,
                         epi, offsets, row_idx, id, ldx, ldy, gsx, gsy, gc);
    else if (wgs < 1024 && kt >= 32)
      hipLaunchKernelGGL(gemm_skinny_kernel<8>, sg, dim3(512), 0, (hipStream_t)stream, (const bf16_t*)x, (const bf16_t*)w, y, M, N, K,
                         epi, offsets, row_idx, id, ldx, ldy, gsx, gsy, gc);
    else
      hipLaunchKernelGGL(gemm_skinny_kernel<4>, sg, dim3(256), 0, (hipStream_t)stream, (const bf16_t*)x, (const bf16_t*)w, y, M, N, K,
                         epi, offsets, row_idx, id, ldx, ldy, gsx, gsy, gc);
    return hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH;
  }
  const int tiles_m = (M + BM - 1) / BM + (offsets ? E : 0);
  const dim3 grid((N + BN - 1) / BN, tiles_m, G);
  const int esz = f32 ? 4 : 2;
  const bool vec_ok = ((size_t)K * esz) % 16 == 0 && x_vec && ((uintptr_t)w % 16 == 0);
  if (f32)
    hipLaunchKernelGGL(gemm_rows_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)x, (const float*)w, y, M, N, K,
                       epi, offsets, E, row_idx, idx_div < 1 ? 1 : idx_div, vec_ok, ldx, ldy, gsx, gsy, gc);
  else
    hipLaunchKernelGGL(gemm_rows_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const bf16_t*)x, (const bf16_t*)w, y, M, N,
                       K, epi, offsets, E, row_idx, idx_div < 1 ? 1 : idx_div, vec_ok, ldx, ldy, gsx, gsy, gc);
  return hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH;
}

}  // namespace

extern "C" int ssd_gemm_rows(const void* x_rows, const void* w_rows, void* y, int M, int N, int K, int epilogue, int f32,
                             void* stream) {
  return launch(x_rows, w_rows, y, M, N, K, epilogue, nullptr, 0, nullptr, 1, f32, stream);
}

extern "C" int ssd_gemm_rows_grouped(const void* x_rows, const void* w_rows, void* y, const int32_t* offsets, int E,
                                     const int32_t* row_idx, int idx_div, int rows, int N, int K, int epilogue, int f32,
                                     void* stream) {
  if (!offsets) return SSD_ERR_ARG;
  return launch(x_rows, w_rows, y, rows, N, K, epilogue, offsets, E, row_idx, idx_div, f32, stream);
}

extern "C" int ssd_gemm_rows_grouped_glu_clamp(const void* x_rows, const void* w_rows, void* y, const int32_t* offsets, int E,
                                               const int32_t* row_idx, int idx_div, int rows, int N, int K, const float* row_scale,
                                               float limit, float alpha, void* stream) {
  if (!offsets) return SSD_ERR_ARG;
  if (!(limit > 0.f)) return SSD_ERR_SHAPE;
  return launch(x_rows, w_rows, y, rows, N, K, 6, offsets, E, row_idx, idx_div, 0, stream, 1, 0, 0, 0, 0, GluClamp{row_scale, limit, alpha});
}

extern "C" int ssd_gemm_rows_glu_clamp(const void* x_rows, const void* w_rows, void* y, int M, int N, int K, float limit, float alpha,
                                       void* stream) {
  if (!(limit > 0.f)) return SSD_ERR_SHAPE;
  return launch(x_rows, w_rows, y, M, N, K, 6, nullptr, 0, nullptr, 1, 0, stream, 1, 0, 0, 0, 0, GluClamp{nullptr, limit, alpha});
}

extern "C" int ssd_gemm_rows_batched(const void* x_rows, const void* w_rows, void* y, int M, int N, int K, int G, long ldx, long gsx,
                                     long ldy, long gsy, int epilogue, int f32, void* stream) {
  if (ldx <= 0 || ldy <= 0 || gsx < 0 || gsy < 0) return SSD_ERR_SHAPE;
  return launch(x_rows, w_rows, y, M, N, K, epilogue, nullptr, 0, nullptr, 1, f32, stream, G, ldx, gsx, ldy, gsy);
}
