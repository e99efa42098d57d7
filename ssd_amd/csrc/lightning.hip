// Linear attention with a per-head scalar decay over a recurrent fp32 state ("lightning" mixers):
//     S_t = decay_h * S_(t-1) + k_t v_t^T        (S: [D][Dv] per sequence and head, zero before position 0)
//     o_t = S_t^T q_t
// q, k, v = silu of the projection rows (act 0), or the rows as they are (act 1: a mixer that prepared them itself, e.g. rotated q / k
// of a retention layer).  The state of a live sequence sits in a slot of a per-layer-run pool
// state[slots][H][D][Dv] (fp32); a forward reads the slot unless the rows it brings start at position 0, walks its rows in order and
// writes the slot back, so a prompt may arrive in portions of any size and decoding is the one-row case of the same kernel.
//  * ssd_lightning_scan       proj rows fp32 [T][ld] holding [q | k | v | ...] -> o fp32 [T][H*Dv], state updated in place
//  * ssd_lightning_gate_norm  out = w * o / sqrt(mean(o^2) + eps) * sigmoid(g) over the concatenated heads, as GEMM-input rows
// Two forms: state in registers (usual head sizes; below) and state in LDS (any sizes).
// The arithmetic of a row is the same whatever the portion: per state element one multiply-add chain in token order, the output a sum
// over d in a fixed order -- whole prompt, portions and token-by-token decoding give bit-identical rows.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float siluf_(float z) { return z * sigmoidf_(z); }

// One workgroup per (sequence, head).  Threads form NG groups of EP lanes (EP = power of two >= min(Dv, 256)): lane e of group g owns
// the state elements (d, e) with d = g, g + NG, ...; the groups' partial outputs meet in LDS and are summed in group order.
__global__ void __launch_bounds__(256)
lightning_scan_kernel(const float* __restrict__ proj, long ld, int q_off, int k_off, int v_off, const float* __restrict__ decay,
                      const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_q, int q_per_seq,
                      const int32_t* __restrict__ state_slots, float* __restrict__ state, float* __restrict__ out, int H, int D, int Dv,
                      int EP, int raw) {
  extern __shared__ float lds[];
  float* S = lds;                         // [D][Dv]
  float* sq = S + (size_t)D * Dv;         // [D]
  float* sk = sq + D;                     // [D]
  float* sv = sk + D;                     // [Dv]
  float* po = sv + Dv;                    // [NG][Dv]
  const int b = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int row0 = cu_q ? cu_q[b] : b * q_per_seq;
  const int row1 = cu_q ? cu_q[b + 1] : (b + 1) * q_per_seq;
  if (row1 <= row0) return;
  const int slot = state_slots[b];
  float* sp = state + ((size_t)slot * H + h) * D * Dv;
  const bool fresh = positions[row0] == 0;
  for (int i = tid; i < D * Dv; i += 256) S[i] = fresh ? 0.f : sp[i];
  const float dc = decay[h];
  const int NG = 256 / EP, g = tid / EP, el = tid % EP;
  for (int r = row0; r < row1; ++r) {
    const float* pr = proj + (size_t)r * ld;
    __syncthreads();                      // the previous row's readers of sq / sk / sv / po are done; S is loaded
    for (int i = tid; i < D; i += 256) {
      const float qv = pr[q_off + h * D + i], kv = pr[k_off + h * D + i];
      sq[i] = raw ? qv : siluf_(qv);
      sk[i] = raw ? kv : siluf_(kv);
    }
    for (int i = tid; i < Dv; i += 256) { const float vv = pr[v_off + h * Dv + i]; sv[i] = raw ? vv : siluf_(vv); }
    __syncthreads();
    for (int e = el; e < Dv; e += EP) {
      const float ve = sv[e];
      float o = 0.f;
      for (int d = g; d < D; d += NG) {
        const float s = fmaf(dc, S[d * Dv + e], sk[d] * ve);
        S[d * Dv + e] = s;
        o = fmaf(s, sq[d], o);
      }
      po[g * Dv + e] = o;
    }
    __syncthreads();
    for (int e = tid; e < Dv; e += 256) {
      float o = 0.f;
      for (int gg = 0; gg < NG; ++gg) o += po[gg * Dv + e];
      out[(size_t)r * H * Dv + h * Dv + e] = o;
    }
  }
  __syncthreads();
  for (int i = tid; i < D * Dv; i += 256) sp[i] = S[i];
}

// Register form (D = 8 * EPT with EPT in {4, 8, 16, 32}, Dv % 32 == 0): a workgroup owns 32 state columns of one (sequence, head) --
// grid.z walks the column blocks -- and thread (g, e) keeps the EPT elements (d = g + 8 n, column e) in registers.  Rows are staged
// eight at a time (silu applied once), every thread then walks the eight tokens without a barrier (it touches only its own state and
// the staged rows), and the eight d-groups' partial outputs are summed in group order.  The arithmetic of a row is the same for any
// portioning: the per-element chain in token order, the output sum over n ascending, then over g ascending.
template <int EPT, bool RAW>
__global__ void __launch_bounds__(256)
lightning_scan_reg_kernel(const float* __restrict__ proj, long ld, int q_off, int k_off, int v_off, const float* __restrict__ decay,
                          const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_q, int q_per_seq,
                          const int32_t* __restrict__ state_slots, float* __restrict__ state, float* __restrict__ out, int H, int Dv) {
  constexpr int TB = 8, NG = 8, CB = 32, D = NG * EPT;
  __shared__ float sq[TB][D], sk[TB][D];
  __shared__ float sv[TB][CB];
  __shared__ float po[TB][NG][CB];
  const int b = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * CB, tid = threadIdx.x;
  const int g = tid >> 5, e = tid & 31;
  const int row0 = cu_q ? cu_q[b] : b * q_per_seq;
  const int row1 = cu_q ? cu_q[b + 1] : (b + 1) * q_per_seq;
  if (row1 <= row0) return;
  float* sp = state + ((size_t)state_slots[b] * H + h) * D * Dv + c0 + e;
  const bool fresh = positions[row0] == 0;
  float S[EPT];
#pragma unroll
  for (int n = 0; n < EPT; ++n) S[n] = fresh ? 0.f : sp[(size_t)(g + NG * n) * Dv];
  const float dc = decay[h];
  // raw projection values of the next batch travel in registers while the current batch is computed (a batch is short: without
  // this every batch would wait a full memory round trip)
  constexpr int QK = TB * D / 256;         // q / k elements of a batch per thread
  float rq[QK], rk[QK], rv = 0.f;
  auto fetch = [&](int r) {
    const int nb = row1 - r < TB ? row1 - r : TB;
#pragma unroll
    for (int c = 0; c < QK; ++c) {
      const int idx = tid + 256 * c, tt = idx / D, d = idx % D;
      rq[c] = rk[c] = 0.f;
      if (tt < nb) {
        const float* pr = proj + (size_t)(r + tt) * ld + h * D + d;
        rq[c] = pr[q_off];
        rk[c] = pr[k_off];
      }
    }
    rv = g < nb ? proj[(size_t)(r + g) * ld + v_off + h * Dv + c0 + e] : 0.f;
  };
  fetch(row0);
  for (int r = row0; r < row1; r += TB) {
    const int nb = row1 - r < TB ? row1 - r : TB;
    __syncthreads();                      // the previous batch's readers are done
#pragma unroll
    for (int c = 0; c < QK; ++c) {
      const int idx = tid + 256 * c;
      sq[idx / D][idx % D] = RAW ? rq[c] : siluf_(rq[c]);
      sk[idx / D][idx % D] = RAW ? rk[c] : siluf_(rk[c]);
    }
    sv[g][e] = RAW ? rv : siluf_(rv);
    __syncthreads();
    if (r + TB < row1) fetch(r + TB);
    for (int tt = 0; tt < nb; ++tt) {
      const float ve = sv[tt][e];
      float o = 0.f;
#pragma unroll
      for (int n = 0; n < EPT; ++n) {
        const int d = g + NG * n;
        const float s = fmaf(dc, S[n], sk[tt][d] * ve);
        S[n] = s;
        o = fmaf(s, sq[tt][d], o);
      }
      po[tt][g][e] = o;
    }
    __syncthreads();
    if (g < nb) {                         // thread (g, e) now finishes token g of the batch
      float o = 0.f;
#pragma unroll
      for (int gg = 0; gg < NG; ++gg) o += po[g][gg][e];
      out[(size_t)(r + g) * H * Dv + h * Dv + c0 + e] = o;
    }
  }
#pragma unroll
  for (int n = 0; n < EPT; ++n) sp[(size_t)(g + NG * n) * Dv] = S[n];
}

template <typename T>
__global__ void __launch_bounds__(256)
lightning_gate_norm_kernel(const float* __restrict__ o, const float* __restrict__ proj, long ld, int g_off, const T* __restrict__ w,
                           float eps, T* __restrict__ out, int N) {
  __shared__ float red[4];
  const size_t t = blockIdx.x;
  const float* orow = o + t * N;
  float ss = 0.f;
  for (int c = threadIdx.x; c < N; c += 256) { const float v = orow[c]; ss += v * v; }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  ss = (red[0] + red[1]) + (red[2] + red[3]);
  const float r = 1.0f / sqrtf(ss / (float)N + eps);
  const float* gr = proj + t * ld + g_off;
  for (int c = threadIdx.x; c < N; c += 256) stf<T>(out + t * N + c, orow[c] * r * ldf<T>(w + c) * sigmoidf_(gr[c]));
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_lightning_scan(const void* proj_rows, long ld, int q_off, int k_off, int v_off, const float* decay,
                                  const int64_t* positions, const int32_t* cu_q, int q_per_seq, const int32_t* state_slots,
                                  void* state, void* out_rows, int B, int H, int D, int Dv, int act, void* stream) {
  if (!proj_rows || !decay || !positions || !state_slots || !state || !out_rows) return SSD_ERR_ARG;
  if (B <= 0 || H <= 0 || D <= 0 || Dv <= 0 || (!cu_q && q_per_seq <= 0) || act < 0 || act > 1) return SSD_ERR_SHAPE;
  if (Dv % 32 == 0 && Dv / 32 <= 65535 && (D == 32 || D == 64 || D == 128 || D == 256)) {
    const dim3 grid(B, H, Dv / 32);
#define SCAN_REG1(EPT, RAW)                                                                                                        \
  hipLaunchKernelGGL((lightning_scan_reg_kernel<EPT, RAW>), grid, dim3(256), 0, (hipStream_t)stream, (const float*)proj_rows, ld,  \
                     q_off, k_off, v_off, decay, positions, cu_q, q_per_seq, state_slots, (float*)state, (float*)out_rows, H, Dv)
#define SCAN_REG(EPT)                                                                                                              \
  do { if (act) SCAN_REG1(EPT, true); else SCAN_REG1(EPT, false); } while (0)
    if (D == 32) SCAN_REG(4);
    else if (D == 64) SCAN_REG(8);
    else if (D == 128) SCAN_REG(16);
    else SCAN_REG(32);
#undef SCAN_REG
#undef SCAN_REG1
    return LAUNCH_OK();
  }
  int EP = 1;
  while (EP < Dv && EP < 256) EP <<= 1;
  const size_t bytes = ((size_t)D * Dv + 2 * (size_t)D + Dv + (size_t)(256 / EP) * Dv) * sizeof(float);
  if (bytes > 160 * 1024) return SSD_ERR_SHAPE;
  if (bytes > 64 * 1024 &&
      hipFuncSetAttribute((const void*)lightning_scan_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess)
    return SSD_ERR_LAUNCH;
  hipLaunchKernelGGL(lightning_scan_kernel, dim3(B, H), dim3(256), bytes, (hipStream_t)stream, (const float*)proj_rows, ld, q_off, k_off,
                     v_off, decay, positions, cu_q, q_per_seq, state_slots, (float*)state, (float*)out_rows, H, D, Dv, EP, act);
  return LAUNCH_OK();
}

extern "C" int ssd_lightning_gate_norm(const void* o_rows, const void* proj_rows, long ld, int g_off, const void* weight, float eps,
                                       void* out_rows, int T, int N, int f32, void* stream) {
  if (!o_rows || !proj_rows || !weight || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || N <= 0) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(lightning_gate_norm_kernel<float>, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)o_rows,
                       (const float*)proj_rows, ld, g_off, (const float*)weight, eps, (float*)out_rows, N);
  else
    hipLaunchKernelGGL(lightning_gate_norm_kernel<bf16_t>, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)o_rows,
                       (const float*)proj_rows, ld, g_off, (const bf16_t*)weight, eps, (bf16_t*)out_rows, N);
  return LAUNCH_OK();
}
