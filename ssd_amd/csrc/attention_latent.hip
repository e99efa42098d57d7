// Latent attention over a paged cache, with a sliding window.  Queries and keys / values pass through low-rank latents:
//     c_q = rms(W_dq h) w_dq,  q = W_uq c_q   (per head [D unrotated | R rotated])
//     [c' | k_r] = W_dkv h,   c = rms(c') w_dkv (the latent, Cr wide),   k_r (R wide): ONE rotated key part for all heads
//     key_h = [W_uk,h c | rope(k_r)],  value_h = W_uv,h c
// Only [c | rope(k_r)] is cached per token (Cr + R numbers for every head together).  The attention runs in the latent space:
//     score(t, j, h) = scale * ( <W_uk,h^T q_unrot(t,h), c_j> + <rope(q_rot(t,h)), rope(k_r,j)> )
//     o_lat(t, h)    = gate(t,h) * sum_j softmax_j(score) c_j          over  0 <= p_t - p_j < window
// and the caller's per-head GEMMs map q_unrot -> W_uk^T q_unrot before and o_lat -> W_uv o_lat after: every head reads the same
// cached rows, which is what makes decoding cheap.
// Rotation: the first `rot_dims` of the R rotated entries turn, entry i pairing with i + rot_dims / 2, by angle p * f_i (fp32) with
// cos and sin scaled by `mag`; f and mag come from the host (they carry the YaRN frequency blend).
//  * ssd_latent_store  fp32 projection rows [dq | dkv | gate logits] -> c_q rows, the cache row of every token, sigmoid gates
//                      (no q norm weight: the first q_rank entries pass as they are -- queries without a latent; no gate_out: no gates)
//  * ssd_latent_attn   MFMA form below (bf16, aligned latent sizes), else the scalar fp32 form for any sizes and both element types: a wave owns a (token, head) row, a lane a key for the
//                      scores and latent columns for the weighted sum; keys in steps of 64 from the window's first key, so a row's
//                      arithmetic depends on its position alone (not on the portion or the batch it arrives in)
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }

// LDS written by some lanes of a wave and read by others: order the accesses (the hardware serves one wave's LDS operations in order)
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

// entry i (< R) of a rotated part x at position pos
template <typename F>
__device__ __forceinline__ float rope_entry(F x, int i, int R, int rot_dims, float pos, const float* __restrict__ freqs, float mag) {
  const int half = rot_dims >> 1;
  if (i >= rot_dims) return x(i);
  const int f = i < half ? i : i - half;
  const float ang = pos * freqs[f];
  const float c = cosf(ang) * mag, s = sinf(ang) * mag;
  return i < half ? x(i) * c - x(i + half) * s : x(i) * c + x(i - half) * s;
}

// grid = (tokens, column blocks): every workgroup of a token computes the row's statistics itself and takes a share of the columns.
template <typename T>
__global__ void __launch_bounds__(256)
latent_store_kernel(const float* __restrict__ proj, long ld, int Qr, int Cr, int R, int H, const T* __restrict__ wq,
                    const T* __restrict__ wkv, float eps, const int64_t* __restrict__ positions, const float* __restrict__ freqs,
                    float mag, int rot_dims, const int32_t* __restrict__ slots, T* __restrict__ cq_out, T* __restrict__ cache,
                    float* __restrict__ gate_out) {
  __shared__ float red[4];
  const size_t t = blockIdx.x;
  const int first = blockIdx.y * 256 + threadIdx.x, step = 256 * gridDim.y;
  const float* pr = proj + t * ld;
  const float* dq = pr;
  const float* dkv = pr + Qr;
  float sq = 0.f, sc = 0.f;
  if (wq)
    for (int i = threadIdx.x; i < Qr; i += 256) sq += dq[i] * dq[i];
  for (int i = threadIdx.x; i < Cr; i += 256) sc += dkv[i] * dkv[i];
  if (wq) sq = block_sum_256(sq, red);
  sc = block_sum_256(sc, red);
  const float rq = 1.0f / sqrtf(sq / (float)Qr + eps), rc = 1.0f / sqrtf(sc / (float)Cr + eps);
  if (wq) {
    for (int i = first; i < Qr; i += step) stf<T>(cq_out + t * Qr + i, dq[i] * rq * ldf<T>(wq + i));
  } else {                                            // queries that pass through no latent: the first Qr entries as they are
    for (int i = first; i < Qr; i += step) stf<T>(cq_out + t * Qr + i, dq[i]);
  }
  if (gate_out)
    for (int i = first; i < H; i += step) gate_out[t * H + i] = sigmoidf_(pr[Qr + Cr + R + i]);
  const int slot = slots[t];
  if (slot < 0) return;
  T* row = cache + (size_t)slot * (Cr + R);
  for (int i = first; i < Cr; i += step) stf<T>(row + i, dkv[i] * rc * ldf<T>(wkv + i));
  const float pos = (float)positions[t];
  const float* kr = dkv + Cr;
  for (int i = first; i < R; i += step)
    stf<T>(row + Cr + i, rope_entry([&](int j) { return kr[j]; }, i, R, rot_dims, pos, freqs, mag));
}

constexpr int LAT_MAXC = 16;       // latent columns per lane: Cr <= 64 * LAT_MAXC

template <typename T>
__global__ void __launch_bounds__(256)
latent_attn_kernel(const float* __restrict__ q_abs, const T* __restrict__ q_rows, const T* __restrict__ cache,
                   const float* __restrict__ gate, const int32_t* __restrict__ block_tables, int max_blocks,
                   const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_q, int q_per_seq, int B, int H, int D, int R,
                   int Cr, int block_size, int window, float scale, const float* __restrict__ freqs, float mag, int rot_dims,
                   T* __restrict__ out) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x, h = blockIdx.y * 4 + wave;
  const int KW = Cr + R;
  float* sq = lds + (size_t)wave * (KW + 128);      // [KW] the row's query in the latent space | rotated part
  float* sp = sq + KW;                              // [64] softmax weights of the current key step
  int* sj = reinterpret_cast<int*>(sp + 64);        // [64] their cache rows
  if (h >= H) return;                               // (whole waves; no block-wide barrier below)
  int b;
  if (cu_q) {
    int lo = 0, hi = B;                             // cu_q[lo] <= t < cu_q[hi]
    while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (cu_q[mid] <= t) lo = mid; else hi = mid; }
    b = lo;
  } else {
    b = t / q_per_seq;
  }
  const long p = positions[t];
  const float pos = (float)p;
  const long first = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  for (int i = lane; i < Cr; i += 64) sq[i] = q_abs[((size_t)t * H + h) * Cr + i];
  const T* qr = q_rows + ((size_t)t * H + h) * (D + R) + D;
  for (int i = lane; i < R; i += 64)
    sq[Cr + i] = rope_entry([&](int j) { return ldf<T>(qr + j); }, i, R, rot_dims, pos, freqs, mag);
  wave_sync();
  float m = -INFINITY, den = 0.f;
  float acc[LAT_MAXC];
#pragma unroll
  for (int c = 0; c < LAT_MAXC; ++c) acc[c] = 0.f;
  const int32_t* bt = block_tables + (size_t)b * max_blocks;
  for (long j0 = first; j0 <= p; j0 += 64) {
    const long j = j0 + lane;
    const bool valid = j <= p;
    int row = 0;
    float s = -INFINITY;
    if (valid) {
      row = bt[j / block_size] * block_size + (int)(j % block_size);
      const T* kp = cache + (size_t)row * KW;
      float d = 0.f;
      for (int i = 0; i < KW; ++i) d = fmaf(sq[i], ldf<T>(kp + i), d);
      s = d * scale;
    }
    const float mn = fmaxf(m, wave_max(s));
    const float pj = valid ? expf(s - mn) : 0.f;
    const float resc = m == -INFINITY ? 0.f : expf(m - mn);
    den = den * resc + wave_sum(pj);
    m = mn;
    wave_sync();
    sp[lane] = pj;
    sj[lane] = row;
    wave_sync();
    const int cnt = (int)((p - j0 + 1) < 64 ? (p - j0 + 1) : 64);
#pragma unroll
    for (int c = 0; c < LAT_MAXC; ++c) {
      const int col = lane + 64 * c;
      if (col < Cr) {
        float a = acc[c] * resc;
        for (int kk = 0; kk < cnt; ++kk) a = fmaf(sp[kk], ldf<T>(cache + (size_t)sj[kk] * KW + col), a);
        acc[c] = a;
      }
    }
  }
  const float g = (gate ? gate[(size_t)t * H + h] : 1.0f) / den;
#pragma unroll
  for (int c = 0; c < LAT_MAXC; ++c) {
    const int col = lane + 64 * c;
    if (col < Cr) stf<T>(out + ((size_t)t * H + h) * Cr + col, acc[c] * g);
  }
}


// ---------------------------------------------------------------------------------------------------------------------
// MFMA form (bf16; kv_rank % 32 == 0, rot % 32 == 0, kv_rank <= 512, kv_rank + rot <= 640).  A workgroup owns one token and 16 heads
// (rows of the score tile = heads: every head reads the SAME cached rows); its NW waves take the 32-key steps of the window round-robin
// and meet in LDS at the end.  Per step and wave:
//   S^T[key][head] = K tile x Q      K rows straight from the cache as the A operand (16-byte loads), Q fragments in registers;
//                                    the two 16-key tiles take the keys in the order (g*8 + r | g*8 + 4 + r), so that a lane ends up
//                                    with the scores of 8 CONSECUTIVE keys of its head -- already the B operand layout of the next product
//   online softmax per head          on the accumulator fragments (two cross-lane steps per reduction)
//   O^T[col][head] += C^T tile x P   the latent part of the K fragments is scattered into LDS transposed ([col][32 keys]) while S is
//                                    computed, so every cached element is loaded once and the A operand is one 16-byte LDS read
// Keys outside [first, p] are never loaded (zeros; -inf scores): unwritten cache rows cannot leak.  The steps start at the window's first
// key, so a row's arithmetic depends on its position alone.
// ---------------------------------------------------------------------------------------------------------------------
constexpr int LAT_KT_MAX = 20, LAT_NT_MAX = 32, LAT_CTS = 40;

template <int NW>
__global__ void __launch_bounds__(NW * 64)
latent_attn_mfma_kernel(const bf16_t* __restrict__ q_lat, const bf16_t* __restrict__ q_rows, const bf16_t* __restrict__ cache,
                        const float* __restrict__ gate, const int32_t* __restrict__ block_tables, int max_blocks,
                        const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_q, int q_per_seq, int B, int H, int D,
                        int R, int Cr, int block_size, int window, float scale, const float* __restrict__ freqs, float mag,
                        int rot_dims, bf16_t* __restrict__ out, int ksplit, float* __restrict__ ws) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, i = lane & 15, g = lane >> 4;
  const int t = blockIdx.x, ht = blockIdx.y;
  const int KW = Cr + R, KT = KW >> 5, CT_K = Cr >> 5, NT = Cr >> 4;
  bf16_t* ct = reinterpret_cast<bf16_t*>(smem) + (size_t)wave * Cr * LAT_CTS;
  int b;
  if (cu_q) {
    int lo = 0, hi = B;
    while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (cu_q[mid] <= t) lo = mid; else hi = mid; }
    b = lo;
  } else {
    b = t / q_per_seq;
  }
  const long p = positions[t];
  const float pos = (float)p;
  const long first = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int h = ht * 16 + i;
  const bool hv = h < H;
  // the head's query in the latent space | its rotated part, as B fragments: lane (head i, chunk g) holds k = kt * 32 + g * 8 .. + 7
  u32x4_t qf[LAT_KT_MAX];
  const bf16_t* ql = q_lat + ((size_t)t * H + (hv ? h : 0)) * Cr;
  const bf16_t* qr = q_rows + ((size_t)t * H + (hv ? h : 0)) * (D + R) + D;
#pragma unroll
  for (int kt = 0; kt < LAT_KT_MAX; ++kt) {
    qf[kt] = u32x4_t{0u, 0u, 0u, 0u};
    if (kt < KT && hv) {
      const int k = kt * 32 + g * 8;
      if (k < Cr) {
        qf[kt] = *reinterpret_cast<const u32x4_t*>(ql + k);
      } else {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = rope_entry([&](int j) { return bf2f(qr[j]); }, k - Cr + e, R, rot_dims, pos, freqs, mag);
        qf[kt] = u32x4_t{pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3]), pack_bf2(v[4], v[5]), pack_bf2(v[6], v[7])};
      }
    }
  }
  f32x4_t acc[LAT_NT_MAX];
#pragma unroll
  for (int nt = 0; nt < LAT_NT_MAX; ++nt) acc[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float mrun = -INFINITY, den = 0.f;
  const int32_t* bt = block_tables + (size_t)b * max_blocks;
  const int nsteps = (int)((p - first) >> 5) + 1;
  const int slot0 = (i >> 2) * 8 + (i & 3);            // key (within the step) of A row i in the first tile; the second tile: + 4
  for (int step = blockIdx.z * NW + wave; step < nsteps; step += NW * ksplit) {
    const long j0 = first + (long)step * 32;
    const long ja = j0 + slot0, jb = ja + 4;
    const bool va = ja <= p, vb = jb <= p;
    const bf16_t* ka = cache + (size_t)(va ? bt[ja / block_size] * block_size + (int)(ja % block_size) : 0) * KW + g * 8;
    const bf16_t* kb = cache + (size_t)(vb ? bt[jb / block_size] * block_size + (int)(jb % block_size) : 0) * KW + g * 8;
    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
    wave_sync();                                       // the previous step's readers of ct are done
#pragma unroll
    for (int kt = 0; kt < LAT_KT_MAX; ++kt) {
      if (kt < KT) {
        u32x4_t a0 = {0u, 0u, 0u, 0u}, a1 = {0u, 0u, 0u, 0u};
        if (va) a0 = *reinterpret_cast<const u32x4_t*>(ka + kt * 32);
        if (vb) a1 = *reinterpret_cast<const u32x4_t*>(kb + kt * 32);
        s0 = mfma16(a0, qf[kt], s0);
        s1 = mfma16(a1, qf[kt], s1);
        if (kt < CT_K) {
          bf16_t* c0 = ct + (size_t)(kt * 32 + g * 8) * LAT_CTS + slot0;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            c0[e * LAT_CTS] = (bf16_t)((a0[e >> 1] >> (16 * (e & 1))) & 0xffffu);
            c0[e * LAT_CTS + 4] = (bf16_t)((a1[e >> 1] >> (16 * (e & 1))) & 0xffffu);
          }
        }
      }
    }
    // lane (head i, g): keys j0 + g * 8 + 0 .. 7
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float raw = e < 4 ? s0[e] : s1[e - 4];
      sv[e] = (j0 + g * 8 + e <= p) ? raw * scale : -INFINITY;
      mx = fmaxf(mx, sv[e]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(mrun, mx);
    const float resc = mrun == -INFINITY ? 0.f : expf(mrun - mn);
    float ps = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) { sv[e] = sv[e] == -INFINITY ? 0.f : expf(sv[e] - mn); ps += sv[e]; }
    ps += __shfl_xor(ps, 16, 64);
    ps += __shfl_xor(ps, 32, 64);
    den = den * resc + ps;
    mrun = mn;
    const u32x4_t pb = {pack_bf2(sv[0], sv[1]), pack_bf2(sv[2], sv[3]), pack_bf2(sv[4], sv[5]), pack_bf2(sv[6], sv[7])};
    wave_sync();                                       // ct is complete
#pragma unroll
    for (int nt = 0; nt < LAT_NT_MAX; ++nt) {
      if (nt < NT) {
        const u32x4_t a = *reinterpret_cast<const u32x4_t*>(ct + (size_t)(nt * 16 + i) * LAT_CTS + g * 8);
        acc[nt] *= resc;
        acc[nt] = mfma16(a, pb, acc[nt]);
      }
    }
  }
  // the waves' partial rows meet in LDS (each wave's own region, reused): [col][head] fp32, then m and den per head
  wave_sync();
  float* part = reinterpret_cast<float*>(ct);
#pragma unroll
  for (int nt = 0; nt < LAT_NT_MAX; ++nt)
    if (nt < NT) {
#pragma unroll
      for (int r = 0; r < 4; ++r) part[(size_t)(nt * 16 + g * 4 + r) * 16 + i] = acc[nt][r];
    }
  if (g == 0) { part[(size_t)Cr * 16 + i] = mrun; part[(size_t)Cr * 16 + 16 + i] = den; }
  __syncthreads();
  const size_t wstride = (size_t)Cr * LAT_CTS / 2;      // floats per wave region
  const float* all = reinterpret_cast<const float*>(smem);
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < NW; ++w) M = fmaxf(M, all[w * wstride + (size_t)Cr * 16 + i]);
  float f[NW], Dn = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    const float mw = all[w * wstride + (size_t)Cr * 16 + i];
    f[w] = mw == -INFINITY ? 0.f : expf(mw - M);
    Dn += all[w * wstride + (size_t)Cr * 16 + 16 + i] * f[w];
  }
  if (ksplit > 1) {        // few rows: the window is cut over ksplit workgroups; this one's sums (relative to its M) go to the workspace
    float* u = ws + ((size_t)(t * gridDim.y + ht) * ksplit + blockIdx.z) * ((size_t)Cr * 16 + 32);
    if (wave == 0 && g == 0) { u[(size_t)Cr * 16 + i] = M; u[(size_t)Cr * 16 + 16 + i] = Dn; }
    for (int nt = wave; nt < NT; nt += NW)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float a = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) a += all[w * wstride + (size_t)(nt * 16 + g * 4 + r) * 16 + i] * f[w];
        u[(size_t)(nt * 16 + g * 4 + r) * 16 + i] = a;
      }
    return;
  }
  if (!hv) return;
  const float gsc = (gate ? gate[(size_t)t * H + h] : 1.0f) / Dn;
  for (int nt = wave; nt < NT; nt += NW) {
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float a = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) a += all[w * wstride + (size_t)(nt * 16 + g * 4 + r) * 16 + i] * f[w];
      v[r] = a * gsc;
    }
    uint2 o2;
    o2.x = pack_bf2(v[0], v[1]);
    o2.y = pack_bf2(v[2], v[3]);
    *reinterpret_cast<uint2*>(out + ((size_t)t * H + h) * Cr + nt * 16 + g * 4) = o2;
  }
}

// The key slices of a row meet: out = gate * sum_z vals_z e^(M_z - M) / sum_z den_z e^(M_z - M), slices in order.
__global__ void __launch_bounds__(256)
latent_attn_merge_kernel(const float* __restrict__ ws, const float* __restrict__ gate, int H, int Cr, int HT, int ksplit,
                         bf16_t* __restrict__ out) {
  // a workgroup: 16 latent columns x 16 heads of one (token, head tile); thread = one output element
  const int t = blockIdx.x / HT, ht = blockIdx.x % HT;
  const size_t unit = (size_t)Cr * 16 + 32;
  const float* u = ws + (size_t)blockIdx.x * ksplit * unit;
  const int idx = blockIdx.y * 256 + threadIdx.x, i = idx & 15, col = idx >> 4, h = ht * 16 + i;
  if (col >= Cr || h >= H) return;
  float M = -INFINITY;
  for (int z = 0; z < ksplit; ++z) M = fmaxf(M, u[z * unit + (size_t)Cr * 16 + i]);
  float Dn = 0.f, a = 0.f;
  for (int z = 0; z < ksplit; ++z) {
    const float mz = u[z * unit + (size_t)Cr * 16 + i];
    const float fz = mz == -INFINITY ? 0.f : expf(mz - M);
    Dn += u[z * unit + (size_t)Cr * 16 + 16 + i] * fz;
    a += u[z * unit + idx] * fz;
  }
  out[((size_t)t * H + h) * Cr + col] = (bf16_t)f2bf(a * ((gate ? gate[(size_t)t * H + h] : 1.0f) / Dn));
}

static inline bool latent_mfma_ok(int Cr, int R) {
  return Cr % 32 == 0 && R % 32 == 0 && Cr <= 16 * LAT_NT_MAX && Cr + R <= 32 * LAT_KT_MAX;
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_latent_store(const void* proj_rows, long ld, int q_rank, int kv_rank, int rot, int H, const void* q_norm_w,
                                const void* kv_norm_w, float eps, const int64_t* positions, const float* freqs, float mag,
                                int rot_dims, const int32_t* slots, void* cq_out, void* cache, void* gate_out, int T, int f32,
                                void* stream) {
  if (!proj_rows || !kv_norm_w || !positions || !freqs || !slots || !cq_out || !cache) return SSD_ERR_ARG;
  if (T <= 0 || q_rank <= 0 || kv_rank <= 0 || rot < 0 || H <= 0 || rot_dims < 0 || rot_dims > rot || (rot_dims & 1) ||
      ld < (long)q_rank + kv_rank + rot + (gate_out ? H : 0))
    return SSD_ERR_SHAPE;
  const int cols = q_rank > kv_rank ? q_rank : kv_rank;
  const dim3 grid(T, T >= 64 ? 1 : ((cols + 255) / 256 < 16 ? (cols + 255) / 256 : 16));
  if (f32)
    hipLaunchKernelGGL(latent_store_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)proj_rows, ld, q_rank,
                       kv_rank, rot, H, (const float*)q_norm_w, (const float*)kv_norm_w, eps, positions, freqs, mag, rot_dims, slots,
                       (float*)cq_out, (float*)cache, (float*)gate_out);
  else
    hipLaunchKernelGGL(latent_store_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)proj_rows, ld, q_rank,
                       kv_rank, rot, H, (const bf16_t*)q_norm_w, (const bf16_t*)kv_norm_w, eps, positions, freqs, mag, rot_dims, slots,
                       (bf16_t*)cq_out, (bf16_t*)cache, (float*)gate_out);
  return LAUNCH_OK();
}

extern "C" int ssd_latent_attn(const void* q_abs, const void* q_rows, const void* cache, const void* gate, const int32_t* block_tables,
                               int max_blocks, const int64_t* positions, const int32_t* cu_q, int q_per_seq, int B, int T, int H, int D,
                               int rot, int kv_rank, int block_size, int window, float scale, const float* freqs, float mag,
                               int rot_dims, void* out_rows, int f32, int q_abs_elem, void* workspace, long workspace_bytes,
                               void* stream) {
  if (!q_abs || !q_rows || !cache || !block_tables || !positions || !freqs || !out_rows) return SSD_ERR_ARG;
  if (B <= 0 || T <= 0 || H <= 0 || D <= 0 || rot < 0 || kv_rank <= 0 || kv_rank > 64 * LAT_MAXC || block_size <= 0 || max_blocks <= 0 ||
      rot_dims < 0 || rot_dims > rot || (rot_dims & 1) || (!cu_q && q_per_seq <= 0))
    return SSD_ERR_SHAPE;
  if (q_abs_elem) {        // q_abs holds element-type rows: the MFMA form
    if (f32 || !latent_mfma_ok(kv_rank, rot)) return SSD_ERR_SHAPE;
    const int HT = (H + 15) / 16, NWv = kv_rank <= 256 ? 4 : 2;
    // few rows (decoding): cut the window over up to 16 workgroups per (token, 16 heads) and merge; the cut depends on T alone
    int ksplit = 1;
    const long unit_bytes = ((long)kv_rank * 16 + 32) * (long)sizeof(float);
    if (workspace && (long)T * HT < 256) {
      const int steps = window > 0 ? (window + 31) / 32 + 1 : 64;
      ksplit = 512 / (T * HT);
      if (ksplit > (steps + NWv - 1) / NWv) ksplit = (steps + NWv - 1) / NWv;
      if (ksplit > 16) ksplit = 16;
      while (ksplit > 1 && (long)T * HT * ksplit * unit_bytes > workspace_bytes) --ksplit;
      if (ksplit < 1) ksplit = 1;
    }
    const dim3 mg(T, HT, ksplit);
    if (kv_rank <= 256) {
      const size_t mb = (size_t)4 * kv_rank * LAT_CTS * sizeof(bf16_t);
      if (mb > 64 * 1024 && hipFuncSetAttribute((const void*)latent_attn_mfma_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                (int)mb) != hipSuccess)
        return SSD_ERR_LAUNCH;
      hipLaunchKernelGGL(latent_attn_mfma_kernel<4>, mg, dim3(256), mb, (hipStream_t)stream, (const bf16_t*)q_abs, (const bf16_t*)q_rows,
                         (const bf16_t*)cache, (const float*)gate, block_tables, max_blocks, positions, cu_q, q_per_seq, B, H, D, rot,
                         kv_rank, block_size, window, scale, freqs, mag, rot_dims, (bf16_t*)out_rows, ksplit, (float*)workspace);
    } else {
      const size_t mb = (size_t)2 * kv_rank * LAT_CTS * sizeof(bf16_t);
      if (mb > 64 * 1024 && hipFuncSetAttribute((const void*)latent_attn_mfma_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                (int)mb) != hipSuccess)
        return SSD_ERR_LAUNCH;
      hipLaunchKernelGGL(latent_attn_mfma_kernel<2>, mg, dim3(128), mb, (hipStream_t)stream, (const bf16_t*)q_abs, (const bf16_t*)q_rows,
                         (const bf16_t*)cache, (const float*)gate, block_tables, max_blocks, positions, cu_q, q_per_seq, B, H, D, rot,
                         kv_rank, block_size, window, scale, freqs, mag, rot_dims, (bf16_t*)out_rows, ksplit, (float*)workspace);
    }
    if (ksplit > 1)
      hipLaunchKernelGGL(latent_attn_merge_kernel, dim3(T * HT, (kv_rank + 15) / 16), dim3(256), 0, (hipStream_t)stream,
                         (const float*)workspace, (const float*)gate, H, kv_rank, HT, ksplit, (bf16_t*)out_rows);
    return LAUNCH_OK();
  }
  const size_t bytes = (size_t)4 * (kv_rank + rot + 128) * sizeof(float);
  const dim3 grid(T, (H + 3) / 4);
  if (f32)
    hipLaunchKernelGGL(latent_attn_kernel<float>, grid, dim3(256), bytes, (hipStream_t)stream, (const float*)q_abs, (const float*)q_rows,
                       (const float*)cache, (const float*)gate, block_tables, max_blocks, positions, cu_q, q_per_seq, B, H, D, rot,
                       kv_rank, block_size, window, scale, freqs, mag, rot_dims, (float*)out_rows);
  else
    hipLaunchKernelGGL(latent_attn_kernel<bf16_t>, grid, dim3(256), bytes, (hipStream_t)stream, (const float*)q_abs,
                       (const bf16_t*)q_rows, (const bf16_t*)cache, (const float*)gate, block_tables, max_blocks, positions, cu_q,
                       q_per_seq, B, H, D, rot, kv_rank, block_size, window, scale, freqs, mag, rot_dims, (bf16_t*)out_rows);
  return LAUNCH_OK();
}

extern "C" int ssd_latent_attn_mfma_ok(int kv_rank, int rot, int f32) {
  if (kv_rank <= 0 || rot < 0) return SSD_ERR_SHAPE;
  return (!f32 && latent_mfma_ok(kv_rank, rot)) ? 1 : 0;
}
