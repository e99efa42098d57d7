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
//                         MFMA form (bf16, D % 32 == 0, D <= 256, Dv % 16 == 0, Dv <= 256, block_size % 32 == 0; the caller gives
//                         max_q, an upper bound of the rows a sequence brings): see below.
//   * ssd_winattn_store_rope  the store of a rotary variant: RMS norm with weights over the WHOLE q and the whole k projection (before
//                         the heads are split), rotary positions on the first rot_dims entries of every q / k head, and (v_freqs given)
//                         every value head turned by its own position over all Dv entries before it is cached; the attention then
//                         turns every head's output back by the query's position (out_freqs), so that the weighted sum carries
//                         relative positions.  Pairs are (i, i + n / 2) throughout.
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

// q' = w_q * q / rms(q) over all H * D entries (k alike over G * D), then per head the pair (i, i + half) turns by pos * qk_freqs[i];
// v heads turn over all Dv entries by pos * v_freqs[i] (v_freqs NULL: stored as they are).  grid = (tokens, column blocks): every
// workgroup of a token sums the squares of the whole row itself (a few thousand cached floats) and takes a share of the work items --
// a pair that turns (one sine and cosine for both entries) or a single entry that does not.
template <typename T>
__global__ void __launch_bounds__(256)
winattn_store_rope_kernel(const float* __restrict__ qkv, long ld, const T* __restrict__ wq, const T* __restrict__ wk, float eps,
                          const int64_t* __restrict__ positions, const float* __restrict__ qk_freqs, int rot_dims,
                          const float* __restrict__ v_freqs, const int32_t* __restrict__ slots, T* __restrict__ q_out,
                          T* __restrict__ kc, T* __restrict__ vc, int H, int G, int D, int Dv, int bs) {
  __shared__ float red[8];
  const int t = blockIdx.x;
  const int Nq = H * D, Nk = G * D;
  const float* row = qkv + (size_t)t * ld;
  const float pos = (float)positions[t];
  const int slot = slots[t];
  const long blk = slot >= 0 ? slot / bs : 0;
  const int off = slot >= 0 ? slot % bs : 0;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < Nq; i += 256) { const float v = row[i]; sq += v * v; }
  for (int i = threadIdx.x; i < Nk; i += 256) { const float v = row[Nq + i]; sk += v * v; }
  sq = wave_sum(sq);                                       // both statistics through one pair of barriers
  sk = wave_sum(sk);
  if ((threadIdx.x & 63) == 0) { red[threadIdx.x >> 6] = sq; red[4 + (threadIdx.x >> 6)] = sk; }
  __syncthreads();
  sq = (red[0] + red[1]) + (red[2] + red[3]);
  sk = (red[4] + red[5]) + (red[6] + red[7]);
  const float rq = 1.0f / sqrtf(sq / (float)Nq + eps), rk = 1.0f / sqrtf(sk / (float)Nk + eps);
  const int half = rot_dims >> 1, per = D - half;          // items of a q / k head: `half` pairs, then the entries that do not turn
  const int hv = Dv >> 1, perv = v_freqs ? hv : Dv;        // items of a v head
  const int n_qk = (H + G) * per, n_all = n_qk + (slot >= 0 ? G * perv : 0);
  for (int u = blockIdx.y * 256 + threadIdx.x; u < n_all; u += 256 * gridDim.y) {
    if (u < n_qk) {
      const int hd = u / per, i = u % per;
      const bool isq = hd < H;
      if (!isq && slot < 0) continue;
      const int base = hd * D;                             // k heads follow the q heads in the row, and their weights in wk
      const T* w = isq ? wq + base : wk + (base - Nq);
      const float r = isq ? rq : rk;
      T* dst = isq ? q_out + (size_t)t * Nq + base : kc + (((size_t)blk * G + (hd - H)) * bs + off) * D;
      if (i < half) {
        const float a = row[base + i] * r * ldf<T>(w + i), b = row[base + i + half] * r * ldf<T>(w + i + half);
        float sn, c;
        sincosf(pos * qk_freqs[i], &sn, &c);
        stf<T>(dst + i, a * c - b * sn);
        stf<T>(dst + i + half, b * c + a * sn);
      } else {
        stf<T>(dst + i + half, row[base + i + half] * r * ldf<T>(w + i + half));
      }
    } else {
      const int g = (u - n_qk) / perv, i = (u - n_qk) % perv;
      const float* src = row + Nq + Nk + g * Dv;
      T* dst = vc + (((size_t)blk * G + g) * Dv) * bs + off;
      if (v_freqs) {
        const float a = src[i], b = src[i + hv];
        float sn, c;
        sincosf(pos * v_freqs[i], &sn, &c);
        stf<T>(dst + (size_t)i * bs, a * c - b * sn);
        stf<T>(dst + (size_t)(i + hv) * bs, b * c + a * sn);
      } else {
        stf<T>(dst + (size_t)i * bs, src[i]);
      }
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
                     int Dv, int bs, int window, float scale, float cap, const float* __restrict__ out_freqs, T* __restrict__ out) {
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
  const int hv = Dv >> 1;
  for (int d = threadIdx.x; d < Dv; d += 256) {
    float s = 0.f;
    for (int w = 0; w < 4; ++w) s += sacc[w * Dv + d] * f[w];
    s = s / L;
    if (out_freqs) {                  // the head's output turns back by the query's position: pair (m, m + Dv / 2) by -pos * freq[m]
      const int dp = d < hv ? d + hv : d - hv;
      float o = 0.f;
      for (int w = 0; w < 4; ++w) o += sacc[w * Dv + dp] * f[w];
      o = o / L;
      float sn, c;
      sincosf((float)pos * out_freqs[d < hv ? d : d - hv], &sn, &c);
      s = d < hv ? s * c + o * sn : s * c - o * sn;
    }
    stf<T>(out + ((size_t)t * H + h) * Dv + d, s);
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// MFMA form (bf16, D % 32 == 0, D <= 256, Dv % 16 == 0, Dv <= 256, block_size % 32 == 0).  For one kv head, the query ROWS of a
// sequence are its (token, head of the group) pairs, token-major; a wave owns 16 rows and walks the keys in steps of 32 that start
// at multiples of 32 of the key index (never across a page):
//   S[key][row]  = K tile (A operand: cache rows as they lie) x Q (B operand, in registers), two 16-key tiles per step, fp32
//   cap, distance penalty, window and causal mask (by select: whatever the cache holds at a masked key cannot leak), online
//   softmax per row in fp32 on the accumulator fragments (a lane holds 8 keys of one row; a row's 4 lanes meet by two shuffles)
//   O[dv][row]  += V^T tile (A operand: two 8-byte loads from the transposed page) x P (B operand: the lane's 8 weights as bf16);
//   the k slots of the second product are the keys in the order the first product's fragments hold them: no data moves between lanes.
// tile mode  (a sequence brings more than 16 rows): workgroup = 4 waves = 64 consecutive rows; every wave walks the keys from the
//            window start of its first row to the position of its last.
// split mode (<= 16 rows: decoding): the 4 waves share the rows and take the steps round-robin; partial (max, sum, O) meet in LDS and
//            are merged in wave order.  The window bounds the steps, so the keys are not cut over the grid.
// V of keys past the last row's position is zeroed (a weight of zero times whatever an unwritten slot holds must stay zero).
// The sink joins the denominator at the end.  The cap's tanh is 1 - 2 / (1 + exp(2x)) on the fast exponential.
// ---------------------------------------------------------------------------------------------------------------------
template <int MK, int MV>        // upper bounds of D / 32 and Dv / 16 (register arrays)
__global__ void __launch_bounds__(256)
winattn_mfma_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vt,
                    const float* __restrict__ slopes, const float* __restrict__ sinks, const int32_t* __restrict__ bt, int max_blocks,
                    const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_q, int q_per_seq, int H, int G, int D, int Dv,
                    int bs, int window, float scale, float cap, const float* __restrict__ out_freqs, bf16_t* __restrict__ out) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, qd = lane >> 4;
  const int b = blockIdx.z, g = blockIdx.y, R = H / G;
  const int KS = D >> 5, DVT = Dv >> 4;
  const int tok0 = cu_q ? cu_q[b] : b * q_per_seq;
  const int nrows = (cu_q ? cu_q[b + 1] - tok0 : q_per_seq) * R;
  const bool split = nrows <= 16;
  if ((int)blockIdx.x * 64 >= nrows) return;
  const int row0 = split ? 0 : blockIdx.x * 64 + wave * 16;
  if (!split && row0 >= nrows) return;                 // (tile mode has no workgroup barriers)
  const int row = row0 + r;
  const bool valid = row < nrows;
  const int rr = valid ? row : row0;
  const int token = tok0 + rr / R, head = g * R + rr % R;
  const int pos = valid ? (int)positions[token] : -1;
  const int first = valid ? (window > 0 && pos + 1 > window ? pos + 1 - window : 0) : 0x7fffffff;
  const float slope = slopes ? slopes[head] : 0.f;
  int kmax = pos, kmin = first;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { kmax = max(kmax, __shfl_xor(kmax, o, 64)); kmin = min(kmin, __shfl_xor(kmin, o, 64)); }
  const int32_t* table = bt + (size_t)b * max_blocks;

  u32x4_t qreg[MK];
  const bf16_t* qrow = q + ((size_t)token * H + head) * D;
#pragma unroll
  for (int ks = 0; ks < MK; ++ks) {
    qreg[ks] = u32x4_t{0u, 0u, 0u, 0u};
    if (ks < KS && valid) qreg[ks] = *reinterpret_cast<const u32x4_t*>(qrow + ks * 32 + qd * 8);
  }
  float mx = -INFINITY, ls = 0.f;
  f32x4_t acc[MV];
#pragma unroll
  for (int i = 0; i < MV; ++i) acc[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;

  const int s_first = kmin >> 5, s_last = kmax >> 5;
  for (int st = s_first + (split ? wave : 0); st <= s_last; st += split ? 4 : 1) {
    const int k0 = st << 5;
    const size_t pg = (size_t)table[k0 / bs] * G + g;
    const int koff = k0 % bs;
    u32x4_t kreg[2][MK];
    u32x2_t vlo[MV], vhi[MV];
#pragma unroll
    for (int hg = 0; hg < 2; ++hg) {
      const bf16_t* kr = kc + (pg * bs + koff + hg * 16 + r) * D + qd * 8;
#pragma unroll
      for (int ks = 0; ks < MK; ++ks) {
        kreg[hg][ks] = u32x4_t{0u, 0u, 0u, 0u};
        if (ks < KS) kreg[hg][ks] = *reinterpret_cast<const u32x4_t*>(kr + ks * 32);
      }
    }
#pragma unroll
    for (int i = 0; i < MV; ++i) {
      vlo[i] = u32x2_t{0u, 0u};
      vhi[i] = u32x2_t{0u, 0u};
      if (i < DVT) {
        const bf16_t* vp = vt + (pg * Dv + i * 16 + r) * bs + koff + qd * 4;
        vlo[i] = *reinterpret_cast<const u32x2_t*>(vp);
        vhi[i] = *reinterpret_cast<const u32x2_t*>(vp + 16);
      }
    }
    if (k0 + 31 > kmax) {       // keys past the last row's position were never stored: whatever lies there must not meet a zero weight
      const int ka = k0 + qd * 4;
      const uint32_t l0 = (ka <= kmax ? 0xffffu : 0u) | (ka + 1 <= kmax ? 0xffff0000u : 0u);
      const uint32_t l1 = (ka + 2 <= kmax ? 0xffffu : 0u) | (ka + 3 <= kmax ? 0xffff0000u : 0u);
      const uint32_t h0 = (ka + 16 <= kmax ? 0xffffu : 0u) | (ka + 17 <= kmax ? 0xffff0000u : 0u);
      const uint32_t h1 = (ka + 18 <= kmax ? 0xffffu : 0u) | (ka + 19 <= kmax ? 0xffff0000u : 0u);
#pragma unroll
      for (int i = 0; i < MV; ++i) { vlo[i][0] &= l0; vlo[i][1] &= l1; vhi[i][0] &= h0; vhi[i][1] &= h1; }
    }
    f32x4_t sc[2];
#pragma unroll
    for (int hg = 0; hg < 2; ++hg) {
      sc[hg] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < MK; ++ks)
        if (ks < KS) sc[hg] = mfma16(kreg[hg][ks], qreg[ks], sc[hg]);
    }
    // lane (row r, keys k0 + hg * 16 + qd * 4 + i)
    float sv[8], smax = -INFINITY;
#pragma unroll
    for (int hg = 0; hg < 2; ++hg)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = k0 + hg * 16 + qd * 4 + i;
        float s = sc[hg][i] * scale;
        if (cap > 0.f) s = cap * (1.0f - 2.0f / (1.0f + __expf(2.0f * s * inv_cap)));
        s -= slope * (float)(pos - key);
        s = (key <= pos && key >= first) ? s : -INFINITY;
        sv[hg * 4 + i] = s;
        smax = fmaxf(smax, s);
      }
    smax = fmaxf(smax, __shfl_xor(smax, 16, 64));
    smax = fmaxf(smax, __shfl_xor(smax, 32, 64));
    const float mn = fmaxf(mx, smax);
    const float c = mn == -INFINITY ? 1.0f : __expf(mx - mn);
    float psum = 0.f, pv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      pv[i] = sv[i] == -INFINITY ? 0.f : __expf(sv[i] - mn);
      psum += pv[i];
    }
    ls = ls * c + psum;
    mx = mn;
    u32x4_t pb;
    pb[0] = pack_bf2_hw(pv[0], pv[1]); pb[1] = pack_bf2_hw(pv[2], pv[3]);
    pb[2] = pack_bf2_hw(pv[4], pv[5]); pb[3] = pack_bf2_hw(pv[6], pv[7]);
#pragma unroll
    for (int i = 0; i < MV; ++i)
      if (i < DVT) {
        acc[i] *= c;
        const u32x4_t va = u32x4_t{vlo[i][0], vlo[i][1], vhi[i][0], vhi[i][1]};
        acc[i] = mfma16(va, pb, acc[i]);
      }
  }
  ls += __shfl_xor(ls, 16, 64);
  ls += __shfl_xor(ls, 32, 64);

  if (split) {
    // partial rows of the four waves meet in LDS: [wave][16 rows][Dv] sums, [wave][16] max and sum; merged in wave order
    float* so = smem;                               // [4][16][Dv]
    float* sm = so + 4 * 16 * Dv;                   // [4][16]
    float* sl = sm + 64;                            // [4][16]
#pragma unroll
    for (int i = 0; i < MV; ++i)
      if (i < DVT)
#pragma unroll
        for (int e = 0; e < 4; ++e) so[(wave * 16 + r) * Dv + i * 16 + qd * 4 + e] = acc[i][e];
    if (qd == 0) { sm[wave * 16 + r] = mx; sl[wave * 16 + r] = ls; }
    __syncthreads();
    if (wave != 0) return;
    float M = -INFINITY;
    for (int w = 0; w < 4; ++w) M = fmaxf(M, sm[w * 16 + r]);
    float f[4], L = 0.f;
    for (int w = 0; w < 4; ++w) {
      f[w] = sl[w * 16 + r] > 0.f ? __expf(sm[w * 16 + r] - M) : 0.f;
      L += sl[w * 16 + r] * f[w];
    }
#pragma unroll
    for (int i = 0; i < MV; ++i)
      if (i < DVT)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float o = 0.f;
          for (int w = 0; w < 4; ++w) o += so[(w * 16 + r) * Dv + i * 16 + qd * 4 + e] * f[w];
          acc[i][e] = o;
        }
    mx = M; ls = L;
  }
  if (!valid) return;
  const float sink = sinks ? sinks[head] : -INFINITY;
  const float M = fmaxf(mx, sink);
  const float fo = ls > 0.f ? __expf(mx - M) : 0.f;
  const float den = ls * fo + (sinks ? __expf(sink - M) : 0.f);
  const float rs = fo / den;
#pragma unroll
  for (int i = 0; i < MV; ++i)
    if (i < DVT) acc[i] *= rs;
  if (out_freqs) {
    // the head's output turns back by the query's position; Dv % 32 == 0 here, so the partner of column i * 16 + qd * 4 + e (the
    // column Dv / 2 further) is element e of tile i + DVT / 2 of the SAME lane
    const int HT = DVT >> 1;
    if (DVT == MV) {
#pragma unroll
      for (int i = 0; i < MV / 2; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float sn, c;
          sincosf((float)pos * out_freqs[i * 16 + qd * 4 + e], &sn, &c);
          const float a = acc[i][e], b = acc[i + MV / 2][e];
          acc[i][e] = a * c + b * sn;
          acc[i + MV / 2][e] = b * c - a * sn;
        }
    } else {          // fewer value tiles than the register array holds: the partner tile's index is not a constant; select it
#pragma unroll
      for (int i = 0; i < MV / 2; ++i)
        if (i < HT) {
          f32x4_t pb = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int k = 0; k < MV; ++k) pb = (k == i + HT) ? acc[k] : pb;
          f32x4_t na, nb;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float sn, c;
            sincosf((float)pos * out_freqs[i * 16 + qd * 4 + e], &sn, &c);
            na[e] = acc[i][e] * c + pb[e] * sn;
            nb[e] = pb[e] * c - acc[i][e] * sn;
          }
          acc[i] = na;
#pragma unroll
          for (int k = 0; k < MV; ++k) acc[k] = (k == i + HT) ? nb : acc[k];
        }
    }
  }
  bf16_t* orow = out + ((size_t)token * H + head) * Dv + qd * 4;
#pragma unroll
  for (int i = 0; i < MV; ++i)
    if (i < DVT) {
      u32x2_t o2;
      o2[0] = pack_bf2_hw(acc[i][0], acc[i][1]);
      o2[1] = pack_bf2_hw(acc[i][2], acc[i][3]);
      *reinterpret_cast<u32x2_t*>(orow + i * 16) = o2;
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

extern "C" int ssd_winattn_store_rope(const void* qkv_rows, long ld, const void* q_norm_w, const void* k_norm_w, float eps,
                                      const int64_t* positions, const float* qk_freqs, int rot_dims, const float* v_freqs,
                                      const int32_t* slots, void* q_out, void* k_cache, void* v_cache, int T, int H, int G, int D, int Dv,
                                      int block_size, int f32, void* stream) {
  if (!qkv_rows || !q_norm_w || !k_norm_w || !positions || !slots || !q_out || !k_cache || !v_cache || (rot_dims > 0 && !qk_freqs))
    return SSD_ERR_ARG;
  if (T <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || block_size <= 0 || rot_dims < 0 || rot_dims > D || (rot_dims & 1) ||
      (v_freqs && (Dv & 1)) || ld < (long)(H + G) * D + (long)G * Dv)
    return SSD_ERR_SHAPE;
  const int items = (H + G) * (D - rot_dims / 2) + G * (v_freqs ? Dv / 2 : Dv);
  const int yb = T >= 64 ? 1 : ((items + 255) / 256 < 16 ? (items + 255) / 256 : 16);
  const dim3 grid(T, yb);
  if (f32)
    hipLaunchKernelGGL(winattn_store_rope_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)qkv_rows, ld,
                       (const float*)q_norm_w, (const float*)k_norm_w, eps, positions, qk_freqs, rot_dims, v_freqs, slots,
                       (float*)q_out, (float*)k_cache, (float*)v_cache, H, G, D, Dv, block_size);
  else
    hipLaunchKernelGGL(winattn_store_rope_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)qkv_rows, ld,
                       (const bf16_t*)q_norm_w, (const bf16_t*)k_norm_w, eps, positions, qk_freqs, rot_dims, v_freqs, slots,
                       (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, H, G, D, Dv, block_size);
  return LAUNCH_OK();
}

extern "C" int ssd_winattn_paged(const void* q_rows, const void* k_cache, const void* v_cache, const float* slopes, const float* sinks,
                                 const int32_t* block_tables, int max_blocks, const int64_t* positions, const int32_t* cu_q,
                                 int q_per_seq, int max_q, int B, int T, int H, int G, int D, int Dv, int block_size, int window,
                                 float scale, float cap, const float* out_freqs, void* out_rows, int f32, void* stream) {
  if (!q_rows || !k_cache || !v_cache || !block_tables || !positions || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || B <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || Dv > 64 * WA_MAXV || block_size <= 0 || window < 0 ||
      max_blocks <= 0 || (!cu_q && q_per_seq <= 0) || H > 65535 || (out_freqs && (Dv & 1)))
    return SSD_ERR_SHAPE;
  if (!f32 && max_q > 0 && D % 32 == 0 && D <= 256 && Dv % (out_freqs ? 32 : 16) == 0 && Dv <= 256 && block_size % 32 == 0 && G <= 65535 &&
      B <= 65535) {
    const int R = H / G;
    const dim3 grid((unsigned)(((long)max_q * R + 63) / 64), G, B);
    const size_t lds = (4 * 16 * (size_t)Dv + 128) * sizeof(float);
#define WIN_MFMA(MK, MV)                                                                                                            \
  hipLaunchKernelGGL((winattn_mfma_kernel<MK, MV>), grid, dim3(256), lds, (hipStream_t)stream, (const bf16_t*)q_rows,               \
                     (const bf16_t*)k_cache, (const bf16_t*)v_cache, slopes, sinks, block_tables, max_blocks, positions, cu_q,      \
                     q_per_seq, H, G, D, Dv, block_size, window, scale, cap, out_freqs, (bf16_t*)out_rows)
    if (D <= 64 && Dv <= 64) WIN_MFMA(2, 4);
    else if (D <= 128 && Dv <= 128) WIN_MFMA(4, 8);
    else {
      if (lds > 64 * 1024 && hipFuncSetAttribute((const void*)winattn_mfma_kernel<8, 16>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 (int)lds) != hipSuccess)
        return SSD_ERR_LAUNCH;
      WIN_MFMA(8, 16);
    }
#undef WIN_MFMA
    return LAUNCH_OK();
  }
  const size_t bytes = ((size_t)D + (D & 1) + 4 * 64 + 2 * 4 * 64 + 4 * (size_t)Dv + 8) * sizeof(float);
  if (bytes > 64 * 1024) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(winattn_paged_kernel<float>, dim3(T, H), dim3(256), bytes, (hipStream_t)stream, (const float*)q_rows,
                       (const float*)k_cache, (const float*)v_cache, slopes, sinks, block_tables, max_blocks, positions, cu_q, q_per_seq,
                       B, H, G, D, Dv, block_size, window, scale, cap, out_freqs, (float*)out_rows);
  else
    hipLaunchKernelGGL(winattn_paged_kernel<bf16_t>, dim3(T, H), dim3(256), bytes, (hipStream_t)stream, (const bf16_t*)q_rows,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, slopes, sinks, block_tables, max_blocks, positions, cu_q,
                       q_per_seq, B, H, G, D, Dv, block_size, window, scale, cap, out_freqs, (bf16_t*)out_rows);
  return LAUNCH_OK();
}
