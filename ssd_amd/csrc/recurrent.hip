// Recurrent mixers whose per-sequence memory is an fp32 matrix state per head plus a few rows of recent inputs, kept in the slot pool
// that the block manager hands out (one slot per live sequence).  A forward reads a slot unless the rows it brings start at position 0,
// walks its rows in order and writes the slot back, so a prompt may arrive in portions of any size; decoding is the one-row case.
//
//  token shift          ssd_token_shift_mix    mix_s = h + (h_prev - h) * mu_s for S interpolation vectors at once (h_prev: the previous
//                                              token's row, from the batch, from the slot's saved row, or zero before position 0)
//  time mixing ("wkv")  ssd_wkv_scan           per head, S [D][D]:  o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,  S_t = diag(w_t) S_(t-1) + k_t v_t^T,
//                                              w_t = exp(-exp(ww_t + w0)) per key channel; also saves the slot's token-shift row
//  short convolution    ssd_causal_conv_silu   out[c] = silu(b[c] + sum_j w[c][j] in_(t - (taps - 1 - j))[c]), inputs before the portion from
//                                              the slot's saved rows, zero before position 0
//  state space          ssd_ssd_scan           per head, S [N][Dv]:  S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T,  y_t = S_t^T C_t + D x_t,
//                                              dt_t = softplus(dt_raw + dt_bias) (no clamp); B / C shared by the heads of a group; also
//                                              saves the slot's last taps - 1 convolution inputs
//  output               ssd_group_gate_norm    RMS norm in `groups` equal parts of the row, a silu gate either BEFORE the norm (gate_first)
//                                              or after it, times a weight, as GEMM-input rows
// Everything that enters a recurrence is fp32: the projections' fp32 accumulators come in as fp32 rows, decays, step sizes, states and
// sums stay fp32.  The arithmetic of a row does not depend on the portioning: per state element one multiply-add chain in token order,
// the output a sum over the state rows in a fixed order.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }

__device__ __forceinline__ float siluf_(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

__device__ __forceinline__ int seq_of_row(const int32_t* cu_q, int q_per_seq, int B, int t) {
  if (!cu_q) return t / q_per_seq;
  int lo = 0, hi = B;
  while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (cu_q[mid] <= t) lo = mid; else hi = mid; }
  return lo;
}

template <typename T>
__global__ void __launch_bounds__(256)
token_shift_mix_kernel(const T* __restrict__ hn, const T* __restrict__ mu, const float* __restrict__ shift_state,
                       const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_q, int q_per_seq,
                       const int32_t* __restrict__ state_slots, int B, T* __restrict__ out, int W, int S) {
  const int t = blockIdx.x;
  const int b = seq_of_row(cu_q, q_per_seq, B, t);
  const int row0 = cu_q ? cu_q[b] : b * q_per_seq;
  const bool from_batch = t > row0, zero = !from_batch && positions[t] == 0;
  const float* st = shift_state + (size_t)state_slots[b] * W;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < W; c += 256 * gridDim.y) {
    const float h = ldf<T>(hn + (size_t)t * W + c);
    const float prev = from_batch ? ldf<T>(hn + (size_t)(t - 1) * W + c) : (zero ? 0.f : st[c]);
    for (int s = 0; s < S; ++s) stf<T>(out + ((size_t)t * S + s) * W + c, fmaf(prev - h, ldf<T>(mu + (size_t)s * W + c), h));
  }
}

// One workgroup per (sequence, head).  Threads form NG groups of EP lanes (EP = power of two >= min(Dv, 256)): lane e of group g owns
// the state elements (d, e) with d = g, g + NG, ...; the groups' partial outputs meet in LDS and are summed in group order.
// MODE 0 (time mixing): the output reads the state BEFORE the update plus the bonus for the current token.
// MODE 1 (state space): the output reads the state AFTER the update, plus skip * v.
template <int MODE>
__device__ __forceinline__ void scan_rows(float* S, const float* sq, const float* sk, const float* sd, const float* su, const float* sv,
                                          float* po, int D, int Dv, int EP, float skip, float* out_row) {
  const int tid = threadIdx.x, NG = 256 / EP, g = tid / EP, el = tid % EP;
  for (int e = el; e < Dv; e += EP) {
    const float ve = sv[e];
    float o = 0.f;
    for (int d = g; d < D; d += NG) {
      const float s = S[d * Dv + e], kv = sk[d] * ve;
      if (MODE == 0) {
        o = fmaf(fmaf(su[d], kv, s), sq[d], o);
        S[d * Dv + e] = fmaf(sd[d], s, kv);
      } else {
        const float n = fmaf(sd[d], s, kv);
        S[d * Dv + e] = n;
        o = fmaf(n, sq[d], o);
      }
    }
    po[g * Dv + e] = o;
  }
  __syncthreads();
  for (int e = tid; e < Dv; e += 256) {
    float o = 0.f;
    for (int gg = 0; gg < NG; ++gg) o += po[gg * Dv + e];
    out_row[e] = MODE == 0 ? o : fmaf(skip, sv[e], o);
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
wkv_scan_kernel(const float* __restrict__ proj, long ld, int r_off, int k_off, int v_off, const float* __restrict__ ww, long ldw,
                const float* __restrict__ w0, const float* __restrict__ u, const int64_t* __restrict__ positions,
                const int32_t* __restrict__ cu_q, int q_per_seq, const int32_t* __restrict__ state_slots, float* __restrict__ state,
                float* __restrict__ out, const T* __restrict__ hn, float* __restrict__ shift_state, int W, int H, int D, int EP) {
  extern __shared__ float lds[];
  float* S = lds;                         // [D][D]
  float* sq = S + (size_t)D * D;
  float* sk = sq + D;
  float* sd = sk + D;
  float* su = sd + D;
  float* sv = su + D;
  float* po = sv + D;                     // [NG][D]
  const int b = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int row0 = cu_q ? cu_q[b] : b * q_per_seq;
  const int row1 = cu_q ? cu_q[b + 1] : (b + 1) * q_per_seq;
  if (row1 <= row0) return;
  const int slot = state_slots[b];
  float* sp = state + ((size_t)slot * H + h) * D * D;
  const bool fresh = positions[row0] == 0;
  for (int i = tid; i < D * D; i += 256) S[i] = fresh ? 0.f : sp[i];
  for (int i = tid; i < D; i += 256) su[i] = u[h * D + i];
  for (int r = row0; r < row1; ++r) {
    const float* pr = proj + (size_t)r * ld + h * D;
    __syncthreads();
    for (int i = tid; i < D; i += 256) {
      sq[i] = pr[r_off + i];
      sk[i] = pr[k_off + i];
      sv[i] = pr[v_off + i];
      sd[i] = expf(-expf(ww[(size_t)r * ldw + h * D + i] + w0[h * D + i]));
    }
    __syncthreads();
    scan_rows<0>(S, sq, sk, sd, su, sv, po, D, D, EP, 0.f, out + (size_t)r * H * D + h * D);
  }
  __syncthreads();
  for (int i = tid; i < D * D; i += 256) sp[i] = S[i];
  // the last row of the portion is the next portion's "previous token": every head's workgroup saves its share of the columns
  const int chunk = (W + H - 1) / H;
  for (int c = h * chunk + tid; c < min(W, (h + 1) * chunk); c += 256)
    shift_state[(size_t)slot * W + c] = ldf<T>(hn + (size_t)(row1 - 1) * W + c);
}

template <typename T>
__global__ void __launch_bounds__(256)
causal_conv_silu_kernel(const float* __restrict__ proj, long ld, int col_off, int C, const T* __restrict__ cw, const T* __restrict__ cb,
                        const float* __restrict__ conv_state, const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_q,
                        int q_per_seq, const int32_t* __restrict__ state_slots, int B, float* __restrict__ out, int taps) {
  const int t = blockIdx.x;
  const int b = seq_of_row(cu_q, q_per_seq, B, t);
  const int row0 = cu_q ? cu_q[b] : b * q_per_seq;
  const long p0 = positions[row0];
  const float* st = conv_state + (size_t)state_slots[b] * (taps - 1) * C;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += 256 * gridDim.y) {
    float acc = ldf<T>(cb + c);
    for (int j = 0; j < taps; ++j) {
      const int src = t - (taps - 1 - j);
      float v;
      if (src >= row0) {
        v = proj[(size_t)src * ld + col_off + c];
      } else {
        const int k = row0 - src;                          // k tokens before the portion's first row
        v = p0 - k >= 0 ? st[(size_t)(taps - 1 - k) * C + c] : 0.f;
      }
      acc = fmaf(ldf<T>(cw + (size_t)c * taps + j), v, acc);
    }
    out[(size_t)t * C + c] = siluf_(acc);
  }
}

constexpr int CONV_MAX_TAPS = 16;

// Channels [c_begin, c_end) of the slot's saved convolution inputs: saved row i holds the input of position p0 + n - (taps - 1) + i.
__device__ __forceinline__ void save_conv_state(const float* proj, long ld, int conv_off, int C, float* conv_state, int taps, int slot,
                                                int row0, int row1, long p0, int c_begin, int c_end) {
  const int n = row1 - row0, K1 = taps - 1;
  float* st = conv_state + (size_t)slot * K1 * C;
  for (int c = c_begin + threadIdx.x; c < c_end; c += 256) {
    float keep[CONV_MAX_TAPS];
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS; ++i) {
      keep[i] = 0.f;
      if (i < K1) {
        const long rel = (long)n - K1 + i;                // position relative to the portion's first row
        if (rel >= 0) keep[i] = proj[(size_t)(row0 + rel) * ld + conv_off + c];
        else if (p0 + rel >= 0) keep[i] = st[(size_t)(i + n) * C + c];
      }
    }
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS; ++i)
      if (i < K1) st[(size_t)i * C + c] = keep[i];
  }
}


__global__ void __launch_bounds__(256)
ssd_scan_kernel(const float* __restrict__ xbc, long ldx, int x_off, int b_off, int c_off, const float* __restrict__ proj, long ld,
                int dt_off, const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ dskip,
                const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_q, int q_per_seq,
                const int32_t* __restrict__ state_slots, float* __restrict__ state, float* __restrict__ out, int conv_off, int C,
                float* __restrict__ conv_state, int taps, int H, int G, int N, int Dv, int EP) {
  extern __shared__ float lds[];
  float* S = lds;                         // [N][Dv]
  float* sq = S + (size_t)N * Dv;
  float* sk = sq + N;
  float* sd = sk + N;
  float* sv = sd + N;                     // [Dv]
  float* po = sv + Dv;                    // [NG][Dv]
  const int b = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int grp = h / (H / G);
  const int row0 = cu_q ? cu_q[b] : b * q_per_seq;
  const int row1 = cu_q ? cu_q[b + 1] : (b + 1) * q_per_seq;
  if (row1 <= row0) return;
  const int slot = state_slots[b];
  float* sp = state + ((size_t)slot * H + h) * N * Dv;
  const long p0 = positions[row0];
  const bool fresh = p0 == 0;
  for (int i = tid; i < N * Dv; i += 256) S[i] = fresh ? 0.f : sp[i];
  const float a = -expf(a_log[h]), dtb = dt_bias[h], skip = dskip[h];
  for (int r = row0; r < row1; ++r) {
    const float* xr = xbc + (size_t)r * ldx;
    const float dt = softplusf_(proj[(size_t)r * ld + dt_off + h] + dtb);
    const float dA = expf(a * dt);
    __syncthreads();
    for (int i = tid; i < N; i += 256) {
      sq[i] = xr[c_off + grp * N + i];
      sk[i] = dt * xr[b_off + grp * N + i];
      sd[i] = dA;
    }
    for (int i = tid; i < Dv; i += 256) sv[i] = xr[x_off + h * Dv + i];
    __syncthreads();
    scan_rows<1>(S, sq, sk, sd, nullptr, sv, po, N, Dv, EP, skip, out + (size_t)r * H * Dv + h * Dv);
  }
  __syncthreads();
  for (int i = tid; i < N * Dv; i += 256) sp[i] = S[i];
  if (taps > 1) {              // the slot's last taps - 1 convolution inputs: every head's workgroup saves its share of the channels
    const int chunk = (C + H - 1) / H;
    save_conv_state(proj, ld, conv_off, C, conv_state, taps, slot, row0, row1, p0, h * chunk, min(C, (h + 1) * chunk));
  }
}

// Register form of both scans (state rows D = 8 * EPT with EPT in {4, 8, 16, 32}, Dv % 32 == 0): a workgroup owns 32 state columns of one
// (sequence, head) -- grid.z walks the column blocks -- and thread (g, e) keeps the EPT elements (d = g + 8 n, column e) in registers.
// Rows are staged eight at a time (decays and step sizes computed once per row), every thread then walks the eight tokens without a
// barrier, and the eight d-groups' partial outputs are summed in group order.  The arithmetic of a row is the same for any portioning:
// the per-element chain in token order, the output sum over n ascending, then over g ascending.
struct WkvArgs {
  const float* proj; long ld; int r_off, k_off, v_off; const float* ww; long ldw; const float* w0; const float* u;
};
struct SsdArgs {
  const float* xbc; long ldx; int x_off, b_off, c_off; const float* proj; long ld; int dt_off; const float* dt_bias; const float* a_log;
  const float* skip; int G, conv_off, C, taps; float* conv_state;
};

template <int MODE, int EPT, typename T>
__global__ void __launch_bounds__(256)
scan_reg_kernel(WkvArgs wa, SsdArgs sa, const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_q, int q_per_seq,
                const int32_t* __restrict__ state_slots, float* __restrict__ state, float* __restrict__ out, const T* __restrict__ hn,
                float* __restrict__ shift_state, int W, int H, int Dv) {
  constexpr int TB = 8, NG = 8, CB = 32, D = NG * EPT;
  __shared__ float sq[TB][D], sk[TB][D], sd[TB][MODE == 0 ? D : 1];
  __shared__ float sv[TB][CB];
  __shared__ float po[TB][NG][CB];
  const int b = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * CB, tid = threadIdx.x;
  const int g = tid >> 5, e = tid & 31;
  const int row0 = cu_q ? cu_q[b] : b * q_per_seq;
  const int row1 = cu_q ? cu_q[b + 1] : (b + 1) * q_per_seq;
  if (row1 <= row0) return;
  const int slot = state_slots[b];
  float* sp = state + ((size_t)slot * H + h) * D * Dv + c0 + e;
  const long p0 = positions[row0];
  const bool fresh = p0 == 0;
  float S[EPT], U[EPT];
#pragma unroll
  for (int n = 0; n < EPT; ++n) {
    S[n] = fresh ? 0.f : sp[(size_t)(g + NG * n) * Dv];
    U[n] = MODE == 0 ? wa.u[h * D + g + NG * n] : 0.f;
  }
  const int grp = MODE == 1 ? h / (H / sa.G) : 0;
  const float a = MODE == 1 ? -expf(sa.a_log[h]) : 0.f, dtb = MODE == 1 ? sa.dt_bias[h] : 0.f, skip = MODE == 1 ? sa.skip[h] : 0.f;
  // raw values of the next batch travel in registers while the current batch is computed (a batch is short: without this every
  // batch would wait a full memory round trip)
  constexpr int QK = TB * D / 256;         // q / k / decay elements of a batch per thread
  float rq[QK], rk[QK], rw[QK], w0r[QK], rv = 0.f;
#pragma unroll
  for (int c = 0; c < QK; ++c) w0r[c] = MODE == 0 ? wa.w0[h * D + (tid + 256 * c) % D] : 0.f;
  auto fetch = [&](int r) {
    const int nb = row1 - r < TB ? row1 - r : TB;
#pragma unroll
    for (int c = 0; c < QK; ++c) {
      const int idx = tid + 256 * c, tt = idx / D, d = idx % D;
      rq[c] = rk[c] = rw[c] = 0.f;
      if (tt < nb) {
        if (MODE == 0) {
          const float* pr = wa.proj + (size_t)(r + tt) * wa.ld + h * D + d;
          rq[c] = pr[wa.r_off];
          rk[c] = pr[wa.k_off];
          rw[c] = wa.ww[(size_t)(r + tt) * wa.ldw + h * D + d];
        } else {
          const float* xr = sa.xbc + (size_t)(r + tt) * sa.ldx + grp * D + d;
          rq[c] = xr[sa.c_off];
          rk[c] = xr[sa.b_off];
          rw[c] = sa.proj[(size_t)(r + tt) * sa.ld + sa.dt_off + h];          // the row's raw step size
        }
      }
    }
    rv = 0.f;
    if (g < nb)
      rv = MODE == 0 ? wa.proj[(size_t)(r + g) * wa.ld + wa.v_off + h * Dv + c0 + e]
                     : sa.xbc[(size_t)(r + g) * sa.ldx + sa.x_off + h * Dv + c0 + e];
  };
  fetch(row0);
  for (int r = row0; r < row1; r += TB) {
    const int nb = row1 - r < TB ? row1 - r : TB;
    __syncthreads();                      // the previous batch's readers are done
#pragma unroll
    for (int c = 0; c < QK; ++c) {
      const int idx = tid + 256 * c, tt = idx / D, d = idx % D;
      sq[tt][d] = rq[c];
      if (MODE == 0) {
        sk[tt][d] = rk[c];
        sd[tt][d] = expf(-expf(rw[c] + w0r[c]));
      } else {
        const float dt = softplusf_(rw[c] + dtb);
        sk[tt][d] = dt * rk[c];
        if (d == 0) sd[tt][0] = expf(a * dt);
      }
    }
    sv[g][e] = rv;
    __syncthreads();
    if (r + TB < row1) fetch(r + TB);
    for (int tt = 0; tt < nb; ++tt) {
      const float ve = sv[tt][e];
      float o = 0.f;
#pragma unroll
      for (int n = 0; n < EPT; ++n) {
        const int d = g + NG * n;
        const float kv = sk[tt][d] * ve;
        if (MODE == 0) {
          o = fmaf(fmaf(U[n], kv, S[n]), sq[tt][d], o);
          S[n] = fmaf(sd[tt][d], S[n], kv);
        } else {
          S[n] = fmaf(sd[tt][0], S[n], kv);
          o = fmaf(S[n], sq[tt][d], o);
        }
      }
      po[tt][g][e] = o;
    }
    __syncthreads();
    if (g < nb) {                         // thread (g, e) now finishes token g of the batch
      float o = 0.f;
#pragma unroll
      for (int gg = 0; gg < NG; ++gg) o += po[g][gg][e];
      if (MODE == 1) o = fmaf(skip, sv[g][e], o);
      out[(size_t)(r + g) * H * Dv + h * Dv + c0 + e] = o;
    }
  }
#pragma unroll
  for (int n = 0; n < EPT; ++n) sp[(size_t)(g + NG * n) * Dv] = S[n];
  // the slot's saved rows (token shift / convolution inputs): every workgroup of the sequence saves its share of the columns
  const int wg = h * gridDim.z + blockIdx.z, nwg = H * gridDim.z;
  if (MODE == 0) {
    const int chunk = (W + nwg - 1) / nwg;
    for (int c = wg * chunk + tid; c < min(W, (wg + 1) * chunk); c += 256)
      shift_state[(size_t)slot * W + c] = ldf<T>(hn + (size_t)(row1 - 1) * W + c);
  } else if (sa.taps > 1) {
    const int chunk = (sa.C + nwg - 1) / nwg;
    save_conv_state(sa.proj, sa.ld, sa.conv_off, sa.C, sa.conv_state, sa.taps, slot, row0, row1, p0, wg * chunk, min(sa.C, (wg + 1) * chunk));
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
group_gate_norm_kernel(const float* __restrict__ o, const float* __restrict__ gate, long ldg, const T* __restrict__ w, float eps,
                       T* __restrict__ out, int N, int groups, int gate_first) {
  const size_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, per = N / groups;
  const float* orow = o + t * N;
  const float* grow = gate + t * ldg;
  for (int g = blockIdx.y * 4 + wave; g < groups; g += 4 * gridDim.y) {
    float ss = 0.f;
    for (int c = g * per + lane; c < (g + 1) * per; c += 64) {
      const float v = gate_first ? orow[c] * siluf_(grow[c]) : orow[c];
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)per + eps);
    for (int c = g * per + lane; c < (g + 1) * per; c += 64) {
      const float gs = siluf_(grow[c]);
      const float v = gate_first ? orow[c] * gs * r * ldf<T>(w + c) : orow[c] * r * ldf<T>(w + c) * gs;
      stf<T>(out + t * N + c, v);
    }
  }
}

int pick_ep(int Dv) {
  int EP = 1;
  while (EP < Dv && EP < 256) EP <<= 1;
  return EP;
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_token_shift_mix(const void* hn_rows, const void* mu, const float* shift_state, const int64_t* positions,
                                   const int32_t* cu_q, int q_per_seq, const int32_t* state_slots, int B, void* out_rows, int T, int W,
                                   int S, int f32, void* stream) {
  if (!hn_rows || !mu || !shift_state || !positions || !state_slots || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0 || S <= 0 || B <= 0 || (!cu_q && q_per_seq <= 0)) return SSD_ERR_SHAPE;
  const int cbk = (W + 255) / 256;
  const dim3 grid(T, T >= 256 ? 1 : (cbk < 32 ? cbk : 32));          // few rows: a row's columns spread over workgroups
  if (f32)
    hipLaunchKernelGGL(token_shift_mix_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)hn_rows, (const float*)mu,
                       shift_state, positions, cu_q, q_per_seq, state_slots, B, (float*)out_rows, W, S);
  else
    hipLaunchKernelGGL(token_shift_mix_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const bf16_t*)hn_rows,
                       (const bf16_t*)mu, shift_state, positions, cu_q, q_per_seq, state_slots, B, (bf16_t*)out_rows, W, S);
  return LAUNCH_OK();
}

extern "C" int ssd_wkv_scan(const void* proj_rows, long ld, int r_off, int k_off, int v_off, const void* decay_rows, long ldw,
                            const float* w0, const float* u, const int64_t* positions, const int32_t* cu_q, int q_per_seq,
                            const int32_t* state_slots, void* state, void* out_rows, const void* hn_rows, void* shift_state, int W,
                            int B, int H, int D, int f32, void* stream) {
  if (!proj_rows || !decay_rows || !w0 || !u || !positions || !state_slots || !state || !out_rows || !hn_rows || !shift_state)
    return SSD_ERR_ARG;
  if (B <= 0 || H <= 0 || D <= 0 || W <= 0 || (!cu_q && q_per_seq <= 0) || H > 65535) return SSD_ERR_SHAPE;
  if (D % 32 == 0 && (D == 32 || D == 64 || D == 128 || D == 256)) {
    const WkvArgs wa{(const float*)proj_rows, ld, r_off, k_off, v_off, (const float*)decay_rows, ldw, w0, u};
    const SsdArgs sa{};
    const dim3 grid(B, H, D / 32);
#define WKV_REG(EPT)                                                                                                                 \
  do {                                                                                                                               \
    if (f32)                                                                                                                         \
      hipLaunchKernelGGL((scan_reg_kernel<0, EPT, float>), grid, dim3(256), 0, (hipStream_t)stream, wa, sa, positions, cu_q, q_per_seq, \
                         state_slots, (float*)state, (float*)out_rows, (const float*)hn_rows, (float*)shift_state, W, H, D);        \
    else                                                                                                                             \
      hipLaunchKernelGGL((scan_reg_kernel<0, EPT, bf16_t>), grid, dim3(256), 0, (hipStream_t)stream, wa, sa, positions, cu_q,        \
                         q_per_seq, state_slots, (float*)state, (float*)out_rows, (const bf16_t*)hn_rows, (float*)shift_state, W, H, \
                         D);                                                                                                         \
  } while (0)
    if (D == 32) WKV_REG(4);
    else if (D == 64) WKV_REG(8);
    else if (D == 128) WKV_REG(16);
    else WKV_REG(32);
#undef WKV_REG
    return LAUNCH_OK();
  }
  const int EP = pick_ep(D);
  const size_t bytes = ((size_t)D * D + 6 * (size_t)D + (size_t)(256 / EP) * D) * sizeof(float);
  if (bytes > 160 * 1024) return SSD_ERR_SHAPE;
  const void* fn = f32 ? (const void*)wkv_scan_kernel<float> : (const void*)wkv_scan_kernel<bf16_t>;
  if (bytes > 64 * 1024 && hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess)
    return SSD_ERR_LAUNCH;
  if (f32)
    hipLaunchKernelGGL(wkv_scan_kernel<float>, dim3(B, H), dim3(256), bytes, (hipStream_t)stream, (const float*)proj_rows, ld, r_off,
                       k_off, v_off, (const float*)decay_rows, ldw, w0, u, positions, cu_q, q_per_seq, state_slots, (float*)state,
                       (float*)out_rows, (const float*)hn_rows, (float*)shift_state, W, H, D, EP);
  else
    hipLaunchKernelGGL(wkv_scan_kernel<bf16_t>, dim3(B, H), dim3(256), bytes, (hipStream_t)stream, (const float*)proj_rows, ld, r_off,
                       k_off, v_off, (const float*)decay_rows, ldw, w0, u, positions, cu_q, q_per_seq, state_slots, (float*)state,
                       (float*)out_rows, (const bf16_t*)hn_rows, (float*)shift_state, W, H, D, EP);
  return LAUNCH_OK();
}

extern "C" int ssd_causal_conv_silu(const void* proj_rows, long ld, int col_off, int C, const void* conv_w, const void* conv_b,
                                    const float* conv_state, const int64_t* positions, const int32_t* cu_q, int q_per_seq,
                                    const int32_t* state_slots, int B, void* out_rows, int T, int taps, int f32, void* stream) {
  if (!proj_rows || !conv_w || !conv_b || !conv_state || !positions || !state_slots || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || C <= 0 || taps < 1 || taps > CONV_MAX_TAPS || B <= 0 || (!cu_q && q_per_seq <= 0) || ld < col_off + C) return SSD_ERR_SHAPE;
  const int cb = (C + 255) / 256;
  const dim3 grid(T, cb < 64 ? cb : 64);
  if (f32)
    hipLaunchKernelGGL(causal_conv_silu_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)proj_rows, ld, col_off, C,
                       (const float*)conv_w, (const float*)conv_b, conv_state, positions, cu_q, q_per_seq, state_slots, B,
                       (float*)out_rows, taps);
  else
    hipLaunchKernelGGL(causal_conv_silu_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)proj_rows, ld, col_off, C,
                       (const bf16_t*)conv_w, (const bf16_t*)conv_b, conv_state, positions, cu_q, q_per_seq, state_slots, B,
                       (float*)out_rows, taps);
  return LAUNCH_OK();
}

extern "C" int ssd_ssd_scan(const void* xbc_rows, long ldx, int x_off, int b_off, int c_off, const void* proj_rows, long ld, int dt_off,
                            const float* dt_bias, const float* a_log, const float* skip, const int64_t* positions, const int32_t* cu_q,
                            int q_per_seq, const int32_t* state_slots, void* state, void* out_rows, int conv_off, int C,
                            void* conv_state, int taps, int B, int H, int G, int N, int Dv, void* stream) {
  if (!xbc_rows || !proj_rows || !dt_bias || !a_log || !skip || !positions || !state_slots || !state || !out_rows || !conv_state)
    return SSD_ERR_ARG;
  if (B <= 0 || H <= 0 || G <= 0 || H % G || N <= 0 || Dv <= 0 || taps < 1 || taps > CONV_MAX_TAPS || C <= 0 ||
      (!cu_q && q_per_seq <= 0) || H > 65535)
    return SSD_ERR_SHAPE;
  if (Dv % 32 == 0 && Dv / 32 <= 65535 && (N == 32 || N == 64 || N == 128 || N == 256)) {
    const WkvArgs wa{};
    const SsdArgs sa{(const float*)xbc_rows, ldx, x_off, b_off, c_off, (const float*)proj_rows, ld, dt_off, dt_bias, a_log, skip, G,
                     conv_off, C, taps, (float*)conv_state};
    const dim3 grid(B, H, Dv / 32);
#define SSD_REG(EPT)                                                                                                               \
  hipLaunchKernelGGL((scan_reg_kernel<1, EPT, float>), grid, dim3(256), 0, (hipStream_t)stream, wa, sa, positions, cu_q, q_per_seq, \
                     state_slots, (float*)state, (float*)out_rows, (const float*)nullptr, (float*)nullptr, 0, H, Dv)
    if (N == 32) SSD_REG(4);
    else if (N == 64) SSD_REG(8);
    else if (N == 128) SSD_REG(16);
    else SSD_REG(32);
#undef SSD_REG
    return LAUNCH_OK();
  }
  const int EP = pick_ep(Dv);
  const size_t bytes = ((size_t)N * Dv + 3 * (size_t)N + Dv + (size_t)(256 / EP) * Dv) * sizeof(float);
  if (bytes > 160 * 1024) return SSD_ERR_SHAPE;
  if (bytes > 64 * 1024 &&
      hipFuncSetAttribute((const void*)ssd_scan_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess)
    return SSD_ERR_LAUNCH;
  hipLaunchKernelGGL(ssd_scan_kernel, dim3(B, H), dim3(256), bytes, (hipStream_t)stream, (const float*)xbc_rows, ldx, x_off, b_off, c_off,
                     (const float*)proj_rows, ld, dt_off, dt_bias, a_log, skip, positions, cu_q, q_per_seq, state_slots, (float*)state,
                     (float*)out_rows, conv_off, C, (float*)conv_state, taps, H, G, N, Dv, EP);
  return LAUNCH_OK();
}

extern "C" int ssd_group_gate_norm(const void* o_rows, const void* gate_rows, long ldg, const void* weight, float eps, void* out_rows,
                                   int T, int N, int groups, int gate_first, int f32, void* stream) {
  if (!o_rows || !gate_rows || !weight || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || N <= 0 || groups <= 0 || N % groups || ldg < N) return SSD_ERR_SHAPE;
  const int gb = (groups + 3) / 4;
  const dim3 grid(T, T >= 256 ? 1 : (gb < 16 ? gb : 16));
  if (f32)
    hipLaunchKernelGGL(group_gate_norm_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)o_rows,
                       (const float*)gate_rows, ldg, (const float*)weight, eps, (float*)out_rows, N, groups, gate_first);
  else
    hipLaunchKernelGGL(group_gate_norm_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)o_rows,
                       (const float*)gate_rows, ldg, (const bf16_t*)weight, eps, (bf16_t*)out_rows, N, groups, gate_first);
  return LAUNCH_OK();
}
