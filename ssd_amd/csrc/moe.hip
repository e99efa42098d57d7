// Routed feed-forward (mixture of experts) around the grouped GEMM of gemm_rows.hip:
//   ssd_moe_route    from the router's fp32 logits z = W_r h (a GEMM with fp32 rows out): the `top` largest per token (lowest index
//                    wins a tie) and the softmax over them
//   ssd_moe_route_softmax  the other common router: scores = softmax over ALL experts, experts in contiguous groups of which only the
//                    best `keep` (by their largest score) stay eligible, the `top` largest eligible scores, divided by their sum
//                    (+ 1e-20) and multiplied by a constant
//   ssd_moe_route_sigmoid  scores = sigmoid of the logits, the `top` largest, weights = those scores unrenormalised
//   ssd_moe_route_sigmoid_grouped  sigmoid scores with a per-expert correction that enters the CHOICE only: choice = score + correction;
//                    experts in contiguous groups, a group's score = the sum of its `group_top` largest choice scores, only the best
//                    `keep` groups stay eligible; the `top` largest eligible choice scores win; weights = the chosen experts' plain scores
//   ssd_moe_plan     counting sort of the T * top (token, slot) pairs by expert: offsets[E+1], perm (sorted row -> pair), inv (pair -> sorted row)
//   ssd_moe_combine  out[t] = sum_j weight[t][j] * y[inv[t * top + j]] (+ shared[t]) in slot order, fp32
// Between plan and combine the caller runs the experts as two grouped GEMMs over the sorted rows (up with the activation as epilogue,
// then down).  A pair's row is computed by itself, so a token's result does not depend on the other tokens of the batch or on the order
// the sort happened to give its expert's rows.
#include "common.h"

namespace {

constexpr int MOE_MAX_E = 4096, MOE_MAX_TOP = 32;

__global__ void __launch_bounds__(64)
moe_route_kernel(const float* __restrict__ zin, int32_t* __restrict__ idx, float* __restrict__ wt, int E, int top) {
  extern __shared__ float z[];      // [E]
  const int t = blockIdx.x, lane = threadIdx.x;
  for (int e = lane; e < E; e += 64) z[e] = zin[(size_t)t * E + e];
  __syncthreads();
  // `top` rounds of a wave-wide argmax; among equal logits the lowest index wins
  float vmax = 0.f, den = 0.f, myval = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY; int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) { const float v = z[e]; if (v > best) { best = v; bi = e; } }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64); const int oi = __shfl_xor(bi, o, 64);
      if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if (j == 0) vmax = best;
    const float p = expf(best - vmax);
    den += p;
    if (lane == j % 64) { myval = p; idx[(size_t)t * top + j] = bi; }
    if (lane == 0) z[bi] = -INFINITY;
    __syncthreads();
  }
  if (lane < top) wt[(size_t)t * top + lane] = myval / den;
}

// Softmax-then-top-k routing with group-limited choice.  One wave per token; logits row stride ldz (other per-token logits may share the
// row).  Among equal scores the lowest index wins, for groups and for experts.
__global__ void __launch_bounds__(64)
moe_route_softmax_kernel(const float* __restrict__ zin, long ldz, int32_t* __restrict__ idx, float* __restrict__ wt, int E, int top,
                         int groups, int keep, float scale) {
  extern __shared__ float z[];      // [E] scores, then [groups] group scores
  float* gs = z + E;
  const int t = blockIdx.x, lane = threadIdx.x;
  float mx = -INFINITY;
  for (int e = lane; e < E; e += 64) { const float v = zin[(size_t)t * ldz + e]; z[e] = v; mx = fmaxf(mx, v); }
  mx = wave_max(mx);
  float den = 0.f;
  for (int e = lane; e < E; e += 64) { const float p = expf(z[e] - mx); z[e] = p; den += p; }
  den = wave_sum(den);
  for (int e = lane; e < E; e += 64) z[e] = z[e] / den;
  __syncthreads();
  if (groups > 1 && keep < groups) {
    const int per = E / groups;
    for (int g = lane; g < groups; g += 64) {
      float b = -INFINITY;
      for (int i = 0; i < per; ++i) b = fmaxf(b, z[g * per + i]);
      gs[g] = b;
    }
    __syncthreads();
    // `keep` rounds of a wave-wide argmax over the groups; a kept group is marked by a score of +inf
    for (int j = 0; j < keep; ++j) {
      float best = -INFINITY; int bi = 0x7fffffff;
      for (int g = lane; g < groups; g += 64) { const float v = gs[g]; if (v != INFINITY && v > best) { best = v; bi = g; } }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64); const int oi = __shfl_xor(bi, o, 64);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
      }
      if (lane == 0 && bi != 0x7fffffff) gs[bi] = INFINITY;
      __syncthreads();
    }
    for (int e = lane; e < E; e += 64) if (gs[e / per] != INFINITY) z[e] = -1.0f;       // not eligible (scores are >= 0)
    __syncthreads();
  }
  float sum = 0.f, myval = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY; int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) { const float v = z[e]; if (v > best) { best = v; bi = e; } }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64); const int oi = __shfl_xor(bi, o, 64);
      if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    sum += best;
    if (lane == j % 64) { myval = best; idx[(size_t)t * top + j] = bi; }
    if (lane == 0) z[bi] = -2.0f;
    __syncthreads();
  }
  if (lane < top) wt[(size_t)t * top + lane] = myval / (sum + 1e-20f) * scale;
}

// Sigmoid routing: scores = sigmoid(logits), the `top` largest (lowest index wins a tie), weights = the chosen scores as they are
// (no renormalisation).  One wave per token; logits row stride ldz.
__global__ void __launch_bounds__(64)
moe_route_sigmoid_kernel(const float* __restrict__ zin, long ldz, int32_t* __restrict__ idx, float* __restrict__ wt, int E, int top) {
  extern __shared__ float z[];      // [E] scores
  const int t = blockIdx.x, lane = threadIdx.x;
  for (int e = lane; e < E; e += 64) z[e] = 1.0f / (1.0f + expf(-zin[(size_t)t * ldz + e]));
  __syncthreads();
  float myval = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY; int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) { const float v = z[e]; if (v > best) { best = v; bi = e; } }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64); const int oi = __shfl_xor(bi, o, 64);
      if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if (lane == j % 64) { myval = best; idx[(size_t)t * top + j] = bi; }
    if (lane == 0) z[bi] = -1.0f;      // scores are >= 0
    __syncthreads();
  }
  if (lane < top) wt[(size_t)t * top + lane] = myval;
}

// Sigmoid routing with a choice correction and group-limited choice.  One wave per token.  Choice scores may be negative, so an
// expert that cannot be chosen is marked by -inf (never by a finite number).  Among equal values the lowest index wins.
constexpr int MOE_MAX_GROUP_TOP = 8;

__global__ void __launch_bounds__(64)
moe_route_sigmoid_grouped_kernel(const float* __restrict__ zin, long ldz, const float* __restrict__ corr, int32_t* __restrict__ idx,
                                 float* __restrict__ wt, int E, int top, int groups, int keep, int group_top) {
  extern __shared__ float z[];      // [E] scores, [E] choice scores, [groups] group scores
  float* ch = z + E;
  float* gs = ch + E;
  const int t = blockIdx.x, lane = threadIdx.x;
  for (int e = lane; e < E; e += 64) {
    const float sc = 1.0f / (1.0f + expf(-zin[(size_t)t * ldz + e]));
    z[e] = sc;
    ch[e] = sc + (corr ? corr[e] : 0.f);
  }
  __syncthreads();
  if (groups > 1 && keep < groups) {
    const int per = E / groups;
    for (int g = lane; g < groups; g += 64) {
      int taken[MOE_MAX_GROUP_TOP];
      float sum = 0.f;
      for (int j = 0; j < group_top && j < per; ++j) {
        float b = -INFINITY; int bi = -1;
        for (int i = 0; i < per; ++i) {
          bool used = false;
          for (int q = 0; q < j; ++q) used |= taken[q] == i;
          const float v = ch[g * per + i];
          if (!used && (bi < 0 || v > b)) { b = v; bi = i; }
        }
        taken[j] = bi;
        sum += b;
      }
      gs[g] = sum;
    }
    __syncthreads();
    // `keep` rounds of a wave-wide argmax over the groups; a kept group is marked by +inf
    for (int j = 0; j < keep; ++j) {
      float best = -INFINITY; int bi = 0x7fffffff;
      for (int g = lane; g < groups; g += 64) { const float v = gs[g]; if (v != INFINITY && (bi == 0x7fffffff || v > best)) { best = v; bi = g; } }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64); const int oi = __shfl_xor(bi, o, 64);
        if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > best || (ov == best && oi < bi))) { best = ov; bi = oi; }
      }
      if (lane == 0 && bi != 0x7fffffff) gs[bi] = INFINITY;
      __syncthreads();
    }
    for (int e = lane; e < E; e += 64) if (gs[e / per] != INFINITY) ch[e] = -INFINITY;
    __syncthreads();
  }
  float myval = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY; int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) { const float v = ch[e]; if (v > best) { best = v; bi = e; } }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64); const int oi = __shfl_xor(bi, o, 64);
      if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if (bi == 0x7fffffff) bi = 0;       // (unreachable for finite logits: top <= eligible experts)
    if (lane == j % 64) { myval = z[bi]; idx[(size_t)t * top + j] = bi; }
    __syncthreads();
    if (lane == 0) ch[bi] = -INFINITY;
    __syncthreads();
  }
  if (lane < top) wt[(size_t)t * top + lane] = myval;
}

__global__ void __launch_bounds__(1024)
moe_plan_kernel(const int32_t* __restrict__ idx, int n, int E, int32_t* __restrict__ offsets, int32_t* __restrict__ perm,
                int32_t* __restrict__ inv) {
  extern __shared__ int cnt[];      // [E] counts, then cursors
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) atomicAdd(&cnt[idx[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) { const int c = cnt[e]; offsets[e] = run; cnt[e] = run; run += c; }
    offsets[E] = run;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int pos = atomicAdd(&cnt[idx[i]], 1);
    perm[pos] = i;
    inv[i] = pos;
  }
}

__global__ void __launch_bounds__(256)
moe_combine_kernel(const float* __restrict__ y, const int32_t* __restrict__ inv, const float* __restrict__ wt,
                   const float* __restrict__ shared, float* __restrict__ out, int top, int W) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += 256) {
    float s = 0.f;
    for (int j = 0; j < top; ++j) s = fmaf(wt[(size_t)t * top + j], y[(size_t)inv[(size_t)t * top + j] * W + c], s);
    if (shared) s += shared[(size_t)t * W + c];
    out[(size_t)t * W + c] = s;
  }
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_moe_route(const float* logits, int32_t* idx, float* weights, int T, int E, int top, void* stream) {
  if (!logits || !idx || !weights) return SSD_ERR_ARG;
  if (T <= 0 || E <= 0 || E > MOE_MAX_E || top <= 0 || top > E || top > MOE_MAX_TOP) return SSD_ERR_SHAPE;
  hipLaunchKernelGGL(moe_route_kernel, dim3(T), dim3(64), E * sizeof(float), (hipStream_t)stream, logits, idx, weights, E, top);
  return LAUNCH_OK();
}

extern "C" int ssd_moe_route_softmax(const float* logits, long ld, int32_t* idx, float* weights, int T, int E, int top, int groups,
                                     int keep, float scale, void* stream) {
  if (!logits || !idx || !weights) return SSD_ERR_ARG;
  if (T <= 0 || E <= 0 || E > MOE_MAX_E || top <= 0 || top > MOE_MAX_TOP || ld < E || groups <= 0 || E % groups || keep <= 0 ||
      keep > groups || top > (E / groups) * keep)
    return SSD_ERR_SHAPE;
  hipLaunchKernelGGL(moe_route_softmax_kernel, dim3(T), dim3(64), (E + groups) * sizeof(float), (hipStream_t)stream, logits, ld, idx,
                     weights, E, top, groups, keep, scale);
  return LAUNCH_OK();
}

extern "C" int ssd_moe_route_sigmoid(const float* logits, long ld, int32_t* idx, float* weights, int T, int E, int top, void* stream) {
  if (!logits || !idx || !weights) return SSD_ERR_ARG;
  if (T <= 0 || E <= 0 || E > MOE_MAX_E || top <= 0 || top > E || top > MOE_MAX_TOP || ld < E) return SSD_ERR_SHAPE;
  hipLaunchKernelGGL(moe_route_sigmoid_kernel, dim3(T), dim3(64), E * sizeof(float), (hipStream_t)stream, logits, ld, idx, weights, E, top);
  return LAUNCH_OK();
}

extern "C" int ssd_moe_route_sigmoid_grouped(const float* logits, long ld, const float* correction, int32_t* idx, float* weights, int T,
                                             int E, int top, int groups, int keep, int group_top, void* stream) {
  if (!logits || !idx || !weights) return SSD_ERR_ARG;
  if (T <= 0 || E <= 0 || E > MOE_MAX_E || top <= 0 || top > MOE_MAX_TOP || ld < E || groups <= 0 || E % groups || keep <= 0 ||
      keep > groups || top > (E / groups) * keep || group_top <= 0 || group_top > MOE_MAX_GROUP_TOP)
    return SSD_ERR_SHAPE;
  hipLaunchKernelGGL(moe_route_sigmoid_grouped_kernel, dim3(T), dim3(64), (2 * E + groups) * sizeof(float), (hipStream_t)stream, logits,
                     ld, correction, idx, weights, E, top, groups, keep, group_top);
  return LAUNCH_OK();
}

extern "C" int ssd_moe_plan(const int32_t* idx, int T, int top, int E, int32_t* offsets, int32_t* perm, int32_t* inv, void* stream) {
  if (!idx || !offsets || !perm || !inv) return SSD_ERR_ARG;
  if (T <= 0 || top <= 0 || E <= 0 || E > MOE_MAX_E) return SSD_ERR_SHAPE;
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), E * sizeof(int), (hipStream_t)stream, idx, T * top, E, offsets, perm, inv);
  return LAUNCH_OK();
}

extern "C" int ssd_moe_combine(const void* y_rows, const int32_t* inv, const float* weights, const void* shared_rows, void* out_rows,
                               int T, int top, int W, void* stream) {
  if (!y_rows || !inv || !weights || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || top <= 0 || W <= 0) return SSD_ERR_SHAPE;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)y_rows, inv, weights,
                     (const float*)shared_rows, (float*)out_rows, top, W);
  return LAUNCH_OK();
}
