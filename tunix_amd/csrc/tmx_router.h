// Routing of one token by one workgroup of kRouterThreads threads (shared by the stand-alone router kernel
// and the row kernel that produces the router's input).
//
// tunix/models/qwen3/model.py:895-902:
//   scores = bf16(x . router)  -> f32;  p = softmax(scores)
//   weights, experts = lax.top_k(p, k)        (ties: lower expert id first)
//   weights = bf16(weights / sum(weights))
#pragma once
#include "tmx_kernels.h"

namespace tmx {

constexpr int kRouterThreads = 512, kRowGroups = kRouterThreads / 16;

// floats of LDS the routing of a token needs: x row [D] | probabilities [E] | partial scores [kRowGroups][E]
inline size_t moe_router_lds_floats(int D, int E) { return (size_t)D + (size_t)(1 + kRowGroups) * E; }

// sm: moe_router_lds_floats(D, E) floats whose first D hold the token's normed hidden state (bf16 values),
// visible to every thread (the caller has synchronised).  Writes expert_of / weight_of of token b.
__device__ __forceinline__ void moe_route_token(const RouterArgs& a, float* sm, const int b) {
  float* xrow = sm;
  float* prob = sm + a.D;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // scores: 16 threads cover 128 expert columns of one router row with 16-byte loads (8 experts
  // each), kRowGroups rows per pass; partial sums over the row groups meet in LDS
  float* part = prob + a.E;  // [kRowGroups][E]
  for (int e0 = 0; e0 < a.E; e0 += 128) {
    const int eg = (tid & 15) * 8 + e0, dsub = tid >> 4;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (eg < a.E) {
      // 16 router rows in flight per thread (the loop is bound by the latency of these loads);
      // rows past D are clamped and weighted by zero
      for (int d0 = dsub; d0 < a.D; d0 += 16 * kRowGroups) {
        uint4 w8[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const int d = d0 + kRowGroups * u;
          w8[u] = *reinterpret_cast<const uint4*>(a.w + (size_t)(d < a.D ? d : a.D - 1) * a.E + eg);
        }
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const int d = d0 + kRowGroups * u;
          const float xv = d < a.D ? xrow[d] : 0.f;
          const uint32_t ww[4] = {w8[u].x, w8[u].y, w8[u].z, w8[u].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            acc[2 * j] = fmaf(xv, bf_lo(ww[j]), acc[2 * j]);
            acc[2 * j + 1] = fmaf(xv, bf_hi(ww[j]), acc[2 * j + 1]);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) part[dsub * a.E + eg + j] = acc[j];
    }
  }
  __syncthreads();
  for (int e = tid; e < a.E; e += kRouterThreads) {
    float s = 0.f;
#pragma unroll
    for (int g = 0; g < kRowGroups; ++g) s += part[g * a.E + e];
    prob[e] = rbf(s);
  }
  __syncthreads();
  // softmax and top-k by the first wave alone (E / 64 values per lane): no barriers between
  // the k rounds.  Sums run over the experts in the same fixed order on every call.
  if (wave != 0) return;
  float mx = -INFINITY;
  for (int e = lane; e < a.E; e += 64) mx = fmaxf(mx, prob[e]);
  mx = wave_max(mx);
  float se = 0.f;
  for (int e = lane; e < a.E; e += 64) {
    const float ex = expf(prob[e] - mx);
    prob[e] = ex;
    se += ex;
  }
  se = wave_sum(se);
  for (int e = lane; e < a.E; e += 64) prob[e] = prob[e] / se;
  // top-k by repeated arg-max; among equal probabilities the lower expert id wins
  float wsum = 0.f, my_w = 0.f;
  for (int j = 0; j < a.top_k; ++j) {
    float bv = -1.f;
    int bi = 0x7FFFFFFF;
    for (int e = lane; e < a.E; e += 64) {
      const float v = prob[e];
      if (v > bv || (v == bv && e < bi)) { bv = v; bi = e; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (lane == (bi & 63)) prob[bi] = -2.f;  // taken (the owner lane updates its own element)
    if (lane == j) { a.expert_of[(size_t)b * a.top_k + j] = bi; my_w = bv; }
    wsum += bv;
  }
  if (lane < a.top_k) a.weight_of[(size_t)b * a.top_k + lane] = rbf(my_w / wsum);
}

}  // namespace tmx
