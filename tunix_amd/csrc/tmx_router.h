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
  float* part = prob + a.E;  // [kRowGroups][E]
  {
    // [D, E]: 16 threads cover 128 expert columns of one router row with 16-byte loads (8 experts
    // each), kRowGroups rows per pass; partial sums over the row groups meet in LDS
    for (int e0 = 0; e0 < a.E; e0 += 128) {
      const int eg = (tid & 15) * 8 + e0, dsub = tid >> 4;
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (eg < a.E) {
        // 16 router rows in flight per thread; rows past D are clamped and weighted by zero.  The loop is bound by
        // what one CU can pull from L2: D * E * 2 bytes per token (512 KB at 2048 x 128, 3.5 us measured, 3.9 us at
        // 64 bytes per clock); the transposed matrix with two products per instruction measured the same
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
  }
  // softmax by the first wave alone (E / 64 values per lane; the sums run over the experts in the same fixed
  // order on every call)
  if (wave == 0) {
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
  }
  __syncthreads();
  // top-k by rank: expert e comes after every expert with a larger probability and after the equal ones with a
  // lower id (lax.top_k's order), so its place is the count of those; one thread per expert counts over all
  // probabilities (broadcast reads) -- no round depends on the one before, as k repeated arg-max searches would
  float* sel = part;  // [top_k] the chosen probabilities by place (the partial scores are spent)
  for (int e = tid; e < a.E; e += kRouterThreads) {
    const float v = prob[e];
    int place = 0;
    for (int j = 0; j < a.E; j += 4) {
      const float4 u = *reinterpret_cast<const float4*>(prob + j);
      place += (u.x > v || (u.x == v && j < e)) ? 1 : 0;
      place += (u.y > v || (u.y == v && j + 1 < e)) ? 1 : 0;
      place += (u.z > v || (u.z == v && j + 2 < e)) ? 1 : 0;
      place += (u.w > v || (u.w == v && j + 3 < e)) ? 1 : 0;
    }
    if (place < a.top_k) {
      a.expert_of[(size_t)b * a.top_k + place] = e;
      sel[place] = v;
    }
  }
  __syncthreads();
  if (tid < a.top_k) {
    float wsum = 0.f;
    for (int j = 0; j < a.top_k; ++j) wsum += sel[j];  // in the order of the places
    a.weight_of[(size_t)b * a.top_k + tid] = rbf(sel[tid] / wsum);
  }
}

}  // namespace tmx
