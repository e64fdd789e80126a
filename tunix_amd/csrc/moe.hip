// Mixture-of-experts routing for decode (Qwen3 MoE).
//
// Replaces MoELayer.__call__'s routing, tunix/models/qwen3/model.py:895-902:
//   scores = bf16(x . router)  -> f32;  p = softmax(scores)
//   weights, experts = lax.top_k(p, k)        (ties: lower expert id first)
//   weights = bf16(weights / sum(weights))
// One workgroup per token.  The expert matrices themselves are multiplied by
// moe_stream_kernel (qlinear.hip); the weighted sum over a token's experts is taken by the
// row kernel that also adds the residual and normalises (glue.hip).
#include "tmx_kernels.h"

namespace tmx {

constexpr int kRouterThreads = 512, kRowGroups = kRouterThreads / 16;

__global__ __launch_bounds__(kRouterThreads) void moe_router_kernel(RouterArgs a) {
  extern __shared__ float sm[];  // x row [D] | probabilities [E] | partial scores [kRowGroups][E]
  float* xrow = sm;
  float* prob = sm + a.D;
  const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int d = tid; d < a.D; d += kRouterThreads) xrow[d] = bf2f(a.x[(size_t)b * a.D + d]);
  __syncthreads();
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

int moe_route(hipStream_t st, const RouterArgs& a, int B) {
  if (!a.x || !a.w || !a.expert_of || !a.weight_of) return TMX_ERR_ARG;
  if (B <= 0 || a.D <= 0 || a.E <= 0 || a.E % 8 || a.top_k <= 0 || a.top_k > 64 || a.top_k > a.E)
    return TMX_ERR_SHAPE;
  const size_t lds = (size_t)(a.D + (1 + kRowGroups) * a.E) * sizeof(float);
  if (lds > 60000) return TMX_ERR_SHAPE;
  hipLaunchKernelGGL(moe_router_kernel, dim3(B), dim3(kRouterThreads), lds, st, a);
  return check_launch();
}

}  // namespace tmx

using namespace tmx;

extern "C" int tmx_moe_route(void* stream, const void* x, const void* router_w, int B, int D, int E,
                             int top_k, int32_t* expert_of, float* weight_of) {
  RouterArgs a = {};
  a.x = (const uint16_t*)x;
  a.w = (const uint16_t*)router_w;
  a.D = D; a.E = E; a.top_k = top_k;
  a.expert_of = expert_of;
  a.weight_of = weight_of;
  return moe_route((hipStream_t)stream, a, B);
}

extern "C" int tmx_moe_experts(void* stream, const void* x, int ldx, const void* qweight, const void* scales,
                               const int32_t* expert_of, int P, int top_k, int E, int K, int N, int G,
                               int down, void* out, int ldo) {
  MoeArgs a = {};
  a.x = (const uint16_t*)x;
  a.ldx = ldx;
  a.qw = (const uint4*)qweight;
  a.scales = (const uint16_t*)scales;
  a.qw_stride = (size_t)K * N / 32;            // 16-byte words of one expert's q4t matrix
  a.sc_stride = (size_t)(K / (G > 0 ? G : 1)) * N;
  a.expert_of = expert_of;
  a.P = P; a.top_k = top_k;
  a.K = K; a.N = N; a.G = G;
  a.out = (uint16_t*)out;
  a.ldo = ldo;
  if (G <= 0) return TMX_ERR_SHAPE;
  return moe_experts((hipStream_t)stream, a, E, down != 0);
}
