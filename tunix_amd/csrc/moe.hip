// Mixture-of-experts routing for decode (Qwen3 MoE).
//
// Replaces MoELayer.__call__'s routing, tunix/models/qwen3/model.py:895-902:
//   scores = bf16(x . router)  -> f32;  p = softmax(scores)
//   weights, experts = lax.top_k(p, k)        (ties: lower expert id first)
//   weights = bf16(weights / sum(weights))
// One workgroup per token.  The expert matrices themselves are multiplied by
// moe_stream_kernel (qlinear.hip); the weighted sum over a token's experts is taken by the
// row kernel that also adds the residual and normalises (glue.hip).
#include "tmx_router.h"

namespace tmx {

__global__ __launch_bounds__(kRouterThreads) void moe_router_kernel(RouterArgs a) {
  extern __shared__ __align__(16) float sm[];
  const int b = blockIdx.x;
  for (int d = threadIdx.x; d < a.D; d += kRouterThreads) sm[d] = bf2f(a.x[(size_t)b * a.D + d]);
  __syncthreads();
  moe_route_token(a, sm, b);
}

int moe_route(hipStream_t st, const RouterArgs& a, int B) {
  if (!a.x || !a.w || !a.expert_of || !a.weight_of) return TMX_ERR_ARG;
  if (B <= 0 || a.D <= 0 || a.D % 4 || a.E <= 0 || a.E % 8 || a.top_k <= 0 || a.top_k > 64 || a.top_k > a.E)
    return TMX_ERR_SHAPE;
  const size_t lds = moe_router_lds_floats(a.D, a.E) * sizeof(float);
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
