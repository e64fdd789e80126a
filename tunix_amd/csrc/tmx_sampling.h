// Device helpers shared by the token-selection kernels: threefry2x32 counter-based random
// bits (the generator behind jax.random), Gumbel noise, and the merge rules for running
// (max, sum-exp) pairs and arg-best candidates.
#pragma once
#include "tmx_common.h"

namespace tmx {

__device__ __forceinline__ uint32_t rotl32(uint32_t x, int r) { return (x << r) | (x >> (32 - r)); }

__device__ __forceinline__ void threefry2x32(uint32_t k0, uint32_t k1, uint32_t c0, uint32_t c1,
                                             uint32_t& o0, uint32_t& o1) {
  const uint32_t ks[3] = {k0, k1, k0 ^ k1 ^ 0x1BD11BDAu};
  uint32_t x0 = c0 + ks[0], x1 = c1 + ks[1];
  const int rot[2][4] = {{13, 15, 26, 6}, {17, 29, 16, 24}};
#pragma unroll
  for (int g = 0; g < 5; ++g) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x0 += x1;
      x1 = rotl32(x1, rot[g & 1][i]);
      x1 ^= x0;
    }
    x0 += ks[(g + 1) % 3];
    x1 += ks[(g + 2) % 3] + (uint32_t)(g + 1);
  }
  o0 = x0;
  o1 = x1;
}

__device__ __forceinline__ float gumbel_from_bits(uint32_t bits) {
  const float tiny = 1.17549435e-38f;
  float f = __uint_as_float((bits >> 9) | 0x3F800000u) - 1.0f;
  f = fmaxf(tiny, f + tiny);
  return -logf(-logf(f));
}

struct Best {
  float key;  // z + gumbel (or raw logit for greedy)
  float z;
  int idx;
};
__device__ __forceinline__ void best_merge(Best& a, const Best& b) {
  if (b.key > a.key || (b.key == a.key && b.idx < a.idx)) a = b;
}
// (mx, se) <- merge with (mx2, se2): running max and sum of exp(z - max)
__device__ __forceinline__ void lse_merge(float& mx, float& se, float mx2, float se2) {
  const float mn = fmaxf(mx, mx2);
  se = se * expf(mx - mn) + se2 * expf(mx2 - mn);
  mx = mn;
}


constexpr float kNegBig = -3.0e38f;

}  // namespace tmx
