// Device-side helpers shared by the gfx950 kernels: bf16 bit handling, wave64
// reductions, MFMA fragment types and the status codes of the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tmx.h"

namespace tmx {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr float kMask = -2.3819763e38f;  // the reference's K_MASK

__device__ __forceinline__ float bf2f(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}
__device__ __forceinline__ float bf_lo(uint32_t p) { return __uint_as_float(p << 16); }
__device__ __forceinline__ float bf_hi(uint32_t p) { return __uint_as_float(p & 0xFFFF0000u); }

// float -> bf16, round to nearest even (hardware conversion on gfx950).
__device__ __forceinline__ uint16_t f2bf(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}
// Round a float to the nearest bf16 and return it widened again.
__device__ __forceinline__ float rbf(float f) { return bf2f(f2bf(f)); }

__device__ __forceinline__ uint32_t pack_bf2(float lo, float hi) {
  f32x2_t v = {lo, hi};
  bf16x2_t b = __builtin_convertvector(v, bf16x2_t);
  return __builtin_bit_cast(uint32_t, b);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Sum over a workgroup of NW waves; every thread receives the total.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* smem /* >= NW floats */) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) smem[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) t += smem[i];
  return t;
}

// Row of MFMA 32x32 accumulator register r held by `lane` (column = lane % 32).
__device__ __forceinline__ int acc_row(int r, int lane) {
  return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
}

inline int check_launch() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TMX_OK : TMX_ERR_LAUNCH;
}

}  // namespace tmx
