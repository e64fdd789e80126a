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

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
// Sum over aligned groups of LPP (8 or 16) lanes; every lane gets the total.
template <int LPP>
__device__ __forceinline__ float group_sum(float v) {
  v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f<0x141>(v);  // row_half_mirror
  if (LPP == 16) v += dpp_f<0x140>(v);  // row_mirror
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

// The same expansion in four parts, for loops that spread the dequantisation between MFMAs:
// dequant_masks() once per word, then register p of the B operand (elements 2p, 2p + 1 =
// nibbles p, p + 4) from dequant_part<p>().  Bit-identical to dequant_word().
__device__ __forceinline__ void dequant_masks(uint32_t d, uint32_t& lo, uint32_t& hi) {
  lo = d & 0x0F0F0F0Fu;
  hi = (d >> 4) & 0x0F0F0F0Fu;
  asm volatile("" : "+v"(lo), "+v"(hi));
}
template <int P>
__device__ __forceinline__ uint32_t dequant_part(uint32_t lo, uint32_t hi, float s, float m8s);

// A byte 0x0U read as an fp8 number (E4M3, bias 7) is U * 2^-9 for every U in 0..15: below 8 it is subnormal
// (U / 8 * 2^-6), from 8 on its exponent field is 1 ((1 + (U - 8) / 8) * 2^-6).  So one v_cvt_pk_f32_fp8 widens
// two nibbles of a masked word at once, where v_cvt_f32_ubyteN takes one instruction per nibble; the factor
// 2^9 goes into the scale (exact).  w: a word of four bytes 0x0U; returns the floats of bytes (0, 1) or (2, 3).
typedef float f32x2_t __attribute__((ext_vector_type(2)));
template <bool HIGH>
__device__ __forceinline__ f32x2_t nibble_pair_f32(uint32_t w) {
  return __builtin_amdgcn_cvt_pk_f32_fp8((int)w, HIGH);
}
constexpr float kNibbleUnit = 512.f;  // 1 / (2^-9)

// Expand one 32-bit word (8 nibbles, element j = 2 (i % 4) + i / 4 for nibble i)
// into the 8 bf16 B-operand values of one MFMA step: bf16((u - 8) * s).
// PAIRS = false: fma(u, s, -8 s) with u widened by v_cvt_f32_ubyteN, one instruction per nibble.
// PAIRS = true: fma(u * 2^-9, s * 2^9, -8 s) with two nibbles widened per v_cvt_pk_f32_fp8 (19 instead of 23
// instructions per word).  Both are (u - 8) * s exactly (4 + 8 significant bits), rounded once to bf16.  The pair
// form pays where the loop is bound by these instructions (the fused gate|up launch -3 %, the expert stream -2 %,
// the 1..4-row projections -2 % of their step);
// in the loops bound by the matrix pipe it measured slower (128-row projections +1.6 % on the step), so they
// keep the byte form.
template <bool PAIRS = false>
__device__ __forceinline__ bf16x8_t dequant_word(uint32_t d, float s, float m8s) {
  uint32_t lo = d & 0x0F0F0F0Fu;         // nibbles 0,2,4,6 in bytes 0..3
  uint32_t hi = (d >> 4) & 0x0F0F0F0Fu;  // nibbles 1,3,5,7 in bytes 0..3
  // register p holds elements j = 2p, 2p + 1  <->  nibbles p, p + 4
  uint32_t p[4];
  if constexpr (PAIRS) {
    const float s9 = s * kNibbleUnit;
    const f32x2_t a = nibble_pair_f32<false>(lo), b = nibble_pair_f32<true>(lo);  // nibbles (0, 2), (4, 6)
    const f32x2_t c = nibble_pair_f32<false>(hi), e = nibble_pair_f32<true>(hi);  // nibbles (1, 3), (5, 7)
    p[0] = pack_bf2(fmaf(a.x, s9, m8s), fmaf(b.x, s9, m8s));
    p[1] = pack_bf2(fmaf(c.x, s9, m8s), fmaf(e.x, s9, m8s));
    p[2] = pack_bf2(fmaf(a.y, s9, m8s), fmaf(b.y, s9, m8s));
    p[3] = pack_bf2(fmaf(c.y, s9, m8s), fmaf(e.y, s9, m8s));
  } else {
    // keep the two masked words opaque so that each byte is widened by one
    // v_cvt_f32_ubyteN instead of a bit-field extract plus a conversion
    asm volatile("" : "+v"(lo), "+v"(hi));
    // nibble i: byte i/2 of (i even ? lo : hi)
    const float n0 = (float)(lo & 0xFF), n1 = (float)(hi & 0xFF);
    const float n2 = (float)((lo >> 8) & 0xFF), n3 = (float)((hi >> 8) & 0xFF);
    const float n4 = (float)((lo >> 16) & 0xFF), n5 = (float)((hi >> 16) & 0xFF);
    const float n6 = (float)(lo >> 24), n7 = (float)(hi >> 24);
    p[0] = pack_bf2(fmaf(n0, s, m8s), fmaf(n4, s, m8s));
    p[1] = pack_bf2(fmaf(n1, s, m8s), fmaf(n5, s, m8s));
    p[2] = pack_bf2(fmaf(n2, s, m8s), fmaf(n6, s, m8s));
    p[3] = pack_bf2(fmaf(n3, s, m8s), fmaf(n7, s, m8s));
  }
  bf16x8_t r;
  __builtin_memcpy(&r, p, 16);
  return r;
}

template <int P>
__device__ __forceinline__ uint32_t dequant_part(uint32_t lo, uint32_t hi, float s, float m8s) {
  const uint32_t w = (P & 1) ? hi : lo;  // nibbles P and P + 4: bytes P / 2 and P / 2 + 2 of that word
  const float a = (float)((w >> (8 * (P / 2))) & 0xFF), b = (float)((w >> (8 * (P / 2) + 16)) & 0xFF);
  return pack_bf2(fmaf(a, s, m8s), fmaf(b, s, m8s));
}


template <int V>
struct IC { static constexpr int value = V; };

// f(IC<0>{}), ..., f(IC<N - 1>{}): a loop whose index is a compile-time constant
template <int N, int I = 0, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(IC<I>{});
    static_for<N, I + 1>(f);
  }
}

// Raw buffer descriptor over `bytes` bytes at p (loads take a per-lane and a scalar byte offset).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// 1 KiB from global memory straight into LDS (buffer_load ... lds): lane i's 16 bytes at byte
// offset voffset + soffset of the buffer land at dst + 16 i; dst and soffset are wave-uniform.
// Counted by vmcnt like any other load.
__device__ __forceinline__ void load_row_to_lds(__amdgpu_buffer_rsrc_t r, void* dst, int voffset, int soffset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)dst, 16, voffset, soffset, 0, 0);
}
// the same with the non-temporal cache policy, for data that is read once
__device__ __forceinline__ void load_row_to_lds_nt(__amdgpu_buffer_rsrc_t r, void* dst, int voffset, int soffset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)dst, 16, voffset, soffset, 0, 2);
}


inline int check_launch() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TMX_OK : TMX_ERR_LAUNCH;
}

}  // namespace tmx
