// int4 group-quantised linear layers for decode: y = x . dequant(Wq, s), with the
// LoRA projection t = x . A computed by extra tiles of the same launch.
//
// Replaces the qwix-wrapped einsum / dot_general of the reference
// (tunix/models/llama3/model.py:216-218 Einsum.__call__, :461-487 nnx.Linear;
// tunix/models/qwen3/model.py:389-393, :1163-1197) for T = 1.
//
// Mapping to CDNA4: weights are the B operand of v_mfma_f32_32x32x16_bf16.  The
// packed tile format stores, for every 64(k) x 32(n) tile, the 32 nibbles a lane
// needs as ONE 128-bit word, so a wave fetches a tile with a single coalesced
// 1 KiB load and never touches LDS for weights.  Nibbles are widened with
// v_cvt_f32_ubyteN, scaled with one fma ((u - 8) * s is exact in f32) and
// rounded pairwise to bf16 by the hardware converter, which reproduces the
// reference's bf16 dequantised weight bit for bit before it enters the MFMA.
#include "tmx_kernels.h"

namespace tmx {

// Expand one 32-bit word (8 nibbles, element j = 2 (i % 4) + i / 4 for nibble i)
// into the 8 bf16 B-operand values of one MFMA step: bf16((u - 8) * s).
__device__ __forceinline__ bf16x8_t dequant_word(uint32_t d, float s, float m8s) {
  const uint32_t lo = d & 0x0F0F0F0Fu;         // nibbles 0,2,4,6 in bytes 0..3
  const uint32_t hi = (d >> 4) & 0x0F0F0F0Fu;  // nibbles 1,3,5,7 in bytes 0..3
  // nibble i: byte i/2 of (i even ? lo : hi)
  const float n0 = (float)(lo & 0xFF), n1 = (float)(hi & 0xFF);
  const float n2 = (float)((lo >> 8) & 0xFF), n3 = (float)((hi >> 8) & 0xFF);
  const float n4 = (float)((lo >> 16) & 0xFF), n5 = (float)((hi >> 16) & 0xFF);
  const float n6 = (float)(lo >> 24), n7 = (float)(hi >> 24);
  // register p holds elements j = 2p, 2p + 1  <->  nibbles p, p + 4
  uint32_t p[4];
  p[0] = pack_bf2(fmaf(n0, s, m8s), fmaf(n4, s, m8s));
  p[1] = pack_bf2(fmaf(n1, s, m8s), fmaf(n5, s, m8s));
  p[2] = pack_bf2(fmaf(n2, s, m8s), fmaf(n6, s, m8s));
  p[3] = pack_bf2(fmaf(n3, s, m8s), fmaf(n7, s, m8s));
  bf16x8_t b;
  __builtin_memcpy(&b, p, 16);
  return b;
}


// One workgroup = 4 waves owns NSUB adjacent 32-column tiles over the whole K;
// the waves take k-tiles round-robin (their loads form one contiguous 4 KiB
// stream per column tile) and the partial accumulators meet in LDS.
template <int MT, int NSUB>
__global__ __launch_bounds__(256) void qlinear_mfma_kernel(QLinearArgs a) {
  extern __shared__ float red[];  // [4][NSUB*MT*16][64]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int h = lane >> 5, nl = lane & 31;
  const int KT = a.K >> 6;
  const bool lora_block = (int)blockIdx.x >= a.n_main_blocks;
  constexpr int NS = NSUB;

  f32x16_t acc[NS][MT];
#pragma unroll
  for (int s = 0; s < NS; ++s)
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[s][m][r] = 0.f;

  const uint16_t* xrow[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    int row = m * 32 + nl;
    row = row < a.M ? row : a.M - 1;
    xrow[m] = a.x + (size_t)row * a.ldx + h * 8;
  }

  if (!lora_block) {
    const int nb0 = blockIdx.x * NS;
    const int kpg = a.G >> 6;  // k-tiles per scale group
    const int KG = a.K / a.G;
#pragma unroll 2
    for (int kb = wave; kb < KT; kb += 4) {
      uint4 w[NS];
      float s[NS];
#pragma unroll
      for (int sub = 0; sub < NS; ++sub) {
        w[sub] = a.qw[((size_t)(nb0 + sub) * KT + kb) * 64 + lane];
        s[sub] = bf2f(a.scales[((size_t)(nb0 + sub) * KG + kb / kpg) * 32 + nl]);
      }
      bf16x8_t xa[MT][4];
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int t = 0; t < 4; ++t)
          xa[m][t] = *reinterpret_cast<const bf16x8_t*>(xrow[m] + kb * 64 + t * 16);
#pragma unroll
      for (int sub = 0; sub < NS; ++sub) {
        const float m8s = -8.f * s[sub];
        const uint32_t wd[4] = {w[sub].x, w[sub].y, w[sub].z, w[sub].w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const bf16x8_t b = dequant_word(wd[t], s[sub], m8s);
#pragma unroll
          for (int m = 0; m < MT; ++m)
            acc[sub][m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[m][t], b, acc[sub][m], 0, 0, 0);
        }
      }
    }
  } else {
    // LoRA A tile: dense bf16 columns c of A^T [Rpad, K]; only sub-tile 0 is used.
    const int ct = blockIdx.x - a.n_main_blocks;
    const uint16_t* arow = a.a_t + (size_t)(ct * 32 + nl) * a.K + h * 8;
#pragma unroll 2
    for (int kb = wave; kb < KT; kb += 4) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const bf16x8_t b = *reinterpret_cast<const bf16x8_t*>(arow + kb * 64 + t * 16);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const bf16x8_t xv = *reinterpret_cast<const bf16x8_t*>(xrow[m] + kb * 64 + t * 16);
          acc[0][m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xv, b, acc[0][m], 0, 0, 0);
        }
      }
    }
  }

  // Cross-wave reduction through LDS, then a coalesced bf16 store.
  constexpr int NIDX = NS * MT * 16;
#pragma unroll
  for (int sub = 0; sub < NS; ++sub)
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        red[((size_t)wave * NIDX + (sub * MT + m) * 16 + r) * 64 + lane] = acc[sub][m][r];
  __syncthreads();
  const int nsub_used = lora_block ? 1 : NS;
  for (int e = threadIdx.x; e < NIDX * 64; e += 256) {
    const int idx = e >> 6, ln = e & 63;
    const int sub = idx / (MT * 16), m = (idx / 16) % MT, r = idx & 15;
    if (sub >= nsub_used) continue;
    const float v = red[(size_t)idx * 64 + ln] + red[((size_t)NIDX + idx) * 64 + ln] +
                    red[((size_t)2 * NIDX + idx) * 64 + ln] + red[((size_t)3 * NIDX + idx) * 64 + ln];
    const int row = m * 32 + acc_row(r, ln);
    if (row >= a.M) continue;
    if (!lora_block) {
      const int col = (blockIdx.x * NS + sub) * 32 + (ln & 31);
      a.y[(size_t)row * a.ldy + col] = f2bf(v);
    } else {
      const int col = (blockIdx.x - a.n_main_blocks) * 32 + (ln & 31);
      a.t[(size_t)row * a.ldt + col] = f2bf(v);
    }
  }
}

template <int MT, int NSUB>
static int launch_qlinear(hipStream_t st, QLinearArgs a) {
  a.n_main_blocks = a.N / (32 * NSUB);
  const int blocks = a.n_main_blocks + (a.a_t ? a.Rpad / 32 : 0);
  const size_t lds = (size_t)4 * NSUB * MT * 16 * 64 * sizeof(float);
  hipLaunchKernelGGL((qlinear_mfma_kernel<MT, NSUB>), dim3(blocks), dim3(256), lds, st, a);
  return check_launch();
}

// Host-side dispatch shared by the C entry point and the decode-step launcher.
int qlinear_base(hipStream_t st, const void* x, int ldx, const void* qw, const void* scales,
                 const void* a_t, void* y, int ldy, void* t, int ldt, int M, int K, int N, int G,
                 int Rpad) {
  if (!x || !qw || !scales || !y) return TMX_ERR_ARG;
  if (M <= 0 || K <= 0 || N <= 0) return TMX_ERR_SHAPE;
  if (K % 64 || N % 32 || G % 64 || K % G || (ldx % 8)) return TMX_ERR_SHAPE;
  if (a_t && (!t || Rpad <= 0 || Rpad % 32)) return TMX_ERR_SHAPE;
  for (int m0 = 0; m0 < M; m0 += 128) {
    const int mc = (M - m0) < 128 ? (M - m0) : 128;
    QLinearArgs a;
    a.x = (const uint16_t*)x + (size_t)m0 * ldx;
    a.ldx = ldx;
    a.qw = (const uint4*)qw;
    a.scales = (const uint16_t*)scales;
    a.a_t = (const uint16_t*)a_t;
    a.y = (uint16_t*)y + (size_t)m0 * ldy;
    a.ldy = ldy;
    a.t = t ? (uint16_t*)t + (size_t)m0 * ldt : nullptr;
    a.ldt = ldt;
    a.M = mc; a.K = K; a.N = N; a.G = G; a.Rpad = Rpad;
    int rc;
    const bool wide = (N % 64 == 0) && (N / 64 >= 384);
    if (mc <= 32) rc = wide ? launch_qlinear<1, 2>(st, a) : launch_qlinear<1, 1>(st, a);
    else if (mc <= 64) rc = wide ? launch_qlinear<2, 2>(st, a) : launch_qlinear<2, 1>(st, a);
    else rc = launch_qlinear<4, 1>(st, a);
    if (rc != TMX_OK) return rc;
  }
  return TMX_OK;
}

// ---------------------------------------------------------------------------
// Bit-exact dequantisation to a dense bf16 [K, N] matrix (checker / fallback for
// callers that want the reference's materialised weight).
__global__ __launch_bounds__(256) void int4_dequant_kernel(const uint4* qw, const uint16_t* scales,
                                                           uint16_t* w, int K, int N, int G) {
  const int lane = threadIdx.x & 63;
  const int tile = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int KT = K >> 6, NT = N >> 5;
  if (tile >= KT * NT) return;
  const int nb = tile / KT, kb = tile % KT;
  const int h = lane >> 5, nl = lane & 31;
  const uint4 q = qw[(size_t)tile * 64 + lane];
  const float s = bf2f(scales[((size_t)nb * (K / G) + (kb * 64) / G) * 32 + nl]);
  const uint32_t wd[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const bf16x8_t b = dequant_word(wd[t], s, -8.f * s);
    uint16_t e[8];
    __builtin_memcpy(e, &b, 16);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = kb * 64 + t * 16 + h * 8 + j;
      w[(size_t)k * N + nb * 32 + nl] = e[j];
    }
  }
}

// y[m][n] <- bf16( y + bf16( bf16(sum_r t[m][r] B[r][n]) * ls ) ) (+ residual).
// Rounding points follow the reference's bf16 einsum -> scale -> add chain.
__global__ __launch_bounds__(256) void lora_apply_kernel(uint16_t* y, int ldy, const uint16_t* t,
                                                         int ldt, const uint16_t* b, int r, float ls,
                                                         const uint16_t* res, int ldres, int M, int N) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  const int m = blockIdx.y;
  if (n >= N) return;
  float v = bf2f(y[(size_t)m * ldy + n]);
  if (t) {
    float d = 0.f;
    for (int rr = 0; rr < r; ++rr) d = fmaf(bf2f(t[(size_t)m * ldt + rr]), bf2f(b[(size_t)rr * N + n]), d);
    v = rbf(v + rbf(rbf(d) * ls));
  }
  if (res) v = rbf(v + bf2f(res[(size_t)m * ldres + n]));
  y[(size_t)m * ldy + n] = f2bf(v);
}

}  // namespace tmx

using namespace tmx;

extern "C" int tmx_int4_dequant(void* stream, const void* qweight, const void* scales, void* w_out,
                                int K, int N, int G) {
  if (!qweight || !scales || !w_out) return TMX_ERR_ARG;
  if (K <= 0 || N <= 0 || K % 64 || N % 32 || G % 64 || K % G) return TMX_ERR_SHAPE;
  const int tiles = (K / 64) * (N / 32);
  hipLaunchKernelGGL(int4_dequant_kernel, dim3((tiles + 3) / 4), dim3(256), 0, (hipStream_t)stream,
                     (const uint4*)qweight, (const uint16_t*)scales, (uint16_t*)w_out, K, N, G);
  return check_launch();
}

extern "C" int tmx_qlora_linear(void* stream, const void* x, const void* qweight, const void* scales,
                                const void* lora_a_t, const void* lora_b, const void* residual,
                                void* y, void* t_ws, int M, int K, int N, int G, int r, int r_pad,
                                float lora_scale) {
  hipStream_t st = (hipStream_t)stream;
  const bool lora = lora_a_t != nullptr;
  if (lora && (!lora_b || !t_ws || r <= 0 || r > r_pad)) return TMX_ERR_ARG;
  int rc = qlinear_base(st, x, K, qweight, scales, lora ? lora_a_t : nullptr, y, N, t_ws, r_pad, M, K, N,
                        G, r_pad);
  if (rc != TMX_OK) return rc;
  if (lora || residual) {
    hipLaunchKernelGGL(lora_apply_kernel, dim3((N + 255) / 256, M), dim3(256), 0, st, (uint16_t*)y, N,
                       lora ? (const uint16_t*)t_ws : nullptr, r_pad, (const uint16_t*)lora_b, r,
                       lora_scale, (const uint16_t*)residual, N, M, N);
    rc = check_launch();
  }
  return rc;
}
