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
  uint32_t lo = d & 0x0F0F0F0Fu;         // nibbles 0,2,4,6 in bytes 0..3
  uint32_t hi = (d >> 4) & 0x0F0F0F0Fu;  // nibbles 1,3,5,7 in bytes 0..3
  // keep the two masked words opaque so that each byte is widened by one
  // v_cvt_f32_ubyteN instead of a bit-field extract plus a conversion
  asm volatile("" : "+v"(lo), "+v"(hi));
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


// One workgroup = 4 waves owns a block of 4 * NSUB adjacent 32-column tiles (one
// group of NSUB tiles per wave) over one K-slice.  The activation k-tile
// x[0:M, 64 kb : 64 kb + 64] is fetched once per workgroup with coalesced 16-byte
// loads, double-buffered in LDS (rows padded to 144 bytes: conflict-free
// ds_read_b128) and shared by the four waves as MFMA A fragments; weights go
// HBM -> registers.  Global loads of k-tile i+1 are issued before the MFMAs of
// k-tile i.  Small-N projections are split along K over blockIdx.y so that
// every CU streams weights; each split writes its own f32 plane (summed by the
// consumer kernel), so results do not depend on scheduling order.
constexpr int kXStride = 72;  // bf16 elements per LDS row (64 + 8 pad)

template <int V>
struct IC { static constexpr int value = V; };

// LORA = false: NSUB int4 column tiles per wave.  LORA = true: the block computes a K-slice
// of t = x . A from bf16 tiles of A (one 32-column tile per wave); A is stored in MFMA
// B-fragment order, [K/64][Rpad/32][64 lanes][4 steps][8], so a wave reads 4 KiB contiguously.
template <int MT, int NSUB, bool LORA>
__device__ __forceinline__ void gemm_block(const QLinearArgs& a, uint16_t (*xs)[MT * 32][kXStride]) {
  // xs: 2 LDS buffers, buffer b holds activation tile i with i % 2 == b
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int h = lane >> 5, nl = lane & 31;
  const int KT = a.K >> 6;
  // K-slice of this block: main blocks follow blockIdx.y; the LoRA blocks of a launch cut K
  // into lora_splits finer slices of their own so that none of them is the last to finish
  const int slice = LORA ? ((int)blockIdx.x - a.n_main_blocks) + a.lora_blocks_per_split * (int)blockIdx.y
                         : (int)blockIdx.y;
  const int per = LORA ? a.kt_per_lora_split : a.kt_per_split;
  const int kb0 = slice * per;
  const int kb1 = (kb0 + per < KT) ? kb0 + per : KT;
  const int kpg_shift = (a.G == 64) ? 0 : __builtin_ctz(a.G >> 6), KG = a.K / a.G;

  // this wave's column tiles; waves past the last tile recompute the last one (their
  // results are dropped) so that the pipelined loop below stays free of branches
  const int NT = LORA ? (a.Rpad >> 5) : (a.N >> 5);
  const int nb_first = LORA ? wave : ((int)blockIdx.x * 4 + wave) * NSUB;
  int nbs[NSUB];
  bool sub_ok[NSUB];
#pragma unroll
  for (int s = 0; s < NSUB; ++s) {
    sub_ok[s] = (nb_first + s) < NT;
    nbs[s] = sub_ok[s] ? nb_first + s : NT - 1;
  }

  f32x16_t acc[NSUB][MT];
#pragma unroll
  for (int s = 0; s < NSUB; ++s)
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[s][m][r] = 0.f;

  // cooperative activation load: chunk c = tid + 256 i -> row c / 8, 16-byte column c % 8
  const uint16_t* xsrc[MT];
  int xrow_l[MT], xcol_l[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int c = tid + 256 * i;
    xrow_l[i] = c >> 3;
    xcol_l[i] = (c & 7) * 8;
    const int row = xrow_l[i] < a.M ? xrow_l[i] : a.M - 1;
    xsrc[i] = a.x + (size_t)row * a.ldx + xcol_l[i];
  }
  const u32x4_t* wsrc[NSUB];
  const uint16_t* ssrc[NSUB];
  size_t wstep;  // 16-byte words between consecutive k-tiles of one column tile
  if (LORA) {
    wstep = (size_t)NT * 64 * 4;
  } else {
    wstep = 64;
  }
#pragma unroll
  for (int s = 0; s < NSUB; ++s) {
    if (LORA) {
      wsrc[s] = reinterpret_cast<const u32x4_t*>(a.a_t) + ((size_t)nbs[s] * 64 + lane) * 4;
      ssrc[s] = nullptr;
    } else {
      wsrc[s] = reinterpret_cast<const u32x4_t*>(a.qw) + (size_t)nbs[s] * KT * 64 + lane;
      ssrc[s] = a.scales + (size_t)nbs[s] * KG * 32 + nl;
    }
  }

  // weight tiles in flight per wave (HBM latency); 8 where the registers allow two waves per SIMD
  constexpr int PW = (!LORA && NSUB == 1 && MT <= 2) ? 8 : 4;
  constexpr int PX = 4;              // activation tiles in flight (L2 latency)
  constexpr int WPT = LORA ? 4 : 1;  // 16-byte words per lane and tile
  u32x4_t xring[PX][MT];
  u32x4_t wring[PW][NSUB][WPT];
  uint16_t sring[PW][NSUB];
  const int nk = kb1 - kb0;
  if (nk <= 0) return;
  const int klast = kb1 - 1;

  // Unconditional loads with clamped tile indices: the compiler can then count the
  // outstanding loads exactly and wait only for the oldest one.
  auto load_w = [&](int kb, auto pc) __attribute__((always_inline)) {
    constexpr int p = decltype(pc)::value;
    kb = kb < klast ? kb : klast;
#pragma unroll
    for (int s = 0; s < NSUB; ++s) {
      if (LORA) {
#pragma unroll
        for (int t = 0; t < 4; ++t) wring[p][s][t] = wsrc[s][(size_t)kb * wstep + t];
      } else {
        wring[p][s][0] = wsrc[s][(size_t)kb * wstep];
        sring[p][s] = ssrc[s][(size_t)(kb >> kpg_shift) * 32];
      }
    }
  };
  auto load_x = [&](int kb, auto pc) __attribute__((always_inline)) {
    constexpr int p = decltype(pc)::value;
    kb = kb < klast ? kb : klast;
#pragma unroll
    for (int i = 0; i < MT; ++i) xring[p][i] = *reinterpret_cast<const u32x4_t*>(xsrc[i] + kb * 64);
  };
  auto stash_x = [&](int buf, auto pc) __attribute__((always_inline)) {
    constexpr int p = decltype(pc)::value;
#pragma unroll
    for (int i = 0; i < MT; ++i)
      *reinterpret_cast<u32x4_t*>(&xs[buf][xrow_l[i]][xcol_l[i]]) = xring[p][i];
  };
  // one k-tile (tile kb = kb0 + i, weight slot i % PW, activation slot i % PX, LDS buffer
  // i & 1): read the A fragments, consume and refill the weight slot, do the math, publish
  // activation tile kb + 1 to the other buffer
  auto tile_step = [&](int kb, auto ic) __attribute__((always_inline)) {
    constexpr int i = decltype(ic)::value;
    constexpr int pw = i % PW, px1 = (i + 1) % PX;
    bf16x8_t xa[MT][4];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        xa[m][t] = *reinterpret_cast<const bf16x8_t*>(&xs[i & 1][m * 32 + nl][t * 16 + h * 8]);
    u32x4_t wc[NSUB][WPT];
    float s_c[NSUB];
#pragma unroll
    for (int s = 0; s < NSUB; ++s) {
#pragma unroll
      for (int t = 0; t < WPT; ++t) wc[s][t] = wring[pw][s][t];
      s_c[s] = LORA ? 0.f : bf2f(sring[pw][s]);
    }
    load_w(kb + PW, IC<pw>{});
#pragma unroll
    for (int s = 0; s < NSUB; ++s) {
      const float m8s = -8.f * s_c[s];
      const uint32_t wd[4] = {wc[s][0].x, wc[s][0].y, wc[s][0].z, wc[s][0].w};
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        bf16x8_t b;
        if (LORA) b = __builtin_bit_cast(bf16x8_t, wc[s][t % WPT]);
        else b = dequant_word(wd[t], s_c[s], m8s);
#pragma unroll
        for (int m = 0; m < MT; ++m)
          acc[s][m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[m][t], b, acc[s][m], 0, 0, 0);
      }
    }
    stash_x((i + 1) & 1, IC<px1>{});
    load_x(kb + 1 + PX, IC<px1>{});
    __syncthreads();
  };

  // prologue: PX activation tiles and PW weight tiles in flight, tile 0 published
  load_x(kb0 + 0, IC<0>{}); load_x(kb0 + 1, IC<1>{}); load_x(kb0 + 2, IC<2>{}); load_x(kb0 + 3, IC<3>{});
  load_w(kb0 + 0, IC<0>{}); load_w(kb0 + 1, IC<1>{}); load_w(kb0 + 2, IC<2>{}); load_w(kb0 + 3, IC<3>{});
  if (PW == 8) {
    load_w(kb0 + 4, IC<4 % PW>{}); load_w(kb0 + 5, IC<5 % PW>{});
    load_w(kb0 + 6, IC<6 % PW>{}); load_w(kb0 + 7, IC<7 % PW>{});
  }
  stash_x(0, IC<0>{});
  load_x(kb0 + PX, IC<0>{});
  __syncthreads();
  const int ngroups = nk / 8;
  for (int g = 0; g < ngroups; ++g) {
    const int kb = kb0 + g * 8;
    tile_step(kb + 0, IC<0>{}); tile_step(kb + 1, IC<1>{}); tile_step(kb + 2, IC<2>{}); tile_step(kb + 3, IC<3>{});
    tile_step(kb + 4, IC<4>{}); tile_step(kb + 5, IC<5>{}); tile_step(kb + 6, IC<6>{}); tile_step(kb + 7, IC<7>{});
  }
  {
    const int kb = kb0 + ngroups * 8;
    const int rem = nk - ngroups * 8;
    if (rem > 0) tile_step(kb + 0, IC<0>{});
    if (rem > 1) tile_step(kb + 1, IC<1>{});
    if (rem > 2) tile_step(kb + 2, IC<2>{});
    if (rem > 3) tile_step(kb + 3, IC<3>{});
    if (rem > 4) tile_step(kb + 4, IC<4>{});
    if (rem > 5) tile_step(kb + 5, IC<5>{});
    if (rem > 6) tile_step(kb + 6, IC<6>{});
  }

  // epilogue: every wave owns its tiles outright
#pragma unroll
  for (int s = 0; s < NSUB; ++s) {
    if (!sub_ok[s]) continue;
    const int col = (nb_first + s) * 32 + nl;
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m * 32 + acc_row(r, lane);
        if (row >= a.M) continue;
        if (LORA) a.t_part[((size_t)slice * a.M + row) * a.ldt + col] = acc[s][m][r];
        else if (a.y_bf16) a.y_bf16[(size_t)row * a.N + col] = f2bf(acc[s][m][r]);
        else a.y_part[((size_t)slice * a.M + row) * a.N + col] = acc[s][m][r];
      }
  }
}

template <int MT, int NSUB>
__global__ __launch_bounds__(256, MT == 4 ? 1 : 2) void qlinear_mfma_kernel(QLinearArgs a) {
  __shared__ __align__(16) uint16_t xs[2][MT * 32][kXStride];
  if ((int)blockIdx.x >= a.n_main_blocks) gemm_block<MT, 1, true>(a, xs);
  else gemm_block<MT, NSUB, false>(a, xs);
}

template <int MT, int NSUB>
static int launch_qlinear(hipStream_t st, QLinearArgs a) {
  const int cols_per_block = 128 * NSUB;
  a.n_main_blocks = (a.N + cols_per_block - 1) / cols_per_block;
  const int blocks = a.n_main_blocks + (a.a_t ? a.lora_blocks_per_split : 0);
  hipLaunchKernelGGL((qlinear_mfma_kernel<MT, NSUB>), dim3(blocks, a.nsplit), dim3(256), 0, st, a);
  return check_launch();
}

static int slice_len(int KT, int s) { return ((KT + s - 1) / s + 3) / 4 * 4; }
static bool slices_ok(int KT, int s) { return (KT + slice_len(KT, s) - 1) / slice_len(KT, s) == s; }

// Number of K-slices for a projection.  Wide projections (>= 192 column blocks) are not
// split: they write bf16 directly.  Otherwise the smallest power of two that gives at least
// 128 workgroups and at most 32 k-tiles per slice, in whole groups of 4 k-tiles, no empty slice.
int qlinear_num_splits(int K, int N, int M) {
  (void)M;
  const int nblocks = (N + 127) / 128;
  const int KT = K / 64;
  if (nblocks >= 192) return 1;
  int best = 1;
  for (int s = 1; s <= TMX_MAX_SPLITS; s *= 2) {
    if (!slices_ok(KT, s)) break;
    best = s;
    if (nblocks * s >= 128 && slice_len(KT, s) <= 32) break;
  }
  return best;
}

// Number of K-slices of the LoRA projection t = x . A: as fine as whole groups of 4 k-tiles
// allow (at most TMX_MAX_LORA_SPLITS planes), so that no LoRA block outlasts the main blocks.
int qlinear_num_lora_splits(int K) {
  const int KT = K / 64;
  for (int per = 4;; per += 4) {
    const int n = (KT + per - 1) / per;
    if (n <= TMX_MAX_LORA_SPLITS) return n;
  }
}

// Host-side dispatch shared by the C entry point and the decode-step launcher.
// Output: y_bf16 [M, N] when nsplit == 1 and y_bf16 != null, else y_part
// [nsplit][M][N] f32 planes.  t_part: [qlinear_num_lora_splits()][M][ldt] f32.
int qlinear_base(hipStream_t st, const void* x, int ldx, const void* qw, const void* scales,
                 const void* a_t, void* y_bf16, float* y_part, float* t_part, int ldt, int M, int K,
                 int N, int G, int Rpad, int nsplit) {
  if (!x || !qw || !scales || (!y_bf16 && !y_part)) return TMX_ERR_ARG;
  if (M <= 0 || M > 128 || K <= 0 || N <= 0) return TMX_ERR_SHAPE;
  if (K % 64 || N % 32 || G % 64 || (G & (G - 1)) || K % G || (ldx % 8)) return TMX_ERR_SHAPE;
  if (a_t && (!t_part || Rpad <= 0 || Rpad % 32 || Rpad > 128 || ldt < Rpad)) return TMX_ERR_SHAPE;
  if (nsplit < 1 || nsplit > TMX_MAX_SPLITS || (nsplit > 1 && !y_part)) return TMX_ERR_ARG;
  const int KT = K / 64;
  if (!slices_ok(KT, nsplit)) return TMX_ERR_SHAPE;  // an empty K-slice
  QLinearArgs a;
  a.x = (const uint16_t*)x;
  a.ldx = ldx;
  a.qw = (const uint4*)qw;
  a.scales = (const uint16_t*)scales;
  a.a_t = (const uint16_t*)a_t;
  a.y_bf16 = (nsplit == 1) ? (uint16_t*)y_bf16 : nullptr;
  a.y_part = y_part;
  a.t_part = t_part;
  a.ldt = ldt;
  a.M = M; a.K = K; a.N = N; a.G = G; a.Rpad = Rpad;
  a.nsplit = nsplit;
  a.kt_per_split = slice_len(KT, nsplit);
  const int nls = qlinear_num_lora_splits(K);
  a.lora_blocks_per_split = (nls + nsplit - 1) / nsplit;
  a.kt_per_lora_split = slice_len(KT, nls);
  const bool wide = false;  // two column tiles per wave did not pay off: see the design notes
  if (M <= 32) return wide ? launch_qlinear<1, 2>(st, a) : launch_qlinear<1, 1>(st, a);
  if (M <= 64) return wide ? launch_qlinear<2, 2>(st, a) : launch_qlinear<2, 1>(st, a);
  return launch_qlinear<4, 1>(st, a);
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

// y[m][n] = bf16( bf16(sum_s y_part[s][m][n]) + bf16( bf16(sum_r t[m][r] B[r][n]) * ls ) )
// (+ residual), t[m][r] = bf16(sum_s t_part[s][m][r]).  Rounding points follow the
// reference's bf16 einsum -> scale -> add chain.
__global__ __launch_bounds__(256) void lora_apply_kernel(uint16_t* y, const float* y_part, int nsplit,
                                                         const float* t_part, int nlsplit, int ldt,
                                                         const uint16_t* b,
                                                         int r, float ls, const uint16_t* res, int M,
                                                         int N) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  const int m = blockIdx.y;
  if (n >= N) return;
  float v = 0.f;
  for (int s = 0; s < nsplit; ++s) v += y_part[((size_t)s * M + m) * N + n];
  v = rbf(v);
  if (t_part) {
    float d = 0.f;
    for (int rr = 0; rr < r; ++rr) {
      float t = 0.f;
      for (int s = 0; s < nlsplit; ++s) t += t_part[((size_t)s * M + m) * ldt + rr];
      d = fmaf(rbf(t), bf2f(b[(size_t)rr * N + n]), d);
    }
    v = rbf(v + rbf(rbf(d) * ls));
  }
  if (res) v = rbf(v + bf2f(res[(size_t)m * N + n]));
  y[(size_t)m * N + n] = f2bf(v);
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

extern "C" size_t tmx_qlora_linear_workspace_bytes(int M, int K, int N) {
  const size_t s = qlinear_num_splits(K, N, M);
  return (s * (size_t)M * N + (size_t)TMX_MAX_LORA_SPLITS * M * TMX_MAX_RPAD) * sizeof(float);
}

extern "C" int tmx_qlora_linear_num_splits(int M, int K, int N) { return qlinear_num_splits(K, N, M); }
extern "C" int tmx_qlora_linear_num_lora_splits(int K) { return qlinear_num_lora_splits(K); }

extern "C" int tmx_qlora_linear_planes(void* stream, const void* x, const void* qweight,
                                       const void* scales, const void* lora_a_t, float* y_part,
                                       float* t_part, int M, int K, int N, int G, int r_pad, int nsplit) {
  return qlinear_base((hipStream_t)stream, x, K, qweight, scales, lora_a_t, nullptr, y_part, t_part,
                      TMX_MAX_RPAD, M, K, N, G, r_pad, nsplit);
}

extern "C" int tmx_qlora_linear(void* stream, const void* x, const void* qweight, const void* scales,
                                const void* lora_a_t, const void* lora_b, const void* residual,
                                void* y, void* workspace, int M, int K, int N, int G, int r, int r_pad,
                                float lora_scale) {
  hipStream_t st = (hipStream_t)stream;
  const bool lora = lora_a_t != nullptr;
  if (!workspace || !y) return TMX_ERR_ARG;
  if (lora && (!lora_b || r <= 0 || r > r_pad)) return TMX_ERR_ARG;
  if (M <= 0 || M > 128) return TMX_ERR_SHAPE;
  const int ns = qlinear_num_splits(K, N, M);
  float* y_part = (float*)workspace;
  float* t_part = y_part + (size_t)ns * M * N;
  int rc = qlinear_base(st, x, K, qweight, scales, lora ? lora_a_t : nullptr, nullptr, y_part, t_part,
                        TMX_MAX_RPAD, M, K, N, G, r_pad, ns);
  if (rc != TMX_OK) return rc;
  hipLaunchKernelGGL(lora_apply_kernel, dim3((N + 255) / 256, M), dim3(256), 0, st, (uint16_t*)y, y_part,
                     ns, lora ? t_part : nullptr, qlinear_num_lora_splits(K), TMX_MAX_RPAD,
                     (const uint16_t*)lora_b, r, lora_scale,
                     (const uint16_t*)residual, M, N);
  return check_launch();
}
