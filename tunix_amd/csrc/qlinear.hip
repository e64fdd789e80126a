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
// v_cvt_f32_ubyteN (or two at a time with v_cvt_pk_f32_fp8: dequant_word in tmx_common.h),
// scaled with one fma ((u - 8) * s is exact in f32) and
// rounded pairwise to bf16 by the hardware converter, which reproduces the
// reference's bf16 dequantised weight bit for bit before it enters the MFMA.
#include <atomic>

#include "tmx_kernels.h"

namespace tmx {

// Three generations of projection kernels share the tile math (the host picks, see four_wave()):
// the 4-wave block below (narrow projections, the old fused gate|up kernel, the routed experts),
// the k-way block gemm_block<MT, 2> (any K % 64 == 0), and the direct-to-LDS blocks further down
// (qlinear_gate_up8_kernel, gemm_block_dma), which carry the decode step wherever K % 256 == 0.
// The 4-wave block:
// One workgroup = 4 waves owns a block of 4 adjacent 32-column tiles (one per wave) over one
// K-slice and advances in steps of KS = 4 k-tiles (256 k).  Per step the activation slab
// x[0:M, 256 s : 256 s + 256] is fetched once per workgroup with coalesced 16-byte loads
// (issued one step ahead), double-buffered in LDS (rows padded by 16 bytes: conflict-free
// ds_read_b128) and shared by the four waves as MFMA A fragments; weights go HBM -> registers
// through a ring that keeps two steps (8 tiles, 8 KiB per wave) in flight.  One barrier per
// step amortises the synchronisation over four tiles.  Small-N projections are split along
// K over blockIdx.y so that every CU streams weights; each split writes its own f32 plane
// (summed by the consumer kernel), so results do not depend on scheduling order.
constexpr int kKS = 4;                    // k-tiles per pipeline step
constexpr int kXStride = kKS * 64 + 8;    // bf16 elements per LDS row

// LORA = false: one int4 column tile per wave.  LORA = true: the block computes a K-slice
// of t = x . A from bf16 tiles of A (one 32-column tile per wave); A is stored in MFMA
// B-fragment order, [K/64][Rpad/32][4 steps][64 lanes][8]: each MFMA operand is one coalesced 1 KiB load.
// FUSE = true (gate | up pairs with LoRA): every wave also multiplies one of the step's four
// k-tiles by the 32-column tile of [A_gate | A_up], reusing the activation fragments it already
// holds, so t = x . A is complete inside the workgroup when the epilogue needs it.
template <int MT, bool LORA, bool FUSE = false>
__device__ __forceinline__ void gemm_block4(const QLinearArgs& a, uint16_t (*xs)[MT * 32][kXStride]) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int h = lane >> 5, nl = lane & 31;
  const int KT = a.K >> 6;
  // K-slice of this block: main blocks follow blockIdx.y; the LoRA blocks of a launch cut K
  // into finer slices of their own so that none of them is the last to finish
  const int slice = LORA ? ((int)blockIdx.x - a.n_main_blocks) + a.lora_blocks_per_split * (int)blockIdx.y
                         : (a.fixed_slice >= 0 ? a.fixed_slice : (int)blockIdx.y);
  const int per = LORA ? a.kt_per_lora_split : a.kt_per_split;
  const int kb0 = slice * per;
  const int kb1 = (kb0 + per < KT) ? kb0 + per : KT;
  const int nsteps = (kb1 - kb0) / kKS;  // slices are whole steps (host guarantees K % 256 == 0)
  if (nsteps <= 0) return;
  const int kpg_shift = (a.G == 64) ? 0 : __builtin_ctz(a.G >> 6), KG = a.K / a.G;

  // this wave's column tile; waves past the last tile recompute the last one (result dropped)
  const int NT = LORA ? (a.Rpad >> 5) : (a.N >> 5);
  // pair mode: waves 0, 1 take two gate tiles, waves 2, 3 the matching up tiles
  const int nb_mine = LORA ? wave
                      : a.pair_off ? (int)blockIdx.x * 2 + (wave & 1) + (wave >> 1) * a.pair_off
                                   : (int)blockIdx.x * 4 + wave;
  const bool tile_ok = nb_mine < NT;
  const int nb = tile_ok ? nb_mine : NT - 1;

  f32x16_t acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[m][r] = 0.f;
  // fused LoRA state: accumulators of t, ring of A tiles (this wave's k-tile of each step)
  f32x16_t tacc[FUSE ? MT : 1];
  u32x4_t lring[FUSE ? 2 : 1][4];
  const u32x4_t* lsrc = nullptr;
  if constexpr (FUSE) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < 16; ++r) tacc[m][r] = 0.f;
    lsrc = reinterpret_cast<const u32x4_t*>(a.a_t) + lane;  // Rpad == 32: 256 words per k-tile, 64 per fragment
  }

  // cooperative activation load: chunk c = tid + 256 i -> row c / 32, 16-byte column c % 32
  constexpr int XC = MT * 4;  // chunks per thread and step
  const uint16_t* xsrc[XC];
  int xoff_l[XC];
#pragma unroll
  for (int i = 0; i < XC; ++i) {
    const int c = tid + 256 * i;
    const int row_l = c >> 5, col_l = (c & 31) * 8;
    xoff_l[i] = row_l * kXStride + col_l;
    int row = row_l < a.M ? row_l : a.M - 1;
    if (a.row_src) row = a.row_src[row];
    xsrc[i] = a.x + (size_t)row * a.ldx + (size_t)kb0 * 64 + col_l;
  }
  constexpr int WPT = LORA ? 4 : 1;  // 16-byte words per lane and tile
  constexpr int DW = LORA ? 1 : 2;   // steps of weights in flight
  const u32x4_t* wsrc;
  const uint16_t* ssrc = nullptr;
  size_t wstep;  // 16-byte words between consecutive k-tiles of one column tile
  if (LORA) {
    wstep = (size_t)NT * 64 * 4;
    wsrc = reinterpret_cast<const u32x4_t*>(a.a_t) + (size_t)nb * 256 + lane + (size_t)kb0 * wstep;
  } else {
    wstep = 64;
    wsrc = reinterpret_cast<const u32x4_t*>(a.qw) + (size_t)nb * KT * 64 + lane + (size_t)kb0 * wstep;
    ssrc = a.scales + (size_t)nb * KG * 32 + nl;
  }
  u32x4_t xreg[XC];
  u32x4_t wring[DW][kKS][WPT];
  uint16_t sring[DW][kKS];
  const int last_step = nsteps - 1;

  // Unconditional loads with clamped step indices: the compiler can then count the
  // outstanding loads exactly and wait only for the oldest one.
  auto load_w_tile = [&](int step, auto dc, auto kc) __attribute__((always_inline)) {
    constexpr int d = decltype(dc)::value, kt = decltype(kc)::value;
    step = step < last_step ? step : last_step;
    const int rel = step * kKS + kt;  // k-tile relative to kb0
#pragma unroll
    for (int t = 0; t < WPT; ++t) wring[d][kt][t] = wsrc[(size_t)rel * wstep + t * (LORA ? 64 : 1)];
    if (!LORA) sring[d][kt] = ssrc[(size_t)((kb0 + rel) >> kpg_shift) * 32];
  };
  auto load_w = [&](int step, auto dc) __attribute__((always_inline)) {
    load_w_tile(step, dc, IC<0>{}); load_w_tile(step, dc, IC<1>{});
    load_w_tile(step, dc, IC<2>{}); load_w_tile(step, dc, IC<3>{});
  };
  auto load_x = [&](int step) __attribute__((always_inline)) {
    step = step < last_step ? step : last_step;
#pragma unroll
    for (int i = 0; i < XC; ++i)
      xreg[i] = *reinterpret_cast<const u32x4_t*>(xsrc[i] + (size_t)step * kKS * 64);
  };
  auto stash_x = [&](int buf) __attribute__((always_inline)) {
    uint16_t* base = &xs[buf][0][0];
#pragma unroll
    for (int i = 0; i < XC; ++i) *reinterpret_cast<u32x4_t*>(base + xoff_l[i]) = xreg[i];
  };
  auto load_l = [&](int step, auto dc) __attribute__((always_inline)) {
    constexpr int d = decltype(dc)::value;
    step = step < last_step ? step : last_step;
    const size_t kb = (size_t)(kb0 + step * kKS + wave);
#pragma unroll
    for (int t = 0; t < 4; ++t) lring[d][t] = lsrc[kb * 256 + t * 64];
  };
  // one of the four k-tiles of a step
  auto tile_math = [&](int step, int buf, auto dc, auto kc) __attribute__((always_inline)) {
    constexpr int d = decltype(dc)::value, kt = decltype(kc)::value;
    bf16x8_t xa[MT][4];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        xa[m][t] = *reinterpret_cast<const bf16x8_t*>(&xs[buf][m * 32 + nl][kt * 64 + t * 16 + h * 8]);
    u32x4_t wc[WPT];
#pragma unroll
    for (int t = 0; t < WPT; ++t) wc[t] = wring[d][kt][t];
    const float s_c = LORA ? 0.f : bf2f(sring[d][kt]);
    load_w_tile(step + DW, dc, kc);  // slot consumed: refill it DW steps ahead
    const float m8s = -8.f * s_c;
    const uint32_t wd[4] = {wc[0].x, wc[0].y, wc[0].z, wc[0].w};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      bf16x8_t b;
      if (LORA) b = __builtin_bit_cast(bf16x8_t, wc[t % WPT]);
      else b = dequant_word(wd[t], s_c, m8s);
#pragma unroll
      for (int m = 0; m < MT; ++m)
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[m][t], b, acc[m], 0, 0, 0);
    }
    if constexpr (FUSE) {
      if (wave == kt) {  // this wave's share of t = x . A: k-tile `wave` of every step
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const bf16x8_t b = __builtin_bit_cast(bf16x8_t, lring[d][t]);
#pragma unroll
          for (int m = 0; m < MT; ++m)
            tacc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[m][t], b, tacc[m], 0, 0, 0);
        }
        load_l(step + DW, dc);
      }
    }
  };
  // step s: activations in LDS buffer s & 1, weights in ring slot s % DW
  auto do_step = [&](int step, auto sc) __attribute__((always_inline)) {
    constexpr int sp = decltype(sc)::value;  // step parity (static)
    constexpr int d = sp % DW;
    load_x(step + 1);
    tile_math(step, sp, IC<d>{}, IC<0>{});
    tile_math(step, sp, IC<d>{}, IC<1>{});
    tile_math(step, sp, IC<d>{}, IC<2>{});
    tile_math(step, sp, IC<d>{}, IC<3>{});
    stash_x(sp ^ 1);
    __syncthreads();
  };

  load_x(0);
  load_w(0, IC<0>{});
  if (DW == 2) load_w(1, IC<1 % DW>{});
  if constexpr (FUSE) {
    load_l(0, IC<0>{});
    load_l(1, IC<1>{});
  }
  stash_x(0);
  __syncthreads();
  const int npairs = nsteps / 2;
  for (int g = 0; g < npairs; ++g) {
    do_step(2 * g, IC<0>{});
    do_step(2 * g + 1, IC<1>{});
  }
  if (nsteps & 1) do_step(nsteps - 1, IC<0>{});

  if (!LORA && a.pair_off) {
    // act = bf16(bf16(g * bf16(sigmoid(g))) * u), g / u = bf16 gate / up projections: the up
    // waves hand their tile to the gate waves through LDS (the slab is free after the last barrier)
    float* ex = reinterpret_cast<float*>(&xs[0][0][0]);  // [2][MT][16][64]
    // y = bf16(x . W) (+ bf16(bf16(t . B) * ls)): the LoRA product runs on the MFMA, t rows as
    // A fragments, the B columns of this tile as B fragments, k = rank padded with zeros
    f32x16_t dl[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < 16; ++r) dl[m][r] = 0.f;
    if constexpr (FUSE) {
      // B fragment of this tile's columns (rows beyond the rank are zero, which also masks
      // the t columns of the other projection inside the 16-wide k window)
      bf16x8_t tb;
      {
        const int colw = nb * 32 + nl;
        float bv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int k = h * 8 + j;
          bv[j] = k < a.lora_r ? bf2f(a.lora_b[(size_t)k * a.N + colw]) : 0.f;
        }
        uint32_t pb[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) pb[j] = pack_bf2(bv[2 * j], bv[2 * j + 1]);
        __builtin_memcpy(&tb, pb, 16);
      }
      // 1. the four waves' partial t tiles meet in LDS   2. summed, rounded to bf16 and laid out
      // row-major   3. read back as MFMA A fragments
      float* part = reinterpret_cast<float*>(&xs[0][0][0]);                      // [4][MT][16][64]
      uint16_t* ts = reinterpret_cast<uint16_t*>(part + 4 * MT * 16 * 64);      // [MT * 32][40]
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int r = 0; r < 16; ++r) part[(((wave * MT + m) * 16 + r) << 6) + lane] = tacc[m][r];
      __syncthreads();
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const int r = wave * 4 + rr;
          float t = 0.f;
#pragma unroll
          for (int w = 0; w < 4; ++w) t += part[(((w * MT + m) * 16 + r) << 6) + lane];
          ts[(m * 32 + acc_row(r, lane)) * 40 + nl] = f2bf(t);
        }
      __syncthreads();
      const int toff = (wave >= 2) ? a.lora_r : 0;
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        uint16_t tv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) tv[j] = ts[(m * 32 + nl) * 40 + toff + h * 8 + j];
        bf16x8_t ta;
        __builtin_memcpy(&ta, tv, 16);
        dl[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ta, tb, dl[m], 0, 0, 0);
      }
      __syncthreads();  // ts / part are overwritten by the exchange below
    }
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float y = rbf(acc[m][r]);
        if (FUSE) y = rbf(y + rbf(rbf(dl[m][r]) * a.lora_ls));
        acc[m][r] = y;
      }
    if (wave >= 2) {
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int r = 0; r < 16; ++r) ex[((((wave - 2) * MT + m) * 16 + r) << 6) + lane] = acc[m][r];
    }
    __syncthreads();
    if (wave < 2 && tile_ok) {
      const int col = ((int)blockIdx.x * 2 + wave) * 32 + nl;
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = m * 32 + acc_row(r, lane);
          if (row >= a.M) continue;
          const float g = acc[m][r], u = ex[(((wave * MT + m) * 16 + r) << 6) + lane];
          const float sg = rbf(1.f / (1.f + expf(-g)));
          const int drow = a.row_dst ? a.row_dst[row] : row;
          a.y_bf16[(size_t)drow * a.ldy + col] = f2bf(rbf(g * sg) * u);
        }
    }
    return;
  }
  // epilogue: every wave owns its tile outright
  if (tile_ok) {
    const int col = nb_mine * 32 + nl;
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m * 32 + acc_row(r, lane);
        if (row >= a.M) continue;
        const int drow = (!LORA && a.row_dst) ? a.row_dst[row] : row;
        if (LORA) a.t_part[((size_t)slice * a.M + row) * a.ldt + col] = acc[m][r];
        else if (a.y_bf16) a.y_bf16[(size_t)drow * a.ldy + col] = f2bf(acc[m][r]);
        else a.y_part[((size_t)slice * a.M + row) * a.N + col] = acc[m][r];
      }
  }
}

template <int MT>
__global__ __launch_bounds__(256, MT == 4 ? 1 : 2) void qlinear_mfma4_kernel(QLinearArgs a) {
  __shared__ __align__(16) uint16_t xs[2][MT * 32][kXStride];
  if ((int)blockIdx.x >= a.n_main_blocks) gemm_block4<MT, true>(a, xs);
  else gemm_block4<MT, false>(a, xs);
}

template <int MT>
__global__ __launch_bounds__(256, 1) void qlinear_gate_up_kernel(QLinearArgs a) {
  __shared__ __align__(16) uint16_t xs[2][MT * 32][kXStride];
  gemm_block4<MT, false, true>(a, xs);
}

template <int MT>
static int launch_qlinear4(hipStream_t st, QLinearArgs a) {
  a.n_main_blocks = (a.N + 127) / 128;
  const int blocks = a.n_main_blocks + (a.a_t ? a.lora_blocks_per_split : 0);
  hipLaunchKernelGGL((qlinear_mfma4_kernel<MT>), dim3(blocks, a.nsplit), dim3(256), 0, st, a);
  return check_launch();
}

// Routed experts (tunix/models/qwen3/model.py:894-939 evaluated for routed pairs only): grid (column
// groups, experts).  Every workgroup first collects the pairs (token, slot) routed to its expert from
// the routing table (at most a few hundred entries) and leaves if there are none, so unrouted experts
// are never streamed.  In decode an expert sees a handful of rows (batch x top_k pairs spread over many
// experts), so the product is nothing but a weight stream: every wave walks its own column tiles (DOWN)
// or gate / up tile pairs (SwiGLU in its epilogue) over all of K with no LDS and no barrier after the
// compaction.  Weight tiles come through a ring of kMoeRing tiles per wave (buffer loads, scalar
// offsets), the x fragments of the live rows straight from global memory (gathered activation rows;
// lanes of absent rows hold zeros), one k-tile ahead; output rows are scattered.  The ring runs on
// across the wave's tiles, so the stream never drains.  More than 32 rows of an expert are taken in
// chunks of 32, each streaming the weights again (rare).
// Weight tiles that ONE wave reads once, whole cache lines per load (the routed experts, the fused gate | up
// launch): non-temporal buffer loads (the nt bit of the cache policy).  A plain streaming read reaches 5.6-6.2 TB/s
// on this part, a non-temporal one 6.3-7.0; the split projections and the 64-row head measured slower with it.
constexpr int kNtLoad = 2;

constexpr int kMoeRing = 4;  // divides K / 64 (K % 256 == 0), so a ring slot is k-tile % 4 in every unit

template <bool DOWN>
__global__ __launch_bounds__(256, 2) void moe_stream_kernel(MoeArgs m) {
  __shared__ int rows_s[TMX_MAX_MOE_PAIRS];
  __shared__ int wave_cnt[4];
  __shared__ int n_s;
  constexpr int TPU = DOWN ? 1 : 2;  // tiles per unit: one column tile, or a gate tile and its up tile
  const int e = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, nl = lane & 31;
  int base = 0;
  int ev = tid < m.P ? m.expert_of[tid] : -1;
  for (int p0 = 0; p0 < m.P; p0 += 256) {  // ordered compaction of { p : expert_of[p] == e }
    const int p = p0 + tid;
    const bool hit = ev == e;
    ev = p + 256 < m.P ? m.expert_of[p + 256] : -1;  // the next round's entry travels during this one's barriers
    const unsigned long long mask = __ballot(hit);
    if (lane == 0) wave_cnt[wave] = __popcll(mask);
    __syncthreads();
    int off = base;
    for (int w = 0; w < wave; ++w) off += wave_cnt[w];
    if (hit) rows_s[off + __popcll(mask & ((1ull << lane) - 1ull))] = p;
    base += wave_cnt[0] + wave_cnt[1] + wave_cnt[2] + wave_cnt[3];
    __syncthreads();
  }
  if (tid == 0) n_s = base;
  __syncthreads();
  const int n = n_s;
  if (n == 0) return;

  const int KT = m.K >> 6, KG = m.K / m.G, gs = __builtin_ctz(m.G >> 6);
  const int NT = m.N >> 5;
  const int units = DOWN ? NT : NT / 2;  // column tiles, or gate | up pairs (F / 32)
  // units of this wave: u = blockIdx.x + groups * (wave + 4 j), j = 0, 1, ... (groups = gridDim.x)
  const int u0 = (int)blockIdx.x + (int)gridDim.x * wave, ustride = (int)gridDim.x * 4;
  if (u0 >= units) return;
  const int nu = (units - u0 + ustride - 1) / ustride;

  const __amdgpu_buffer_rsrc_t rw = make_rsrc(m.qw + (size_t)e * m.qw_stride, (uint32_t)NT * KT * 1024u);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(m.scales + (size_t)e * m.sc_stride, (uint32_t)NT * KG * 64u);

  for (int c0 = 0; c0 < n; c0 += 32) {
    const int rows = n - c0 < 32 ? n - c0 : 32;
    // A fragments: lane (row nl, h) reads x[src][64 kt + 16 t + 8 h ..]; absent rows stay zero
    const bool live = nl < rows;
    const int pr = live ? rows_s[c0 + nl] : 0;
    const uint16_t* xrow = m.x + (size_t)(DOWN ? pr : pr / m.top_k) * m.ldx + 8 * h;
    u32x4_t wring[kMoeRing][TPU];
    uint16_t sring[kMoeRing][TPU];
    // tile (unit ui of this wave, k-tile kt) into ring slot sl; past the last unit: its last tile again
    auto load_w = [&](int ui, int kt, auto sc) __attribute__((always_inline)) {
      constexpr int sl = decltype(sc)::value;
      if (ui >= nu) { ui = nu - 1; kt = KT - 1; }
#pragma unroll
      for (int c = 0; c < TPU; ++c) {
        const int nb = u0 + ui * ustride + c * units;  // the gate tile, or the up tile F / 32 further on
        wring[sl][c] = __builtin_amdgcn_raw_buffer_load_b128(rw, lane * 16, (nb * KT + kt) * 1024, kNtLoad);
        sring[sl][c] = __builtin_amdgcn_raw_buffer_load_b16(rs, nl * 2, (nb * KG + (kt >> gs)) * 64, 0);
      }
    };
    u32x4_t xq[2][4];
    auto load_x = [&](int kt, int slot) __attribute__((always_inline)) {
#pragma unroll
      for (int t = 0; t < 4; ++t)
        xq[slot][t] = live ? *reinterpret_cast<const u32x4_t*>(xrow + kt * 64 + 16 * t) : u32x4_t{0, 0, 0, 0};
    };
    static_for<kMoeRing>([&](auto sc) __attribute__((always_inline)) { load_w(0, decltype(sc)::value, sc); });
    load_x(0, 0);
    f32x16_t acc[TPU];
    for (int u = 0; u < nu; ++u) {
#pragma unroll
      for (int c = 0; c < TPU; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
      for (int k0 = 0; k0 < KT; k0 += kMoeRing) {  // host: K % 256 == 0, so every group is whole
        static_for<kMoeRing>([&](auto sc) __attribute__((always_inline)) {
          constexpr int sl = decltype(sc)::value;
          const int kt = k0 + sl;
          load_x(kt + 1 < KT ? kt + 1 : 0, (sl & 1) ^ 1);  // the next k-tile (of the next unit: the same rows)
          u32x4_t wc[TPU];
          float s_c[TPU];
#pragma unroll
          for (int c = 0; c < TPU; ++c) { wc[c] = wring[sl][c]; s_c[c] = bf2f(sring[sl][c]); }
          // slot consumed: refill it with the tile kMoeRing steps on in the wave's unit-major order
          if (kt + kMoeRing < KT) load_w(u, kt + kMoeRing, sc);
          else load_w(u + 1, kt + kMoeRing - KT, sc);
#pragma unroll
          for (int c = 0; c < TPU; ++c) {
            const float m8s = -8.f * s_c[c];
            const uint32_t wd[4] = {wc[c].x, wc[c].y, wc[c].z, wc[c].w};
#pragma unroll
            for (int t = 0; t < 4; ++t)
              acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, xq[sl & 1][t]),
                                                               dequant_word<true>(wd[t], s_c[c], m8s), acc[c], 0, 0, 0);
          }
        });
      }
      // epilogue of the unit
      const int ut = u0 + u * ustride;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = acc_row(r, lane);
        if (row >= rows) continue;
        const int p = rows_s[c0 + row];
        if (DOWN) {
          m.out[(size_t)p * m.ldo + ut * 32 + nl] = f2bf(acc[0][r]);
        } else {
          const float g = rbf(acc[0][r]), up = rbf(acc[TPU - 1][r]);
          const float sg = rbf(1.f / (1.f + expf(-g)));
          m.out[(size_t)p * m.ldo + ut * 32 + nl] = f2bf(rbf(g * sg) * up);
        }
      }
    }
  }
}

// Many rows per expert (cache fill and scoring passes of a MoE model: thousands of routed pairs): the
// stream kernel above would re-read the gathered activation rows in every wave, so here a workgroup
// (column block, expert) runs the 4-wave block over the expert's rows in chunks of 32 with the
// activation slab shared in LDS (gathered rows in, scattered rows out).  DOWN = false fuses SwiGLU: the
// workgroup owns 64 gate columns and the matching 64 up columns.
template <bool DOWN>
__global__ __launch_bounds__(256, 2) void moe_block_kernel(MoeArgs m) {
  __shared__ __align__(16) uint16_t xs[2][32][kXStride];
  __shared__ int rows_s[TMX_MAX_MOE_PAIRS];
  __shared__ int src_s[32], dst_s[32];
  __shared__ int wave_cnt[4];
  __shared__ int n_s;
  const int e = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int base = 0;
  int ev = tid < m.P ? m.expert_of[tid] : -1;
  for (int p0 = 0; p0 < m.P; p0 += 256) {  // ordered compaction of { p : expert_of[p] == e }
    const int p = p0 + tid;
    const bool hit = ev == e;
    ev = p + 256 < m.P ? m.expert_of[p + 256] : -1;  // the next round's entry travels during this one's barriers
    const unsigned long long mask = __ballot(hit);
    if (lane == 0) wave_cnt[wave] = __popcll(mask);
    __syncthreads();
    int off = base;
    for (int w = 0; w < wave; ++w) off += wave_cnt[w];
    if (hit) rows_s[off + __popcll(mask & ((1ull << lane) - 1ull))] = p;
    base += wave_cnt[0] + wave_cnt[1] + wave_cnt[2] + wave_cnt[3];
    __syncthreads();
  }
  if (tid == 0) n_s = base;
  __syncthreads();
  const int n = n_s;
  if (n == 0) return;
  QLinearArgs a = {};
  a.x = m.x;
  a.ldx = m.ldx;
  a.qw = m.qw + (size_t)e * m.qw_stride;
  a.scales = m.scales + (size_t)e * m.sc_stride;
  a.y_bf16 = m.out;
  a.ldy = m.ldo;
  a.K = m.K; a.N = m.N; a.G = m.G;
  a.n_main_blocks = gridDim.x;
  a.nsplit = 1;
  a.kt_per_split = m.K >> 6;
  a.fixed_slice = 0;
  a.row_src = src_s;
  a.row_dst = dst_s;
  a.pair_off = DOWN ? 0 : (m.N >> 6);  // tiles in F = N / 2 columns
  for (int c0 = 0; c0 < n; c0 += 32) {
    if (tid < 32 && c0 + tid < n) {
      const int p = rows_s[c0 + tid];
      src_s[tid] = DOWN ? p : p / m.top_k;
      dst_s[tid] = p;
    }
    __syncthreads();
    a.M = n - c0 < 32 ? n - c0 : 32;
    gemm_block4<1, false>(a, xs);
    __syncthreads();
  }
}


int moe_experts(hipStream_t st, const MoeArgs& a, int E, bool down) {
  if (!a.x || !a.qw || !a.scales || !a.expert_of || !a.out) return TMX_ERR_ARG;
  if (a.P <= 0 || a.P > TMX_MAX_MOE_PAIRS || a.top_k <= 0 || E <= 0) return TMX_ERR_SHAPE;
  if (a.K % 256 || a.G % 64 || (a.G & (a.G - 1)) || a.K % a.G || a.ldx % 8) return TMX_ERR_SHAPE;
  if (a.N % 128) return TMX_ERR_SHAPE;  // gate | up: F % 64 == 0
  if (a.P > 1024) {  // many rows per expert: the block kernel with the activation slab in LDS
    if (down) hipLaunchKernelGGL(moe_block_kernel<true>, dim3(a.N / 128, E), dim3(256), 0, st, a);
    else hipLaunchKernelGGL(moe_block_kernel<false>, dim3(a.N / 128, E), dim3(256), 0, st, a);
    return check_launch();
  }
  // decode: few rows per expert, a pure weight stream
  // column groups per expert: one gate | up pair (2 x K / 64 weight tiles) or two down tiles per wave
  // (measured on the 30B-A3B shapes: 6 groups for gate | up, 8 for down; fewer leave CUs short of
  // loads in flight, more leave waves without work)
  const int units = down ? a.N / 32 : a.N / 64;
  int groups = units / (down ? 8 : 4);
  groups = groups < 1 ? 1 : (groups > 32 ? 32 : groups);
  if (down) hipLaunchKernelGGL(moe_stream_kernel<true>, dim3(groups, E), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(moe_stream_kernel<false>, dim3(groups, E), dim3(256), 0, st, a);
  return check_launch();
}

// One workgroup owns a block of 4 adjacent 32-column tiles over one K-slice.  It runs 4 * KW
// waves: wave (ct, kw) multiplies column tile ct by every KW-th group of TPW k-tiles, so a CU
// holds 2-4 waves per SIMD whose dequantisation (VALU), MFMA and load latencies overlap.  The
// workgroup advances in steps of KS k-tiles: the activation slab x[0:M, step] is fetched once
// with coalesced 16-byte loads (issued one step ahead), double-buffered in LDS (rows padded by
// 16 bytes: conflict-free ds_read_b128) and shared by all waves as MFMA A fragments; weights go
// HBM -> registers through a ring that keeps two steps in flight per wave.  The KW partial
// accumulators of a column tile are added through LDS at the end.  Small-N projections are also
// split along K over blockIdx.y so that every CU streams weights; each split writes its own f32
// plane (summed by the consumer kernel), so results do not depend on scheduling order.
template <int MT, int KW_>
struct Shape {
  static constexpr int KW = KW_;                // k-ways: waves sharing one column tile
  static constexpr int KS = (MT == 4 || KW_ == 1) ? 4 : 8;  // k-tiles per step
  static constexpr int TPW = KS / KW;           // k-tiles per wave and step
  static constexpr int NTHR = 256 * KW;
  static constexpr int ROWS = MT * 32;
  static constexpr int XS = KS * 64 + 8;        // bf16 elements per LDS row
  static constexpr size_t LDS = (size_t)2 * ROWS * XS * 2;
};

// LORA = false: int4 column tiles.  LORA = true: the block computes a K-slice of t = x . A from
// bf16 tiles of A; A is stored in MFMA B-fragment order, [K/64][Rpad/32][4 steps][64 lanes][8],
// so a wave reads the 4 KiB of a tile contiguously.
template <int MT, int KW_, bool LORA>
__device__ __forceinline__ void gemm_block(const QLinearArgs& a, uint16_t* smem) {
  using S = Shape<MT, KW_>;
  constexpr int KW = S::KW, KS = S::KS, TPW = S::TPW, NTHR = S::NTHR, ROWS = S::ROWS, XS = S::XS;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ct = wave & 3, kw = wave >> 2;
  const int h = lane >> 5, nl = lane & 31;
  const int KT = a.K >> 6;
  // K-slice of this block: main blocks follow blockIdx.y; the LoRA blocks of a launch cut K
  // into finer slices of their own so that none of them is the last to finish
  const int slice = LORA ? ((int)blockIdx.x - a.n_main_blocks) + a.lora_blocks_per_split * (int)blockIdx.y
                         : (int)blockIdx.y;
  const int per = LORA ? a.kt_per_lora_split : a.kt_per_split;
  const int kb0 = slice * per;
  const int kb1 = (kb0 + per < KT) ? kb0 + per : KT;
  const int ntiles = kb1 - kb0;
  if (ntiles <= 0) return;
  const int nsteps = (ntiles + KS - 1) / KS;
  const int kpg_shift = (a.G == 64) ? 0 : __builtin_ctz(a.G >> 6), KG = a.K / a.G;

  // this wave's column tile; waves past the last tile idle through the steps
  const int NT = LORA ? (a.Rpad >> 5) : (a.N >> 5);
  const int nb = LORA ? ct : (int)blockIdx.x * 4 + ct;
  const bool tile_ok = nb < NT;

  f32x16_t acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[m][r] = 0.f;

  // cooperative activation load: chunk c = tid + NTHR i -> row c / CPR, 16-byte column c % CPR
  constexpr int CPR = KS * 8;
  constexpr int XC = ROWS * CPR / NTHR;
  const uint16_t* xsrc[XC];
  int xoff_l[XC], xmax[XC];
#pragma unroll
  for (int i = 0; i < XC; ++i) {
    const int c = tid + NTHR * i;
    const int row_l = c / CPR, col_l = (c % CPR) * 8;
    xoff_l[i] = row_l * XS + col_l;
    const int row = row_l < a.M ? row_l : a.M - 1;
    xsrc[i] = a.x + (size_t)row * a.ldx + (size_t)kb0 * 64 + col_l;
    xmax[i] = a.K - 8 - (kb0 * 64 + col_l);  // last in-bounds offset (columns of skipped tiles)
  }
  constexpr int WPT = LORA ? 4 : 1;  // 16-byte words per lane and tile
  constexpr int DW = LORA ? 1 : 2;   // steps of weights in flight
  const u32x4_t* wsrc = nullptr;
  const uint16_t* ssrc = nullptr;
  size_t wstep = 0;  // 16-byte words between consecutive k-tiles of one column tile
  if (tile_ok) {
    if (LORA) {
      wstep = (size_t)NT * 64 * 4;
      wsrc = reinterpret_cast<const u32x4_t*>(a.a_t) + (size_t)nb * 256 + lane + (size_t)kb0 * wstep;
    } else {
      wstep = 64;
      wsrc = reinterpret_cast<const u32x4_t*>(a.qw) + (size_t)nb * KT * 64 + lane + (size_t)kb0 * wstep;
      ssrc = a.scales + (size_t)nb * KG * 32 + nl;
    }
  }
  u32x4_t xreg[XC];
  u32x4_t wring[DW][TPW][WPT];
  uint16_t sring[DW][TPW];
  const int last_step = nsteps - 1, last_tile = ntiles - 1;

  // Unconditional loads with clamped indices: the compiler can then count the outstanding
  // loads exactly and wait only for the oldest one.
  auto load_w_tile = [&](int step, auto dc, auto jc) __attribute__((always_inline)) {
    constexpr int d = decltype(dc)::value, j = decltype(jc)::value;
    step = step < last_step ? step : last_step;
    int rel = step * KS + kw * TPW + j;  // k-tile relative to kb0
    rel = rel < last_tile ? rel : last_tile;
#pragma unroll
    for (int t = 0; t < WPT; ++t) wring[d][j][t] = wsrc[(size_t)rel * wstep + t * (LORA ? 64 : 1)];
    if (!LORA) sring[d][j] = ssrc[(size_t)((kb0 + rel) >> kpg_shift) * 32];
  };
  auto load_w = [&](int step, auto dc) __attribute__((always_inline)) {
    static_for<TPW>([&](auto jc) __attribute__((always_inline)) { load_w_tile(step, dc, jc); });
  };
  auto load_x = [&](int step) __attribute__((always_inline)) {
    step = step < last_step ? step : last_step;
#pragma unroll
    for (int i = 0; i < XC; ++i) {
      int off = step * KS * 64;
      off = off < xmax[i] ? off : xmax[i];
      xreg[i] = *reinterpret_cast<const u32x4_t*>(xsrc[i] + off);
    }
  };
  auto stash_x = [&](int buf) __attribute__((always_inline)) {
    uint16_t* base = smem + (size_t)buf * ROWS * XS;
#pragma unroll
    for (int i = 0; i < XC; ++i) *reinterpret_cast<u32x4_t*>(base + xoff_l[i]) = xreg[i];
  };
  // one k-tile of this wave
  auto tile_math = [&](int step, int buf, auto dc, auto jc) __attribute__((always_inline)) {
    constexpr int d = decltype(dc)::value, j = decltype(jc)::value;
    const uint16_t* xb = smem + (size_t)buf * ROWS * XS + (kw * TPW + j) * 64 + h * 8;
    bf16x8_t xa[MT][4];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        xa[m][t] = *reinterpret_cast<const bf16x8_t*>(xb + (m * 32 + nl) * XS + t * 16);
    u32x4_t wc[WPT];
#pragma unroll
    for (int t = 0; t < WPT; ++t) wc[t] = wring[d][j][t];
    const float s_c = LORA ? 0.f : bf2f(sring[d][j]);
    load_w_tile(step + DW, dc, jc);  // slot consumed: refill it DW steps ahead
    if (step * KS + kw * TPW + j > last_tile) return;  // past the slice (ragged last step)
    const float m8s = -8.f * s_c;
    const uint32_t wd[4] = {wc[0].x, wc[0].y, wc[0].z, wc[0].w};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      bf16x8_t b;
      if (LORA) b = __builtin_bit_cast(bf16x8_t, wc[t % WPT]);
      else b = dequant_word(wd[t], s_c, m8s);
#pragma unroll
      for (int m = 0; m < MT; ++m)
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[m][t], b, acc[m], 0, 0, 0);
    }
  };
  // step s: activations in LDS buffer s & 1, weights in ring slot s % DW
  auto do_step = [&](int step, auto sc) __attribute__((always_inline)) {
    constexpr int sp = decltype(sc)::value;  // step parity (static)
    constexpr int d = sp % DW;
    load_x(step + 1);
    if (tile_ok)
      static_for<TPW>([&](auto jc) __attribute__((always_inline)) { tile_math(step, sp, IC<d>{}, jc); });
    stash_x(sp ^ 1);
    __syncthreads();
  };

  load_x(0);
  if (tile_ok) {
    load_w(0, IC<0>{});
    if (DW == 2) load_w(1, IC<1 % DW>{});
  }
  stash_x(0);
  __syncthreads();
  const int npairs = nsteps / 2;
  for (int g = 0; g < npairs; ++g) {
    do_step(2 * g, IC<0>{});
    do_step(2 * g + 1, IC<1>{});
  }
  if (nsteps & 1) do_step(nsteps - 1, IC<0>{});

  // add the KW partial accumulators of each column tile through LDS (the slab is free now: the
  // last step ended with a barrier); layout [kw - 1][ct][m][r][lane] keeps every access linear
  float* red = reinterpret_cast<float*>(smem);
  if (kw > 0) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        red[(((((kw - 1) * 4 + ct) * MT + m) * 16 + r) << 6) + lane] = acc[m][r];
  }
  if (KW > 1) __syncthreads();
  if (kw > 0 || !tile_ok) return;
#pragma unroll
  for (int k = 1; k < KW; ++k)
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[m][r] += red[(((((k - 1) * 4 + ct) * MT + m) * 16 + r) << 6) + lane];

  const int col = nb * 32 + nl;
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = m * 32 + acc_row(r, lane);
      if (row >= a.M) continue;
      if (LORA) a.t_part[((size_t)slice * a.M + row) * a.ldt + col] = acc[m][r];
      else if (a.y_bf16) a.y_bf16[(size_t)row * a.ldy + col] = f2bf(acc[m][r]);
      else a.y_part[((size_t)slice * a.M + row) * a.N + col] = acc[m][r];
    }
}

template <int MT, int KW>
__global__ __launch_bounds__((Shape<MT, KW>::NTHR), 1) void qlinear_mfma_kernel(QLinearArgs a) {
  extern __shared__ __align__(16) uint16_t smem[];
  if ((int)blockIdx.x >= a.n_main_blocks) gemm_block<MT, KW, true>(a, smem);
  else gemm_block<MT, KW, false>(a, smem);
}

template <int MT, int KW>
static int launch_qlinear(hipStream_t st, QLinearArgs a) {
  using S = Shape<MT, KW>;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(&qlinear_mfma_kernel<MT, KW>), hipFuncAttributeMaxDynamicSharedMemorySize,
      (int)S::LDS);
  if (attr != hipSuccess) return TMX_ERR_LAUNCH;
  a.n_main_blocks = (a.N + 127) / 128;
  const int blocks = a.n_main_blocks + (a.a_t ? a.lora_blocks_per_split : 0);
  hipLaunchKernelGGL((qlinear_mfma_kernel<MT, KW>), dim3(blocks, a.nsplit), dim3(S::NTHR), S::LDS, st, a);
  return check_launch();
}

// ---------------------------------------------------------------------------
// gate | up with SwiGLU (and LoRA) in the epilogue, 8 waves per workgroup.  The workgroup owns
// 2 gate tiles and the 2 matching up tiles like the 4-wave pair block, but two waves share each
// column tile: wave (cw, kh) multiplies tile cw by k-tiles kh * TPW .. kh * TPW + TPW - 1 of
// every step (starting at k-tile kh * TPW + cw, the one whose LoRA product x . A it also owns), so each SIMD holds two waves whose dequantisation, MFMA and load waits overlap.
// All global reads are buffer loads: a per-lane byte offset that never changes plus a scalar
// offset that advances per step, so the loop carries no per-lane address arithmetic.  Weights
// are requested one step (3-4 us) ahead: a deeper ring only lengthened the queue in front of the
// memory pipeline (measured).
template <int MT>
struct GU8 {
  static constexpr int TS = 8;                 // k-tiles per step
  static constexpr int TPW = TS / 2;           // k-tiles per wave and step
  static constexpr int XS = TS * 64 + 8;       // bf16 elements per LDS row
  static constexpr int ROWS = MT * 32;
  static constexpr size_t SLAB = (size_t)2 * ROWS * XS * 2;
  static constexpr size_t EPI = (size_t)12 * MT * 16 * 64 * 4 + (size_t)ROWS * 40 * 2;
  static constexpr size_t LDS = SLAB > EPI ? SLAB : EPI;
};



// LoRA inside the gate | up launch, two ways.  LORA == 1: every workgroup multiplies x by [A_gate | A_up]
// itself (one extra MFMA group and one extra 4 KiB tile per wave and step).  LORA == 2: the first
// a.sync_blocks workgroups of the launch compute t = x . A once (a K-slice of 4 k-tiles each, partial
// tiles added by the last one to arrive) and hand it to the others through memory: every store of the
// hand-over is a write-through store (sc1) followed by a wait for its completion, the arrival counter
// and the ready flag are device-scope atomics, and the readers load with sc1, so nothing depends on
// the per-XCD L2 caches being written back or invalidated inside the kernel.  The main workgroups need
// t only in their epilogue, long after the producers are done; their wait is bounded (*a.sync_status is
// set and t taken as zero if the flag never comes).  The last reader puts the three counters back to zero,
// so the state is all-zero between launches (also under graph replay).
__device__ __forceinline__ void sc1_store_b128(__amdgpu_buffer_rsrc_t r, u32x4_t v, int off) {
  __builtin_amdgcn_raw_buffer_store_b128(v, r, off, 0, 0x10);
}
__device__ __forceinline__ u32x4_t sc1_load_b128(__amdgpu_buffer_rsrc_t r, int off) {
  return __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0x10));
}

template <int MT>
__device__ __forceinline__ void lora_producer_block(const QLinearArgs& a, float* red /* [8][16][64] */) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, nl = lane & 31;
  const int slice = blockIdx.x, P = a.sync_blocks;
  constexpr int WM = 8 / MT;            // waves per row tile: each takes one k-tile of the slice
  const int m = wave / WM, kt = slice * WM + wave % WM;  // host: K / 64 == P * WM
  const int row = min(m * 32 + nl, a.M - 1);
  f32x16_t acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  u32x4_t xa[4], at[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    xa[t] = *reinterpret_cast<const u32x4_t*>(a.x + (size_t)row * a.ldx + kt * 64 + t * 16 + h * 8);
    at[t] = reinterpret_cast<const u32x4_t*>(a.a_t)[(size_t)(kt * 4 + t) * 64 + lane];
  }
#pragma unroll
  for (int t = 0; t < 4; ++t)
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, xa[t]), __builtin_bit_cast(bf16x8_t, at[t]),
                                                  acc, 0, 0, 0);
#pragma unroll
  for (int r = 0; r < 16; ++r) red[((wave * 16 + r) << 6) + lane] = acc[r];
  __syncthreads();
  // partial tile of the slice: the WM k-tile waves of each row tile added in wave order, kept in
  // accumulator layout [m][r][lane]
  const __amdgpu_buffer_rsrc_t rp = make_rsrc(a.sync_part, (uint32_t)P * MT * 4096u);
  const __amdgpu_buffer_rsrc_t rt = make_rsrc(a.sync_t16, (uint32_t)MT * 32 * 64u);
  constexpr int VPT = MT * 1024 / 512 / 4;  // 16-byte groups per thread (MT == 2: one, MT == 1: every other thread)
  const int e0 = tid * 4;                    // element index in [m][r][lane], 4 adjacent lanes
  const bool mine = e0 < MT * 1024;
  (void)VPT;
  if (mine) {
    const int mm = e0 >> 10, rest = e0 & 1023;
    f32x4_t v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < WM; ++w) {
      const f32x4_t p = *reinterpret_cast<const f32x4_t*>(red + (((mm * WM + w) * 16) << 6) + rest);
      v += p;
    }
    sc1_store_b128(rp, __builtin_bit_cast(u32x4_t, v), (slice * MT * 1024 + e0) * 4);
  }
  __builtin_amdgcn_s_waitcnt(0);  // the write-through stores are complete
  __syncthreads();
  __shared__ uint32_t s_old;
  if (tid == 0) s_old = __hip_atomic_fetch_add(a.sync + 0, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (s_old != (uint32_t)(P - 1)) return;
  // the last slice to arrive: t = bf16(sum of the partial tiles in slice order), row-major [rows][32]
  if (mine) {
    const int mm = e0 >> 10, r = (e0 & 1023) >> 6, l0 = e0 & 63;
    f32x4_t v = {0.f, 0.f, 0.f, 0.f};
    for (int sl = 0; sl < P; ++sl)
      v += __builtin_bit_cast(f32x4_t, sc1_load_b128(rp, (sl * MT * 1024 + e0) * 4));
    // lanes l0 .. l0 + 3 share h and hold 4 adjacent columns of one row
    const int trow = mm * 32 + acc_row(r, l0), col = l0 & 31;
    const uint32_t lo = pack_bf2(v[0], v[1]), hi = pack_bf2(v[2], v[3]);
    __builtin_amdgcn_raw_buffer_store_b32(lo, rt, (trow * 32 + col) * 2, 0, 0x10);
    __builtin_amdgcn_raw_buffer_store_b32(hi, rt, (trow * 32 + col + 2) * 2, 0, 0x10);
  }
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (tid == 0) {
    __hip_atomic_store(a.sync + 0, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(a.sync + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <int MT, int LORA>
__global__ __launch_bounds__(512, 1) void qlinear_gate_up8_kernel(QLinearArgs a) {
  using S = GU8<MT>;
  constexpr bool FUSE = LORA == 1, SYNC = LORA == 2;
  constexpr int TS = S::TS, TPW = S::TPW, XS = S::XS, ROWS = S::ROWS;
  extern __shared__ __align__(16) uint16_t smem[];
  if constexpr (SYNC) {
    if ((int)blockIdx.x < a.sync_blocks) {
      lora_producer_block<MT>(a, reinterpret_cast<float*>(smem));
      return;
    }
  }
  const int bx = SYNC ? (int)blockIdx.x - a.sync_blocks : (int)blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), cw = wave & 3, kh = wave >> 2;
  const int h = lane >> 5, nl = lane & 31;
  const int KT = a.K >> 6, nsteps = KT / TS, last_step = nsteps - 1;  // host: K % (64 TS) == 0
  const int gs = __builtin_ctz(a.G >> 6), KG = a.K / a.G;
  const int nb = bx * 2 + (cw & 1) + (cw >> 1) * a.pair_off;  // host: F % 64 == 0

  const __amdgpu_buffer_rsrc_t rw = make_rsrc(a.qw, (uint32_t)(a.N >> 5) * KT * 1024u);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(a.scales, (uint32_t)(a.N >> 5) * KG * 64u);
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(a.x, (uint32_t)a.M * a.ldx * 2u);
  const __amdgpu_buffer_rsrc_t rl = make_rsrc(FUSE ? a.a_t : a.x, FUSE ? (uint32_t)KT * 4096u : 16u);
  const int wv = (nb * KT * 64 + lane) * 16;  // per-lane byte offsets
  const int sv = (nb * KG * 32 + nl) * 2;
  const int lv = lane * 16;
  // LoRA B values of this tile's columns for the epilogue (rows h * 8 .. + 7 of B): read now, so
  // that the cold reads complete under the main loop
  uint16_t tbv[8];
  if constexpr (FUSE || SYNC) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = h * 8 + j;
      tbv[j] = a.lora_b[(size_t)(k < a.lora_r ? k : 0) * a.N + nb * 32 + nl];
    }
  }

  f32x16_t acc[MT], tacc[FUSE ? MT : 1];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[m][r] = 0.f;
  if constexpr (FUSE) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < 16; ++r) tacc[m][r] = 0.f;
  }

  // activation slab of a step: one row (TS * 64 bf16 = 1 KiB) per direct-to-LDS load, rows
  // wave, wave + 8, ... of the slab; the global address is wave-uniform apart from lane * 16
  constexpr int XR = ROWS / 8;  // rows per wave and step
  const int xv = lane * 16;
  int xrow_off[XR];             // byte offset of each of this wave's rows (rows past M repeat the last)
#pragma unroll
  for (int i = 0; i < XR; ++i) {
    const int row_l = wave + 8 * i;
    xrow_off[i] = (row_l < a.M ? row_l : a.M - 1) * a.ldx * 2;
  }
  u32x4_t wring[TPW];   // weights of the next step (refilled tile by tile as they are consumed)
  uint16_t sring[TPW];
  u32x4_t lring[4];

  auto load_w_tile = [&](int step, auto jc) __attribute__((always_inline)) {
    constexpr int j = decltype(jc)::value;
    step = step < last_step ? step : last_step;
    const int kt = step * TS + kh * TPW + ((j + cw) & (TPW - 1));
    wring[j] = __builtin_amdgcn_raw_buffer_load_b128(rw, wv, kt * 1024, kNtLoad);
    sring[j] = __builtin_amdgcn_raw_buffer_load_b16(rs, sv, (kt >> gs) * 64, 0);
  };
  // global -> LDS without passing through registers (buffer_load ... lds: lane i lands at
  // base + 16 i, so a row of the slab arrives contiguously and the 16-byte row pad is skipped)
  auto dma_x = [&](int step, int buf) __attribute__((always_inline)) {
    step = step < last_step ? step : last_step;
    uint16_t* base = smem + (size_t)buf * ROWS * XS + wave * XS;
#pragma unroll
    for (int i = 0; i < XR; ++i)
      load_row_to_lds(rx, base + i * 8 * XS, xv, xrow_off[i] + step * (TS * 128));
  };
  auto load_l = [&](int step) __attribute__((always_inline)) {
    step = step < last_step ? step : last_step;
    const int so = (step * TS + kh * TPW + cw) * 4096;
#pragma unroll
    for (int t = 0; t < 4; ++t) lring[t] = __builtin_amdgcn_raw_buffer_load_b128(rl, lv + t * 1024, so, 0);
  };
  // activation fragments of the wave's j-th k-tile of a step, read one tile ahead of their use
  bf16x8_t xq[2][MT][4];
  auto read_x = [&](int buf, auto jc) __attribute__((always_inline)) {
    constexpr int j = decltype(jc)::value;
    const uint16_t* xb = smem + (size_t)buf * ROWS * XS + (kh * TPW + ((j + cw) & (TPW - 1))) * 64 + h * 8 + nl * XS;
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int t = 0; t < 4; ++t) xq[j & 1][m][t] = *reinterpret_cast<const bf16x8_t*>(xb + m * 32 * XS + t * 16);
  };
  auto tile_math = [&](int step, int buf, auto jc) __attribute__((always_inline)) {
    constexpr int j = decltype(jc)::value;
    if constexpr (j + 1 < TPW) read_x(buf, IC<j + 1>{});
    auto& xa = xq[j & 1];
    const u32x4_t wc = wring[j];
    const float s_c = bf2f(sring[j]);
    load_w_tile(step + 1, jc);  // slot consumed: refill it for the next step
    const float m8s = -8.f * s_c;
    const uint32_t wd[4] = {wc.x, wc.y, wc.z, wc.w};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const bf16x8_t b = dequant_word<true>(wd[t], s_c, m8s);
#pragma unroll
      for (int m = 0; m < MT; ++m)
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[m][t], b, acc[m], 0, 0, 0);
    }
    if constexpr (FUSE && j == 0) {  // the wave's first k-tile of a step is kh * TPW + cw: its LoRA share
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const bf16x8_t b = __builtin_bit_cast(bf16x8_t, lring[t]);
#pragma unroll
        for (int m = 0; m < MT; ++m)
          tacc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[m][t], b, tacc[m], 0, 0, 0);
      }
      load_l(step + 1);
    }
  };
  // Loads of a step younger than its slab transfer: a weight tile and a scale per k-tile plus the
  // four LoRA fragments of the duty tile.  s_waitcnt vmcnt(that count) therefore waits for the
  // slab (in-order counter) while the weight prefetch stays in flight.
  constexpr int kYounger = TPW * 2 + (FUSE ? 4 : 0);
  static_assert(TPW == 4, "every wave has exactly one LoRA duty tile per step");
  auto do_step = [&](int step, auto sc) __attribute__((always_inline)) {
    constexpr int sp = decltype(sc)::value;
    dma_x(step + 1, sp ^ 1);
    __builtin_amdgcn_sched_barrier(0);
    read_x(sp, IC<0>{});
    static_for<TPW>([&](auto jc) __attribute__((always_inline)) { tile_math(step, sp, jc); });
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0F70 | (kYounger & 15) | ((kYounger >> 4) << 14));
    __syncthreads();
  };

  dma_x(0, 0);
  static_for<TPW>([&](auto jc) __attribute__((always_inline)) { load_w_tile(0, jc); });
  if constexpr (FUSE) load_l(0);
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(0x0F70 | (kYounger & 15) | ((kYounger >> 4) << 14));
  __syncthreads();
  const int npairs = nsteps / 2;
  for (int g = 0; g < npairs; ++g) {
    do_step(2 * g, IC<0>{});
    do_step(2 * g + 1, IC<1>{});
  }
  if (nsteps & 1) do_step(nsteps - 1, IC<0>{});

  // ---- epilogue (the slab is free: the last step ended with a barrier) ----
  // LDS regions (f32 unless noted): P [8 waves][MT][16][64] partial LoRA tiles, later reused as
  // Y [4 tiles][MT][16][64] finished gate / up values; H [4 tiles][MT][16][64] accumulators of the
  // second k-half; ts bf16 [ROWS][40] the LoRA projection t
  float* fl = reinterpret_cast<float*>(smem);
  float* hb = fl + 8 * MT * 1024;
  uint16_t* ts = reinterpret_cast<uint16_t*>(fl + 12 * MT * 1024);
  bf16x8_t tb;
  if constexpr (FUSE || SYNC) {
    // B fragment of this tile's columns: rows beyond the rank are zero, which also masks the t
    // columns of the other projection inside the 16-wide k window
    uint16_t bz[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) bz[j] = (h * 8 + j) < a.lora_r ? tbv[j] : (uint16_t)0;
    __builtin_memcpy(&tb, bz, 16);
  }
  if constexpr (FUSE) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < 16; ++r) fl[(((wave * MT + m) * 16 + r) << 6) + lane] = tacc[m][r];
  }
  bf16x8_t tsync[MT];
  if constexpr (SYNC) {
    // t from the producer workgroups: wait (bounded) for the ready flag, then read the rows this
    // lane needs as MFMA A fragments with loads that bypass this XCD's L2
    __shared__ uint32_t s_ready;
    if (tid == 0) {
      uint32_t ok = 0;
      for (int spin = 0; spin < (1 << 20); ++spin) {
        if (__hip_atomic_load(a.sync + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) { ok = 1; break; }
        __builtin_amdgcn_s_sleep(1);
      }
      if (!ok && a.sync_status) __hip_atomic_store(a.sync_status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_ready = ok;
    }
    __syncthreads();
    const __amdgpu_buffer_rsrc_t rt = make_rsrc(a.sync_t16, (uint32_t)MT * 32 * 64u);
    const int toff = (cw >= 2) ? a.lora_r : 0;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      u32x4_t v = {0u, 0u, 0u, 0u};
      if (s_ready) v = sc1_load_b128(rt, ((m * 32 + nl) * 32 + toff + h * 8) * 2);
      tsync[m] = __builtin_bit_cast(bf16x8_t, v);
    }
  }
  // the two k-halves of a tile swap halves of their accumulators: the first half finishes
  // registers 0..7, the second 8..15 (a + b == b + a: the sum does not depend on who adds)
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r8 = 0; r8 < 8; ++r8) {
      const int r = kh ? r8 : r8 + 8;
      hb[(((cw * MT + m) * 16 + r) << 6) + lane] = kh ? acc[m][r8] : acc[m][r8 + 8];
    }
  __syncthreads();
  if constexpr (FUSE) {
    // t = x . [A_gate | A_up]: partial tiles summed in wave order, rounded to bf16, row-major
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int rr = 0; rr < 2; ++rr) {
        const int r = wave * 2 + rr;
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < 8; ++w) t += fl[(((w * MT + m) * 16 + r) << 6) + lane];
        ts[(m * 32 + acc_row(r, lane)) * 40 + nl] = f2bf(t);
      }
      __syncthreads();
    }
  {
    // y = bf16(x . W) (+ bf16(bf16(t . B) * ls)): the LoRA product runs on the MFMA, t rows as A
    // fragments, the B columns of this tile as B fragments, k = rank padded with zeros
    const int toff = (cw >= 2) ? a.lora_r : 0;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      f32x16_t dl;
#pragma unroll
      for (int r = 0; r < 16; ++r) dl[r] = 0.f;
      if constexpr (FUSE) {
        uint16_t tv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) tv[j] = ts[(m * 32 + nl) * 40 + toff + h * 8 + j];
        bf16x8_t ta;
        __builtin_memcpy(&ta, tv, 16);
        dl = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ta, tb, dl, 0, 0, 0);
      }
      if constexpr (SYNC) dl = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tsync[m], tb, dl, 0, 0, 0);
#pragma unroll
      for (int r8 = 0; r8 < 8; ++r8) {
        const int r = kh ? r8 + 8 : r8;
        float y = rbf((kh ? acc[m][r8 + 8] : acc[m][r8]) + hb[(((cw * MT + m) * 16 + r) << 6) + lane]);
        if (FUSE || SYNC) y = rbf(y + rbf(rbf(kh ? dl[r8 + 8] : dl[r8]) * a.lora_ls));
        fl[(((cw * MT + m) * 16 + r) << 6) + lane] = y;  // partial tiles were consumed before the last barrier
      }
    }
  }
  __syncthreads();
  // act = bf16(bf16(g * bf16(sigmoid(g))) * u): every wave finishes a quarter of one gate tile
  {
    const int gt = wave & 1, q = wave >> 1;
    const int col = (bx * 2 + gt) * 32 + nl;
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int r = q * 4 + rr;
        const int row = m * 32 + acc_row(r, lane);
        if (row >= a.M) continue;
        const float g = fl[(((gt * MT + m) * 16 + r) << 6) + lane];
        const float u = fl[((((2 + gt) * MT + m) * 16 + r) << 6) + lane];
        const float sg = rbf(1.f / (1.f + expf(-g)));
        a.y_bf16[(size_t)row * a.ldy + col] = f2bf(rbf(g * sg) * u);
      }
  }
  if constexpr (SYNC) {
    // every lane's t fragments were consumed before the barrier above; the last reader of the launch
    // puts the hand-over state back to zero
    if (tid == 0) {
      const uint32_t old = __hip_atomic_fetch_add(a.sync + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (old == (uint32_t)(a.n_main_blocks - 1)) {
        __hip_atomic_store(a.sync + 2, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(a.sync + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
}

template <int MT, int LORA>
static int launch_gate_up8(hipStream_t st, const QLinearArgs& a) {
  using S = GU8<MT>;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(&qlinear_gate_up8_kernel<MT, LORA>),
      hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS);
  if (attr != hipSuccess) return TMX_ERR_LAUNCH;
  const int blocks = a.n_main_blocks + (LORA == 2 ? a.sync_blocks : 0);
  hipLaunchKernelGGL((qlinear_gate_up8_kernel<MT, LORA>), dim3(blocks, 1), dim3(512), S::LDS, st, a);
  return check_launch();
}

// ---------------------------------------------------------------------------
// The k-way block for slices made of whole 4-tile steps (K % 256 == 0, up to 64 rows): wave
// (ct, kw) multiplies column tile ct by k-tiles 2 kw, 2 kw + 1 of every step.  Every global read
// is a buffer load with a fixed per-lane offset and a scalar offset that advances per step, and
// the activation slab goes from global memory straight into LDS, so the loop has no per-lane
// address arithmetic, no staging registers and no LDS stores.  A slab row is 512 bytes; a
// direct-to-LDS load lands 1 KiB contiguously, i.e. two rows back to back, so rows are stored
// unpadded and the 16-byte chunks of row r are XOR-swizzled by r % 16 instead (the global
// address of every lane is free, so the swizzle costs nothing).  A 16-byte LDS read serves 16
// lanes per clock over 64 banks: 16 consecutive rows must land in 16 different chunk columns
// for the fragment reads to stay conflict-free (a swizzle by r % 8 runs at half rate).  64 KiB of LDS and <= 128 registers: two workgroups = 16 waves per CU.
struct KD {
  static constexpr int TS = 4, TPW = 2, XS = 256;
  static constexpr size_t lds(int MT) { return (size_t)2 * MT * 32 * XS * 2; }
};

// LoRA delta by the LoRA blocks of a split projection.  Every LoRA block that holds k-tiles has stored
// its plane of t = x . A with write-through stores and counts itself in (stores complete before the
// counter moves).  Then ALL LoRA blocks of the launch (also those whose slice is empty) wait until every
// slice has arrived, a bounded number of polls; each adds the planes in slice order (loads past its L2),
// rounds to bf16, and takes its share of the column tiles of delta = bf16(bf16(t . B) * ls): t rows are
// the MFMA A operand, B columns the B operand, the rank in steps of 16 with zeros past it.  The B
// fragments of a wave's first tiles are requested before the wait.  The main blocks never wait for any
// of this, and the LoRA blocks' slices are short, so the stage runs while the main blocks still
// multiply.  The last block to finish puts the two counters back to zero.
template <int MT>
__device__ __forceinline__ void lora_delta_stage(const QLinearArgs& a, uint16_t* smem, const bool holds_slice) {
  __shared__ uint32_t s_flag;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, nl = lane & 31;
  const int L = a.lora_blocks_per_split * a.nsplit;
  const int me = ((int)blockIdx.x - a.n_main_blocks) + a.lora_blocks_per_split * (int)blockIdx.y;
  const int rows = a.M < MT * 32 ? a.M : MT * 32;
  const __amdgpu_buffer_rsrc_t rp = make_rsrc(a.t_part, 0x7FFFFFFFu);
  if (holds_slice) {
    __builtin_amdgcn_s_waitcnt(0);  // this block's plane is in memory
    __syncthreads();
    if (tid == 0) __hip_atomic_fetch_add(a.sync + 0, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // B fragments (rank step 0) of this wave's first tiles: they do not depend on t
  constexpr int PT = 2;  // host: at most two tiles per wave
  const int ntiles = a.N >> 5, ksteps = (a.lora_r + 15) >> 4, tstride = L * 8;
  const int tile0 = me * 8 + wave;
  bf16x8_t tb0[PT];
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const int tile = tile0 + i * tstride;
    uint16_t bz[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = h * 8 + j;
      bz[j] = (tile < ntiles && k < a.lora_r) ? a.lora_b[(size_t)k * a.N + tile * 32 + nl] : (uint16_t)0;
    }
    __builtin_memcpy(&tb0[i], bz, 16);
  }
  if (tid == 0) {
    uint32_t ok = 0;
    for (int spin = 0; spin < (1 << 20); ++spin) {
      if (__hip_atomic_load(a.sync + 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= (uint32_t)a.n_lora_slices) { ok = 1; break; }
      __builtin_amdgcn_s_sleep(1);
    }
    if (!ok && a.sync_status) __hip_atomic_store(a.sync_status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_flag = ok;
  }
  __syncthreads();
  const bool ready = s_flag != 0;  // false: t is taken as zero (the status word says so)
  // t = bf16(sum of the planes in slice order) into LDS (the slab area is free), bf16 [MT * 32][Rpad];
  // a thread takes four adjacent columns, up to 16 planes requested at a time
  uint16_t* ts = smem;
  const int TSR = a.Rpad + 8;  // padded row: 16-byte fragment reads of 32 rows spread over the banks
  const int quads = a.Rpad >> 2;
  for (int e = tid; e < MT * 32 * quads; e += 512) {
    const int row = e / quads, c = (e - row * quads) * 4;
    f32x4_t t = {0.f, 0.f, 0.f, 0.f};
    if (ready && row < rows) {
      constexpr int PB = MT == 1 ? 8 : 16;  // planes requested at a time
      for (int p0 = 0; p0 < a.n_lora_slices; p0 += PB) {
        u32x4_t v[PB];
#pragma unroll
        for (int u = 0; u < PB; ++u) {
          const int p = p0 + u < a.n_lora_slices ? p0 + u : a.n_lora_slices - 1;
          v[u] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rp, (int)((((size_t)p * a.M + row) * a.ldt + c) * 4), 0, 0x10));
        }
#pragma unroll
        for (int u = 0; u < PB; ++u)
          if (p0 + u < a.n_lora_slices) t += __builtin_bit_cast(f32x4_t, v[u]);
      }
    }
    uint2 pk;
    pk.x = pack_bf2(t[0], t[1]);
    pk.y = pack_bf2(t[2], t[3]);
    *reinterpret_cast<uint2*>(ts + row * TSR + c) = pk;
  }
  __syncthreads();
  // delta^T = B^T . t^T: with the B columns as the MFMA A operand and the t rows as its B operand a lane ends
  // up with 16 columns of ONE row, four adjacent ones per register group, which leave as 8-byte stores
  const bool vec_t = (a.lora_r & 7) == 0;  // whole 8-rank groups: one 16-byte LDS read per fragment
  for (int i = 0, tile = tile0; tile < ntiles; ++i, tile += tstride) {
    const int n = tile * 32 + nl;
    const int seg = tile * 32 >= a.seg_end[0] ? (tile * 32 >= a.seg_end[1] ? 2 : 1) : 0;  // host: ends are multiples of 32
    const int toff = seg * a.lora_r;
    bf16x8_t tbf = tb0[0];
#pragma unroll
    for (int q = 1; q < PT; ++q)
      if (i == q) tbf = tb0[q];
    // one row tile at a time (the stage must not raise the register count of the multiply loop)
#pragma unroll 1
    for (int m = 0; m < MT; ++m) {
      if (m * 32 >= a.M) break;
      f32x16_t dl;
#pragma unroll
      for (int r = 0; r < 16; ++r) dl[r] = 0.f;
#pragma unroll 1
      for (int ks = 0; ks < ksteps; ++ks) {
        const int k0 = ks * 16 + h * 8;
        bf16x8_t tb = tbf, ta;
        if (vec_t) {
          u32x4_t z = {0u, 0u, 0u, 0u};
          if (k0 < a.lora_r) z = *reinterpret_cast<const u32x4_t*>(ts + (m * 32 + nl) * TSR + toff + k0);
          ta = __builtin_bit_cast(bf16x8_t, z);
        } else {
          uint16_t tz[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) tz[j] = k0 + j < a.lora_r ? ts[(m * 32 + nl) * TSR + toff + k0 + j] : (uint16_t)0;
          __builtin_memcpy(&ta, tz, 16);
        }
        if (ks > 0) {
          uint16_t bz[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) bz[j] = k0 + j < a.lora_r ? a.lora_b[(size_t)(k0 + j) * a.N + n] : (uint16_t)0;
          __builtin_memcpy(&tb, bz, 16);
        }
        dl = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tb, ta, dl, 0, 0, 0);
      }
      // register r of lane (row nl, h): column (r >> 2) * 8 + h * 4 + (r & 3) of the tile
      const int row = m * 32 + nl;
      if (row < a.M) {
        uint16_t* dst = a.delta + (size_t)row * a.N + tile * 32 + h * 4;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          uint2 pk;
          pk.x = pack_bf2(rbf(rbf(dl[4 * g]) * a.lora_ls), rbf(rbf(dl[4 * g + 1]) * a.lora_ls));
          pk.y = pack_bf2(rbf(rbf(dl[4 * g + 2]) * a.lora_ls), rbf(rbf(dl[4 * g + 3]) * a.lora_ls));
          *reinterpret_cast<uint2*>(dst + g * 8) = pk;
        }
      }
    }
  }
  // the last block to finish puts the counters back
  __syncthreads();
  if (tid == 0) {
    const uint32_t old = __hip_atomic_fetch_add(a.sync + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old == (uint32_t)(L - 1)) {
      __hip_atomic_store(a.sync + 2, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(a.sync + 0, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

template <int MT, bool LORA>
__device__ __forceinline__ void gemm_block_dma(const QLinearArgs& a, uint16_t* smem) {
  constexpr int TS = KD::TS, TPW = KD::TPW, XS = KD::XS, ROWS = MT * 32;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), ct = wave & 3, kw = wave >> 2;
  const int h = lane >> 5, nl = lane & 31;
  const int KT = a.K >> 6;
  const int slice = LORA ? ((int)blockIdx.x - a.n_main_blocks) + a.lora_blocks_per_split * (int)blockIdx.y
                         : (int)blockIdx.y;
  const int per = LORA ? a.kt_per_lora_split : a.kt_per_split;
  const int kb0 = slice * per;
  const int kb1 = (kb0 + per < KT) ? kb0 + per : KT;
  const int nsteps = (kb1 - kb0) / TS, last_step = nsteps - 1;  // host: whole steps
  if (nsteps <= 0) {
    if constexpr (LORA) {
      if (a.delta) lora_delta_stage<MT>(a, smem, false);
    }
    return;
  }
  const int gs = __builtin_ctz(a.G >> 6), KG = a.K / a.G;
  const int NT = LORA ? (a.Rpad >> 5) : (a.N >> 5);
  const int nb = LORA ? ct : (int)blockIdx.x * 4 + ct;
  const bool tile_ok = nb < NT;  // waves past the last tile only help with the slab

  const __amdgpu_buffer_rsrc_t rw =
      LORA ? make_rsrc(a.a_t, (uint32_t)KT * NT * 4096u) : make_rsrc(a.qw, (uint32_t)NT * KT * 1024u);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(a.scales, LORA ? 0u : (uint32_t)NT * KG * 64u);
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(a.x, (uint32_t)a.M * a.ldx * 2u);
  // LoRA: A in fragment order [K/64][NT][4][64 lanes][8], 4 KiB per (k-tile, column tile)
  const int wv = LORA ? nb * 4096 + lane * 16 : (nb * KT * 64 + lane) * 16;
  const int wstep = LORA ? NT * 4096 : 1024;  // bytes between consecutive k-tiles
  const int sv = (nb * KG * 32 + nl) * 2;
  // slab transfer: XR loads per wave and step; load i moves rows 2 wave + 16 i (lanes 0..31)
  // and the next one (lanes 32..63), lane l delivering chunk (l % 32) ^ (row % 16) to slot l % 32
  constexpr int XR = ROWS / 16;
  int xoff[XR];  // per-lane byte offset of the row's first step (rows past M repeat the last)
#pragma unroll
  for (int i = 0; i < XR; ++i) {
    const int row_l = 2 * wave + 16 * i + h;
    xoff[i] = (row_l < a.M ? row_l : a.M - 1) * a.ldx * 2 + ((nl ^ (row_l & 15)) * 16) + kb0 * 128;
  }

  f32x16_t acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[m][r] = 0.f;
  constexpr int WPT = LORA ? 4 : 1;  // 16-byte words per lane and tile
  constexpr int DW = 1;              // steps of weights in flight
  u32x4_t wring[DW][TPW][WPT];
  uint16_t sring[DW][TPW];

  auto load_w_tile = [&](int step, auto dc, auto jc) __attribute__((always_inline)) {
    constexpr int d = decltype(dc)::value, j = decltype(jc)::value;
    step = step < last_step ? step : last_step;
    const int kt = kb0 + step * TS + kw * TPW + j;
#pragma unroll
    for (int t = 0; t < WPT; ++t) wring[d][j][t] = __builtin_amdgcn_raw_buffer_load_b128(rw, wv + t * 1024, kt * wstep, 0);
    if (!LORA) sring[d][j] = __builtin_amdgcn_raw_buffer_load_b16(rs, sv, (kt >> gs) * 64, 0);
  };
  auto dma_x = [&](int step, int buf) __attribute__((always_inline)) {
    step = step < last_step ? step : last_step;
    uint16_t* base = smem + (size_t)buf * ROWS * XS + wave * 2 * XS;
#pragma unroll
    for (int i = 0; i < XR; ++i) load_row_to_lds(rx, base + i * 16 * XS, xoff[i], step * (TS * 128));
  };
  auto tile_math = [&](int step, int buf, auto dc, auto jc) __attribute__((always_inline)) {
    constexpr int d = decltype(dc)::value, j = decltype(jc)::value;
    const uint16_t* xb = smem + (size_t)buf * ROWS * XS + kw * TPW * 64 + nl * XS;
    bf16x8_t xa[MT][4];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        // chunk 8 j + 2 t + h of the wave's tile pair sits at slot (8 j + 2 t + h) ^ (row % 16)
        xa[m][t] = *reinterpret_cast<const bf16x8_t*>(xb + m * 32 * XS + (((8 * j + 2 * t + h) ^ (nl & 15)) * 8));
      }
    u32x4_t wc[WPT];
#pragma unroll
    for (int t = 0; t < WPT; ++t) wc[t] = wring[d][j][t];
    const float s_c = LORA ? 0.f : bf2f(sring[d][j]);
    load_w_tile(step + DW, dc, jc);  // slot consumed: refill it DW steps ahead
    const float m8s = -8.f * s_c;
    const uint32_t wd[4] = {wc[0].x, wc[0].y, wc[0].z, wc[0].w};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      bf16x8_t b;
      if (LORA) b = __builtin_bit_cast(bf16x8_t, wc[t % WPT]);
      else b = dequant_word(wd[t], s_c, m8s);
#pragma unroll
      for (int m = 0; m < MT; ++m)
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[m][t], b, acc[m], 0, 0, 0);
    }
  };
  // loads of a step younger than its slab transfer (in-order counter: waiting until only these
  // are outstanding completes the slab while the weight prefetch stays in flight)
  constexpr int kYounger = TPW * (LORA ? 4 : 2);
  auto wait_slab = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    if (tile_ok) __builtin_amdgcn_s_waitcnt(0x0F70 | (kYounger & 15) | ((kYounger >> 4) << 14));
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
  };
  auto do_step = [&](int step, auto sc) __attribute__((always_inline)) {
    constexpr int sp = decltype(sc)::value;
    constexpr int d = sp % DW;
    dma_x(step + 1, sp ^ 1);
    __builtin_amdgcn_sched_barrier(0);
    if (tile_ok)
      static_for<TPW>([&](auto jc) __attribute__((always_inline)) { tile_math(step, sp, IC<d>{}, jc); });
    wait_slab();
  };

  dma_x(0, 0);
  if (tile_ok) static_for<TPW>([&](auto jc) __attribute__((always_inline)) { load_w_tile(0, IC<0>{}, jc); });
  wait_slab();
  if (DW == 2 && tile_ok)
    static_for<TPW>([&](auto jc) __attribute__((always_inline)) { load_w_tile(1, IC<1 % DW>{}, jc); });
  const int npairs = nsteps / 2;
  for (int g = 0; g < npairs; ++g) {
    do_step(2 * g, IC<0>{});
    do_step(2 * g + 1, IC<1>{});
  }
  if (nsteps & 1) do_step(nsteps - 1, IC<0>{});

  // the two k-halves of a tile swap halves of their accumulators through LDS (the slab is free:
  // the last step ended with a barrier): the first finishes registers 0..7, the second 8..15
  float* hb = reinterpret_cast<float*>(smem);  // [4 tiles][MT][16][64]
  if (tile_ok) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r8 = 0; r8 < 8; ++r8) {
        const int r = kw ? r8 : r8 + 8;
        hb[(((ct * MT + m) * 16 + r) << 6) + lane] = kw ? acc[m][r8] : acc[m][r8 + 8];
      }
  }
  __syncthreads();
  const bool with_delta = LORA && a.delta != nullptr;
  if (!tile_ok && !with_delta) return;
  if (tile_ok) {
    const int col = nb * 32 + nl;
    const __amdgpu_buffer_rsrc_t rtp = make_rsrc(a.t_part, 0x7FFFFFFFu);
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r8 = 0; r8 < 8; ++r8) {
        const int r = kw ? r8 + 8 : r8;
        const int row = m * 32 + acc_row(r, lane);
        if (row >= a.M) continue;
        const float mine = kw ? acc[m][r8 + 8] : acc[m][r8], other = hb[(((ct * MT + m) * 16 + r) << 6) + lane];
        const float v = kw ? other + mine : mine + other;  // first half + second half
        if (LORA) {
          const size_t idx = ((size_t)slice * a.M + row) * a.ldt + col;
          if (with_delta) __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), rtp, (int)(idx * 4), 0, 0x10);
          else a.t_part[idx] = v;
        } else if (a.y_bf16) {
          a.y_bf16[(size_t)row * a.ldy + col] = f2bf(v);
        } else {
          a.y_part[((size_t)slice * a.M + row) * a.N + col] = v;
        }
      }
  }
  if constexpr (LORA) {
    if (with_delta) {
      __syncthreads();  // every wave is done with the exchange area before t is staged there
      lora_delta_stage<MT>(a, smem, true);
    }
  }
}

template <int MT>
__global__ __launch_bounds__(512, MT == 4 ? 1 : 2) void qlinear_mfma_dma_kernel(QLinearArgs a) {
  extern __shared__ __align__(16) uint16_t smem[];
  if ((int)blockIdx.x >= a.n_main_blocks) gemm_block_dma<MT, true>(a, smem);
  else gemm_block_dma<MT, false>(a, smem);
}

template <int MT>
static int launch_qlinear_dma(hipStream_t st, QLinearArgs a) {
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(&qlinear_mfma_dma_kernel<MT>), hipFuncAttributeMaxDynamicSharedMemorySize,
      (int)KD::lds(MT));
  if (attr != hipSuccess) return TMX_ERR_LAUNCH;
  a.n_main_blocks = (a.N + 127) / 128;
  const int blocks = a.n_main_blocks + (a.a_t ? a.lora_blocks_per_split : 0);
  hipLaunchKernelGGL((qlinear_mfma_dma_kernel<MT>), dim3(blocks, a.nsplit), dim3(512), KD::lds(MT), st, a);
  return check_launch();
}

// ---------------------------------------------------------------------------
// Many rows (cache fill over whole prompts: more than 128 rows per pass).  At this size the
// bound is what a CU can pull through its vector memory path (about 30 GB/s per CU, L2 hits
// included), so the block is as large as the registers allow: 256 rows x 256 columns, 0.31 bytes
// loaded per kFLOP.  Wave ct owns column tile ct and multiplies both k-tiles of every 2-tile step
// against all 8 row tiles (128 accumulator registers), so a dequantised weight fragment feeds 8
// MFMAs.  Same buffer loads and direct-to-LDS slab as the k-way block above, with 256-byte slab
// rows (four rows per 1 KiB transfer), chunks XOR-swizzled by row % 16.  Two waves per SIMD: one
// dequantises while the other multiplies.  Row blocks are blockIdx.z, K-slices blockIdx.y.
struct KW {
  static constexpr int MT = 8, ROWS = 256, COLS = 256, TS = 2, XS = 128;
  static constexpr size_t LDS = (size_t)2 * ROWS * XS * 2;  // 128 KiB
};

template <bool LORA>
__device__ __forceinline__ void gemm_block_wide(const QLinearArgs& a, uint16_t* smem, int bx, int by, int bz) {
  constexpr int MT = KW::MT, TS = KW::TS, XS = KW::XS, ROWS = KW::ROWS;
  const int tid = threadIdx.x, lane = tid & 63;
  const int ct = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, nl = lane & 31;
  const int KT = a.K >> 6;
  const int slice = LORA ? (bx - a.n_main_blocks) + a.lora_blocks_per_split * by : by;
  const int per = LORA ? a.kt_per_lora_split : a.kt_per_split;
  const int kb0 = slice * per;
  const int kb1 = (kb0 + per < KT) ? kb0 + per : KT;
  const int nsteps = (kb1 - kb0) / TS, last_step = nsteps - 1;  // host: whole steps
  if (nsteps <= 0) return;
  const int row0 = bz * ROWS;
  const int rows = a.M - row0 < ROWS ? a.M - row0 : ROWS;  // host: >= 1
  const int gs = __builtin_ctz(a.G >> 6), KG = a.K / a.G;
  const int NT = LORA ? (a.Rpad >> 5) : (a.N >> 5);
  const int nb = LORA ? ct : bx * 8 + ct;
  const bool tile_ok = nb < NT;  // waves past the last tile only help with the slab

  const __amdgpu_buffer_rsrc_t rw =
      LORA ? make_rsrc(a.a_t, (uint32_t)KT * NT * 4096u) : make_rsrc(a.qw, (uint32_t)NT * KT * 1024u);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(a.scales, LORA ? 0u : (uint32_t)NT * KG * 64u);
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(a.x + (size_t)row0 * a.ldx, (uint32_t)rows * a.ldx * 2u);
  const int wv = LORA ? nb * 4096 + lane * 16 : (nb * KT * 64 + lane) * 16;
  const int wstep = LORA ? NT * 4096 : 1024;  // bytes between consecutive k-tiles
  const int sv = (nb * KG * 32 + nl) * 2;
  // slab transfer: 8 loads per wave and step; load i moves rows 4 wave + 32 i .. + 3 (16 lanes
  // each), lane l delivering chunk (l % 16) ^ (row % 16) of the step to slot l % 16
  constexpr int XR = ROWS / 32;
  int xoff[XR];  // per-lane byte offset in the row block (rows past the end repeat the last)
#pragma unroll
  for (int i = 0; i < XR; ++i) {
    const int row_l = 4 * ct + 32 * i + (lane >> 4);
    xoff[i] = (row_l < rows ? row_l : rows - 1) * a.ldx * 2 + (((lane & 15) ^ (row_l & 15)) * 16) + kb0 * 128;
  }

  f32x16_t acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[m][r] = 0.f;
  constexpr int WPT = LORA ? 4 : 1;  // 16-byte words per lane and tile
  u32x4_t wring[TS][WPT];
  uint16_t sring[TS];

  auto load_w_tile = [&](int step, auto jc) __attribute__((always_inline)) {
    constexpr int j = decltype(jc)::value;
    step = step < last_step ? step : last_step;
    const int kt = kb0 + step * TS + j;
#pragma unroll
    for (int t = 0; t < WPT; ++t) wring[j][t] = __builtin_amdgcn_raw_buffer_load_b128(rw, wv + t * 1024, kt * wstep, 0);
    if (!LORA) sring[j] = __builtin_amdgcn_raw_buffer_load_b16(rs, sv, (kt >> gs) * 64, 0);
  };
  auto dma_x = [&](int step, int buf) __attribute__((always_inline)) {
    step = step < last_step ? step : last_step;
    uint16_t* base = smem + (size_t)buf * ROWS * XS + ct * 4 * XS;
#pragma unroll
    for (int i = 0; i < XR; ++i) load_row_to_lds(rx, base + i * 32 * XS, xoff[i], step * (TS * 128));
  };
  // One step: 8 fragment groups g = 4 j + t (k-tile j, 16-wide k-block t) of 8 MFMAs, one per row
  // tile.  Between the MFMAs of group g the wave reads the x fragments of group g + 1 (one LDS
  // read per MFMA; chunk 2 g + h of a row sits at slot (2 g + h) ^ (row % 16)) and dequantises its
  // weight fragment a quarter at a time, so the matrix pipe waits neither for LDS nor for the
  // VALU, also when both waves of a SIMD run in phase after a barrier.  The order is pinned.
  auto step_math = [&](int step, int buf) __attribute__((always_inline)) {
    u32x4_t wc[TS][WPT];
    float s_c[TS], m8s[TS];
    static_for<TS>([&](auto jc) __attribute__((always_inline)) {
      constexpr int j = decltype(jc)::value;
#pragma unroll
      for (int t = 0; t < WPT; ++t) wc[j][t] = wring[j][t];
      s_c[j] = LORA ? 0.f : bf2f(sring[j]);
      m8s[j] = -8.f * s_c[j];
      load_w_tile(step + 1, jc);  // registers consumed: refill them one step ahead
    });
    const uint16_t* xb = smem + (size_t)buf * ROWS * XS + nl * XS;
    auto word_of = [&](auto gc) __attribute__((always_inline)) {
      constexpr int g = decltype(gc)::value, j = g / 4, t = g % 4;
      return t == 0 ? wc[j][0].x : (t == 1 ? wc[j][0].y : (t == 2 ? wc[j][0].z : wc[j][0].w));
    };
    bf16x8_t xq[2][MT];
    u32x4_t bq[2];
    {
      const int slot = (h ^ (nl & 15)) * 8;
#pragma unroll
      for (int m = 0; m < MT; ++m) xq[0][m] = *reinterpret_cast<const bf16x8_t*>(xb + m * 32 * XS + slot);
      if (LORA) bq[0] = wc[0][0];
      else bq[0] = __builtin_bit_cast(u32x4_t, dequant_word(word_of(IC<0>{}), s_c[0], m8s[0]));
    }
    __builtin_amdgcn_sched_barrier(0);
    static_for<4 * TS>([&](auto gc) __attribute__((always_inline)) {
      constexpr int g = decltype(gc)::value, cur = g & 1, nxt = cur ^ 1;
      constexpr bool more = g + 1 < 4 * TS;
      constexpr int jn = (g + 1) / 4 % TS, tn = (g + 1) % 4;
      const int slot = ((2 * (g + 1) + h) ^ (nl & 15)) * 8;
      uint32_t lo = 0, hi = 0;
      static_for<MT>([&](auto mc) __attribute__((always_inline)) {
        constexpr int m = decltype(mc)::value;
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xq[cur][m], __builtin_bit_cast(bf16x8_t, bq[cur]), acc[m],
                                                         0, 0, 0);
        if constexpr (more) {
          xq[nxt][m] = *reinterpret_cast<const bf16x8_t*>(xb + m * 32 * XS + slot);
          if (LORA) {
            if (m == 0) bq[nxt] = wc[jn][tn % WPT];
          } else {
            if (m == 0) dequant_masks(word_of(IC<g + 1>{}), lo, hi);
            if (m == 1) bq[nxt].x = dequant_part<0>(lo, hi, s_c[jn], m8s[jn]);
            if (m == 2) bq[nxt].y = dequant_part<1>(lo, hi, s_c[jn], m8s[jn]);
            if (m == 3) bq[nxt].z = dequant_part<2>(lo, hi, s_c[jn], m8s[jn]);
            if (m == 4) bq[nxt].w = dequant_part<3>(lo, hi, s_c[jn], m8s[jn]);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      });
    });
  };
  // loads of a step younger than its slab transfer (in-order counter)
  constexpr int kYounger = TS * (LORA ? 4 : 2);
  auto wait_slab = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    if (tile_ok) __builtin_amdgcn_s_waitcnt(0x0F70 | (kYounger & 15) | ((kYounger >> 4) << 14));
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
  };

  dma_x(0, 0);
  if (tile_ok) static_for<TS>([&](auto jc) __attribute__((always_inline)) { load_w_tile(0, jc); });
  wait_slab();
  for (int step = 0; step < nsteps; ++step) {
    const int buf = step & 1;
    dma_x(step + 1, buf ^ 1);
    __builtin_amdgcn_sched_barrier(0);
    if (tile_ok) step_math(step, buf);
    wait_slab();
  }
  if (!tile_ok) return;
  const int col = nb * 32 + nl;
  if (!LORA && a.t16) {
    // LoRA in the epilogue: delta tile [32 rows, 32 columns] = t16 rows . B columns, 16 ranks per
    // MFMA (t rows are the A operand, so the delta lands in the accumulator layout of acc[m]);
    // y = bf16(bf16(base) + bf16(bf16(delta) ls))
    const int seg = nb * 32 >= a.seg_end[0] ? (nb * 32 >= a.seg_end[1] ? 2 : 1) : 0;
    const int tc0 = seg * a.lora_r;
    const int nkb = (a.lora_r + 15) >> 4;  // host: <= 4
    u32x4_t bfr[4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      uint32_t w[4] = {0, 0, 0, 0};
      if (kb < nkb) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int rr = kb * 16 + 8 * h + j;
          const uint32_t e = rr < a.lora_r ? a.lora_b[(size_t)rr * a.N + col] : 0u;
          w[j >> 1] |= e << (16 * (j & 1));
        }
      }
      bfr[kb] = u32x4_t{w[0], w[1], w[2], w[3]};
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const int trow = row0 + m * 32 + nl;
      const uint16_t* tp = a.t16 + (size_t)(trow < a.M ? trow : a.M - 1) * a.ldt16 + tc0 + 8 * h;
      f32x16_t d;
#pragma unroll
      for (int r = 0; r < 16; ++r) d[r] = 0.f;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
        if (kb < nkb) {
          const bf16x8_t tf = *reinterpret_cast<const bf16x8_t*>(tp + kb * 16);
          d = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tf, __builtin_bit_cast(bf16x8_t, bfr[kb]), d, 0, 0, 0);
        }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = row0 + m * 32 + acc_row(r, lane);
        if (row >= a.M) continue;
        a.y_bf16[(size_t)row * a.ldy + col] = f2bf(rbf(acc[m][r]) + rbf(rbf(d[r]) * a.lora_ls));
      }
    }
    return;
  }
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = row0 + m * 32 + acc_row(r, lane);
      if (row >= a.M) continue;
      const float v = acc[m][r];
      if (LORA) a.t_part[((size_t)slice * a.M + row) * a.ldt + col] = v;
      else if (a.y_bf16) a.y_bf16[(size_t)row * a.ldy + col] = f2bf(v);
      else a.y_part[((size_t)slice * a.M + row) * a.N + col] = v;
    }
}

// Workgroups are dispatched round-robin over the 8 XCDs (linear id % 8), each with its own L2.
// The launch is one-dimensional and maps ids so that the workgroups of an XCD share row blocks:
// with S = gcd(row blocks, 8), XCD x works on row blocks x % S, x % S + S, ... in turn, all column
// blocks and K-slices of one before the next, so the activation slab of a step is fetched into
// that L2 once and the other workgroups of the XCD hit it.  Ids past the end do nothing.
__global__ __launch_bounds__(512, 1) void qlinear_mfma_wide_kernel(QLinearArgs a, int blocks, int row_blocks, int S) {
  extern __shared__ __align__(16) uint16_t smem[];
  const int id = (int)blockIdx.x, xcd = id & 7, idx = id >> 3;
  const int per_rb = blocks * a.nsplit;
  const int p = xcd / S + (8 / S) * idx;
  // an XCD with an even number of row blocks takes them two at a time, the same column block on both in
  // consecutive workgroups, so that a weight tile fetched for one is an L2 hit for the other
  const int R = (row_blocks + S - 1) / S, Gr = (R & 1) ? 1 : 2;
  const int blk = p / (per_rb * Gr), within = p % (per_rb * Gr);
  const int bz = xcd % S + S * (blk * Gr + within % Gr);
  if (bz >= row_blocks) return;
  const int cb = within / Gr, bx = cb % blocks, by = cb / blocks;
  if (bx >= a.n_main_blocks) gemm_block_wide<true>(a, smem, bx, by, bz);
  else gemm_block_wide<false>(a, smem, bx, by, bz);
}

// t16[m][c] = bf16(sum of the planes' values) for c < cols, 0 up to the row stride ldt
__global__ __launch_bounds__(256) void lora_t_reduce_kernel(const float* t_part, int nsplit, int M, int ldt,
                                                            uint16_t* t16, int cols) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= M * ldt) return;
  const int m = i / ldt, c = i - m * ldt;
  float t = 0.f;
  if (c < cols)
    for (int sp = 0; sp < nsplit; ++sp) t += t_part[((size_t)sp * M + m) * ldt + c];
  t16[(size_t)m * ldt + c] = f2bf(t);
}

// part: 0 = main blocks and LoRA blocks in one launch, 1 = LoRA blocks only, 2 = main blocks only
static int launch_qlinear_wide(hipStream_t st, QLinearArgs a, int part = 0) {
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(&qlinear_mfma_wide_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
      (int)KW::LDS);
  if (attr != hipSuccess) return TMX_ERR_LAUNCH;
  a.n_main_blocks = part == 1 ? 0 : (a.N + KW::COLS - 1) / KW::COLS;
  const int blocks = a.n_main_blocks + ((a.a_t && part != 2) ? a.lora_blocks_per_split : 0);
  const int row_blocks = (a.M + KW::ROWS - 1) / KW::ROWS;
  int S = 8;
  while (row_blocks % S) S >>= 1;  // gcd(row_blocks, 8)
  // ids cover 8 / S XCDs x (row_blocks / S) row blocks x blocks x nsplit per residue, rounded up to 8
  const long total = (long)blocks * a.nsplit * row_blocks;
  const int ids = (int)((total + 7) / 8 * 8);
  hipLaunchKernelGGL(qlinear_mfma_wide_kernel, dim3(ids), dim3(512), KW::LDS, st, a, blocks, row_blocks, S);
  return check_launch();
}

// Which kernel serves a projection: narrow ones (fewer than 16 column blocks) with K % 256 == 0
// below 8192 run the 4-wave kernel; everything else a k-way kernel: the direct-to-LDS one when
// K % 256 == 0 (measured faster than the 4-wave kernel on the o, q|k|v, down and unsplit gate|up
// shapes of the 8B and 30B-A3B models at 1, 32, 64 and 128 rows), the plain one otherwise.
static bool four_wave_shape(int K) { return K % 256 == 0 && K < 8192; }
static bool four_wave(int K, int N) { return four_wave_shape(K) && (N + 127) / 128 < 16; }

static int slice_len(int KT, int s) { return ((KT + s - 1) / s + 3) / 4 * 4; }
static bool slices_ok(int KT, int s) { return (KT + slice_len(KT, s) - 1) / slice_len(KT, s) == s; }

// Number of K-slices for a projection: the count that minimises (rounds of workgroups over the
// device's CUs: 256 on the MI355X, also assumed when no device is present) x (steps per slice + fixed
// start-up / reduction work), with a small charge per plane for the f32 traffic of the partial sums.
// No slice may be empty.
// The four-wave kernel: wide projections (column blocks for three quarters of the CUs) are not
// split: they write bf16 directly.  Otherwise the smallest power of two that gives workgroups for
// half of the CUs and at most 32 k-tiles per slice, in whole groups of 4 k-tiles, no empty slice.
static int num_splits4(int K, int N) {
  const int nblocks = (N + 127) / 128;
  const int KT = K / 64;
  const int cus = device_cus();
  if (nblocks >= cus * 3 / 4) return 1;
  int best = 1;
  for (int s = 1; s <= TMX_MAX_SPLITS; s *= 2) {
    if (!slices_ok(KT, s)) break;
    best = s;
    if (nblocks * s >= cus / 2 && slice_len(KT, s) <= 32) break;
  }
  return best;
}

int qlinear_num_lora_splits(int K, int N);
int qlinear_num_splits(int K, int N, int M) {
  if (M > 128) {
    // 256-row blocks: K-slices only while the launch has fewer workgroups than CUs
    const int wgs = (N + 255) / 256 * ((M + 255) / 256);
    int s = 1;
    while (wgs * s < device_cus() * 3 / 4 && s * 2 <= TMX_MAX_SPLITS && slices_ok(K / 64, s * 2) && slice_len(K / 64, s * 2) >= 8) s *= 2;
    return s;
  }
  if (four_wave(K, N)) return num_splits4(K, N);
  const int nblocks = (N + 127) / 128;
  const int KT = K / 64;
  // steps of 4 k-tiles (direct-to-LDS kernel, 128-row k-way kernel) or 8; the workgroups
  // of the LoRA projection share the launch, and a launch that does not fit one workgroup per CU
  // pays a second round (measured: 272 workgroups run slower than 144 with twice the steps); the
  // charge per plane covers the consumer's reads (measured on the o projection: 4 slices beat 6)
  const int ks = (M > 64 || K % 256 == 0) ? 4 : 8;
  const int nls = qlinear_num_lora_splits(K, N);
  const int cus = device_cus();
  int best = 1;
  float best_cost = 1e30f;
  for (int s = 1; s <= TMX_MAX_SPLITS; ++s) {
    if (!slices_ok(KT, s)) continue;
    const int rounds = (nblocks * s + (nls + s - 1) / s * s + cus - 1) / cus;
    const int nsteps = (slice_len(KT, s) + ks - 1) / ks;
    const float cost = rounds * (nsteps + (ks == 4 ? 4.0f : 2.0f)) + (ks == 4 ? 0.6f : 0.15f) * s;
    if (cost < best_cost) { best_cost = cost; best = s; }
  }
  return best;
}

// Number of K-slices of the LoRA projection t = x . A: as fine as whole steps (4 or 8 k-tiles,
// by kernel) allow, at most TMX_MAX_LORA_SPLITS planes, so that no LoRA block outlasts the
// main blocks.
static int lora_step(int K, int N) { return four_wave(K, N) ? 4 : 8; }
int qlinear_num_lora_splits(int K, int N) {
  const int KT = K / 64, g = lora_step(K, N);
  for (int per = g;; per += g) {
    const int n = (KT + per - 1) / per;
    if (n <= TMX_MAX_LORA_SPLITS) return n;
  }
}

static int lora_slice_len(int K, int N) {
  const int KT = K / 64, n = qlinear_num_lora_splits(K, N), g = lora_step(K, N);
  return ((KT + n - 1) / n + g - 1) / g * g;
}

// gate | up projection with the LoRA deltas and SwiGLU in the epilogue: act[M, F] =
// bf16(silu(gate) * up).  Needs the 4-wave kernel (K % 256 == 0, K < 8192) and F % 64 == 0;
// with LoRA: a_t = [A_gate | A_up] in fragment order with r_pad == 32 (2 r <= 32), lora_b [r][2 F].
size_t qlinear_gate_up_sync_bytes(int M, int K) {
  // hand-over state (4 words, 256 bytes reserved) | partial tiles [K / 256][rows / 32][16][64] f32 | t bf16 [rows][32]
  const size_t mt = M <= 32 ? 1 : 2;
  return 256 + (size_t)(K / 256) * mt * 4096 + mt * 32 * 64;
}

// The hand-over mode of the 8-wave kernel: t = x . A by K / 256 extra workgroups of the launch.  The main
// workgroups wait (a bounded number of polls) for the producers, which sit first in dispatch order; the
// launch is kept to one workgroup per compute unit of the device so that no main workgroup can hold a
// unit a producer still needs.
static bool gate_up_handover_shape(int M, int K, int F, int r) {
  return M > 0 && M <= 64 && K % 512 == 0 && K < 8192 && F % 64 == 0 && r > 0 && 2 * r <= 32 && K / 256 <= 32 &&
         F / 64 + K / 256 <= device_cus();
}

size_t qlinear_gate_up_handover_bytes(int M, int K, int F, int r) {
  return gate_up_handover_shape(M, K, F, r) ? qlinear_gate_up_sync_bytes(M, K) : 0;
}

int qlinear_gate_up_swiglu(hipStream_t st, const void* x, int ldx, const void* qw, const void* scales,
                           const void* a_t, const void* lora_b, int r, float ls, void* act, int M, int K,
                           int F, int G, void* sync_ws, uint32_t* status) {
  if (!x || !qw || !scales || !act) return TMX_ERR_ARG;
  if (M <= 0 || M > 128 || !four_wave_shape(K) || F % 64 || G % 64 || (G & (G - 1)) || K % G || ldx % 8)
    return TMX_ERR_SHAPE;
  if (a_t && (!lora_b || r <= 0 || 2 * r > 32)) return TMX_ERR_SHAPE;
  QLinearArgs a = {};
  a.fixed_slice = -1;
  a.x = (const uint16_t*)x;
  a.ldx = ldx;
  a.qw = (const uint4*)qw;
  a.scales = (const uint16_t*)scales;
  a.a_t = (const uint16_t*)a_t;
  a.Rpad = 32;
  a.y_bf16 = (uint16_t*)act;
  a.ldy = F;
  a.M = M; a.K = K; a.N = 2 * F; a.G = G;
  a.nsplit = 1;
  a.kt_per_split = K / 64;
  a.pair_off = F / 32;
  a.lora_b = (const uint16_t*)lora_b;
  a.lora_r = r;
  a.lora_ls = ls;
  a.n_main_blocks = F / 64;
  auto launch = [&](auto kern) {
    hipLaunchKernelGGL(kern, dim3(a.n_main_blocks, 1), dim3(256), 0, st, a);
    return check_launch();
  };
  // up to 64 rows: 8 waves per workgroup, when steps of 8 k-tiles divide K and 32-bit byte
  // offsets reach every operand (128 rows would not fit the register file at 2 waves per SIMD)
  if (M <= 64 && K % 512 == 0 && (size_t)M * ldx * 2 < (1u << 31) && (size_t)K * F < (1u << 31)) {
    if (a_t && sync_ws && gate_up_handover_shape(M, K, F, r)) {
      // t = x . A by K / 256 extra workgroups of the launch, handed to the others through memory
      const int mt = M <= 32 ? 1 : 2;
      a.sync = (uint32_t*)sync_ws;
      a.sync_status = status;
      a.sync_part = (float*)((char*)sync_ws + 256);
      a.sync_t16 = (uint16_t*)((char*)sync_ws + 256 + (size_t)(K / 256) * mt * 4096);
      a.sync_blocks = mt == 1 ? K / 512 : K / 256;  // 8 / MT k-tiles per producer
      return M <= 32 ? launch_gate_up8<1, 2>(st, a) : launch_gate_up8<2, 2>(st, a);
    }
    if (a_t) return M <= 32 ? launch_gate_up8<1, 1>(st, a) : launch_gate_up8<2, 1>(st, a);
    return M <= 32 ? launch_gate_up8<1, 0>(st, a) : launch_gate_up8<2, 0>(st, a);
  }
  if (a_t) {
    if (M <= 32) return launch(qlinear_gate_up_kernel<1>);
    if (M <= 64) return launch(qlinear_gate_up_kernel<2>);
    return launch(qlinear_gate_up_kernel<4>);
  }
  if (M <= 32) return launch(qlinear_mfma4_kernel<1>);
  if (M <= 64) return launch(qlinear_mfma4_kernel<2>);
  return launch(qlinear_mfma4_kernel<4>);
}

// Host-side dispatch shared by the C entry point and the decode-step launcher.
// Output: y_bf16 [M, N] when nsplit == 1 and y_bf16 != null, else y_part
// [nsplit][M][N] f32 planes.  t_part: [qlinear_num_lora_splits(K, N)][M][ldt] f32.
size_t qlinear_delta_sync_bytes(int M, int Rpad) {
  // hand-over state (3 words, 256 bytes reserved) | t bf16 [rows rounded up to 32][Rpad]
  return 256 + (size_t)((M + 31) / 32 * 32) * Rpad * 2;
}

static bool dma_shape(int M, int K, int N, int Rpad, int nsplit, bool lora) {
  const int KT = K / 64;
  return M <= 128 && !four_wave(K, N) && K % 256 == 0 && slices_ok(KT, nsplit) && slice_len(KT, nsplit) % 4 == 0 &&
         (!lora || lora_slice_len(K, N) % 4 == 0) && (size_t)K * N / 2 < (1u << 31) && (size_t)K * Rpad * 2 < (1u << 31);
}

bool qlinear_delta_ok(int M, int K, int N, int Rpad, int r, int nsplit) {
  if (M <= 0 || K % 64 || N % 32 || nsplit < 1 || nsplit > TMX_MAX_SPLITS) return false;
  if (r <= 0 || r > 64 || Rpad <= 0 || Rpad % 32 || Rpad > 128) return false;
  if (!dma_shape(M, K, N, Rpad, nsplit, true)) return false;
  // every workgroup of the launch is resident at once (the LoRA blocks wait for one another): one per CU
  // at 128 rows, two below
  const int nls = qlinear_num_lora_splits(K, N);
  const int lbps = (nls + nsplit - 1) / nsplit;
  const int blocks = ((N + 127) / 128 + lbps) * nsplit;
  if (blocks > device_cus() * (M > 64 ? 1 : 2) || (size_t)M * N * 2 >= (1u << 31)) return false;
  // The stage is a chain of round trips behind the LoRA blocks' own slices (arrive, wait, sum of the planes,
  // tiles: 6 to 10 us); it stays hidden only behind main blocks of at least 8 steps, and with at most two
  // column tiles per wave.  Shorter projections (measured: q|k|v and o of the 8B shape, 4 steps, 14.5 -> 21 us and
  // 13 -> 15.4 us per launch) keep the LoRA product in their consumer.
  return slice_len(K / 64, nsplit) >= 32 && N / 32 <= lbps * nsplit * 8 * 2;
}

int qlinear_base(hipStream_t st, const void* x, int ldx, const void* qw, const void* scales,
                 const void* a_t, void* y_bf16, float* y_part, float* t_part, int ldt, int M, int K,
                 int N, int G, int Rpad, int nsplit, const LoraDelta* ld) {
  if (!x || !qw || !scales || (!y_bf16 && !y_part)) return TMX_ERR_ARG;
  if (M <= 0 || K <= 0 || N <= 0) return TMX_ERR_SHAPE;
  if (K % 64 || N % 32 || G % 64 || (G & (G - 1)) || K % G || (ldx % 8)) return TMX_ERR_SHAPE;
  if (a_t && (!t_part || Rpad <= 0 || Rpad % 32 || Rpad > 128 || ldt < Rpad)) return TMX_ERR_SHAPE;
  if (nsplit < 1 || nsplit > TMX_MAX_SPLITS || (nsplit > 1 && !y_part)) return TMX_ERR_ARG;
  const int KT = K / 64;
  if (!slices_ok(KT, nsplit)) return TMX_ERR_SHAPE;  // an empty K-slice
  QLinearArgs a = {};
  a.fixed_slice = -1;
  a.ldy = N;
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
  const int nls = qlinear_num_lora_splits(K, N);
  a.lora_blocks_per_split = (nls + nsplit - 1) / nsplit;
  a.kt_per_lora_split = lora_slice_len(K, N);
  if (ld) {
    // the LoRA blocks also produce delta = bf16(bf16(t . B) * ls): only the direct-to-LDS kernel does that
    if (!a_t || !ld->delta || !ld->lora_b || !ld->sync_ws) return TMX_ERR_ARG;
    if (!qlinear_delta_ok(M, K, N, Rpad, ld->r, nsplit) || (size_t)M * ldx * 2 >= (1u << 31)) return TMX_ERR_UNSUPPORTED;
    for (int i = 0; i < 3; ++i)
      if (ld->seg_end[i] % 32) return TMX_ERR_SHAPE;
    a.delta = ld->delta;
    a.lora_b = ld->lora_b; a.lora_r = ld->r; a.lora_ls = ld->ls;
    a.seg_end[0] = ld->seg_end[0]; a.seg_end[1] = ld->seg_end[1]; a.seg_end[2] = ld->seg_end[2];
    a.sync = (uint32_t*)ld->sync_ws;
    a.sync_t16 = (uint16_t*)((char*)ld->sync_ws + 256);
    a.sync_status = ld->status;
    a.n_lora_slices = (KT + a.kt_per_lora_split - 1) / a.kt_per_lora_split;  // slices that hold k-tiles
  }
  if (M > 128) {
    // more than 128 rows: the 256-row block (whole 2-tile steps, 32-bit byte offsets per row block)
    if (K % 128 || a.kt_per_split % 2 || (a_t && a.kt_per_lora_split % 2) || (size_t)256 * ldx * 2 >= (1u << 31) ||
        (size_t)K * N / 2 >= (1u << 31) || (size_t)K * Rpad * 2 >= (1u << 31))
      return TMX_ERR_SHAPE;
    return launch_qlinear_wide(st, a);
  }
  if (four_wave(K, N)) {
    if (M <= 32) return launch_qlinear4<1>(st, a);
    if (M <= 64) return launch_qlinear4<2>(st, a);
    return launch_qlinear4<4>(st, a);
  }
  // slices of whole steps, up to 64 rows, 32-bit byte offsets: the direct-to-LDS variant
  if (K % 256 == 0 && a.kt_per_split % 4 == 0 && (!a_t || a.kt_per_lora_split % 4 == 0) &&
      (size_t)M * ldx * 2 < (1u << 31) && (size_t)K * N / 2 < (1u << 31) && (size_t)K * Rpad * 2 < (1u << 31))
    return M <= 32 ? launch_qlinear_dma<1>(st, a) : (M <= 64 ? launch_qlinear_dma<2>(st, a) : launch_qlinear_dma<4>(st, a));
  if (M <= 32) return launch_qlinear<1, 2>(st, a);
  if (M <= 64) return launch_qlinear<2, 2>(st, a);
  return launch_qlinear<4, 2>(st, a);
}

int qlinear_wide_lora(hipStream_t st, const void* x, int ldx, const void* qw, const void* scales, const void* a_t,
                      const void* lora_b, int r, float ls, const int* seg_end, void* y_bf16, float* t_part,
                      uint16_t* t16, int M, int K, int N, int G, int Rpad) {
  if (!x || !qw || !scales || !y_bf16) return TMX_ERR_ARG;
  if (a_t && (!lora_b || !t_part || !t16 || r <= 0)) return TMX_ERR_ARG;
  if (M <= 128 || K % 128 || N % 32 || G % 64 || (G & (G - 1)) || K % G || ldx % 8) return TMX_ERR_SHAPE;
  if (a_t && (r % 8 || r > 64 || Rpad <= 0 || Rpad % 32 || Rpad > TMX_MAX_RPAD)) return TMX_ERR_UNSUPPORTED;
  if (qlinear_num_splits(K, N, M) != 1) return TMX_ERR_UNSUPPORTED;
  if ((size_t)256 * ldx * 2 >= (1u << 31) || (size_t)K * N / 2 >= (1u << 31) || (size_t)K * Rpad * 2 >= (1u << 31))
    return TMX_ERR_SHAPE;
  const int KT = K / 64;
  QLinearArgs a = {};
  a.fixed_slice = -1;
  a.ldy = N;
  a.x = (const uint16_t*)x;
  a.ldx = ldx;
  a.qw = (const uint4*)qw;
  a.scales = (const uint16_t*)scales;
  a.a_t = (const uint16_t*)a_t;
  a.y_bf16 = (uint16_t*)y_bf16;
  a.t_part = t_part;
  a.ldt = TMX_MAX_RPAD;
  a.M = M; a.K = K; a.N = N; a.G = G; a.Rpad = Rpad;
  a.nsplit = 1;
  a.kt_per_split = slice_len(KT, 1);
  const int nls = qlinear_num_lora_splits(K, N);
  a.lora_blocks_per_split = nls;
  a.kt_per_lora_split = lora_slice_len(K, N);
  if (a_t) {
    if (a.kt_per_lora_split % 2) return TMX_ERR_UNSUPPORTED;
    int rc = launch_qlinear_wide(st, a, 1);
    if (rc != TMX_OK) return rc;
    hipLaunchKernelGGL(lora_t_reduce_kernel, dim3((M * TMX_MAX_RPAD + 255) / 256), dim3(256), 0, st, t_part, nls, M,
                       TMX_MAX_RPAD, t16, Rpad);
    if ((rc = check_launch()) != TMX_OK) return rc;
    a.t16 = t16;
    a.ldt16 = TMX_MAX_RPAD;
    a.lora_b = (const uint16_t*)lora_b;
    a.lora_r = r;
    a.lora_ls = ls;
    for (int i = 0; i < 3; ++i) a.seg_end[i] = seg_end ? seg_end[i] : N;
  }
  return launch_qlinear_wide(st, a, 2);
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
    const bf16x8_t b = dequant_word<true>(wd[t], s, -8.f * s);
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
  // f32 K-slice planes, f32 LoRA planes, bf16 LoRA projection (many rows)
  return (s * (size_t)M * N + (size_t)TMX_MAX_LORA_SPLITS * M * TMX_MAX_RPAD) * sizeof(float) +
         (size_t)M * TMX_MAX_RPAD * 2;
}

extern "C" int tmx_qlora_linear_num_splits(int M, int K, int N) { return qlinear_num_splits(K, N, M); }
extern "C" int tmx_qlora_linear_num_lora_splits(int K, int N) { return qlinear_num_lora_splits(K, N); }

extern "C" int tmx_qlora_linear_planes(void* stream, const void* x, const void* qweight,
                                       const void* scales, const void* lora_a_t, float* y_part,
                                       float* t_part, int M, int K, int N, int G, int r_pad, int nsplit) {
  return qlinear_base((hipStream_t)stream, x, K, qweight, scales, lora_a_t, nullptr, y_part, t_part,
                      TMX_MAX_RPAD, M, K, N, G, r_pad, nsplit);
}

// Word of a hand-over workspace (the first 256 bytes are its state block, cleared by the call) that a
// kernel sets when its bounded wait ran out; tmx_handover_status reads it.
static constexpr int kHandoverStatusWord = 63;

extern "C" int tmx_handover_status(void* stream, void* workspace) {
  if (!workspace) return TMX_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  uint32_t flag = 0;
  uint32_t* word = (uint32_t*)workspace + kHandoverStatusWord;
  if (hipMemcpyAsync(&flag, word, 4, hipMemcpyDeviceToHost, st) != hipSuccess) return TMX_ERR_LAUNCH;
  if (hipStreamSynchronize(st) != hipSuccess) return TMX_ERR_LAUNCH;
  if (flag == 0) return TMX_OK;
  int rc = zero_words(st, word, 1);
  if (rc != TMX_OK) return rc;
  if (hipStreamSynchronize(st) != hipSuccess) return TMX_ERR_LAUNCH;
  return TMX_ERR_DEVICE_WAIT;
}

extern "C" size_t tmx_qlora_linear_delta_workspace_bytes(int M, int K, int N, int r, int r_pad, int nsplit) {
  return qlinear_delta_ok(M, K, N, r_pad, r, nsplit) ? qlinear_delta_sync_bytes(M, r_pad) : 0;
}

extern "C" int tmx_qlora_linear_planes_delta(void* stream, const void* x, const void* qweight, const void* scales,
                                             const void* lora_a_t, const void* lora_b, float* y_part, float* t_part,
                                             void* delta, void* workspace, int M, int K, int N, int G, int r,
                                             int r_pad, float lora_scale, int seg_end0, int seg_end1, int nsplit) {
  if (!lora_a_t || !lora_b || !delta || !workspace) return TMX_ERR_ARG;
  LoraDelta ld = {};
  ld.delta = (uint16_t*)delta;
  ld.lora_b = (const uint16_t*)lora_b; ld.r = r; ld.ls = lora_scale;
  ld.seg_end[0] = seg_end0; ld.seg_end[1] = seg_end1; ld.seg_end[2] = N;
  ld.sync_ws = workspace;
  ld.status = (uint32_t*)workspace + kHandoverStatusWord;
  int rc = zero_words((hipStream_t)stream, (uint32_t*)workspace, 64);
  if (rc != TMX_OK) return rc;
  return qlinear_base((hipStream_t)stream, x, K, qweight, scales, lora_a_t, nullptr, y_part, t_part, TMX_MAX_RPAD, M, K, N, G,
                      r_pad, nsplit, &ld);
}

extern "C" int tmx_qlora_linear(void* stream, const void* x, const void* qweight, const void* scales,
                                const void* lora_a_t, const void* lora_b, const void* residual,
                                void* y, void* workspace, int M, int K, int N, int G, int r, int r_pad,
                                float lora_scale) {
  hipStream_t st = (hipStream_t)stream;
  const bool lora = lora_a_t != nullptr;
  if (!workspace || !y) return TMX_ERR_ARG;
  if (lora && (!lora_b || r <= 0 || r > r_pad)) return TMX_ERR_ARG;
  if (M <= 0) return TMX_ERR_SHAPE;
  const int ns = qlinear_num_splits(K, N, M);
  float* y_part = (float*)workspace;
  float* t_part = y_part + (size_t)ns * M * N;
  if (M > 128 && !residual && ns == 1) {
    // many rows, unsplit: LoRA in the projection's epilogue
    uint16_t* t16 = (uint16_t*)(t_part + (size_t)TMX_MAX_LORA_SPLITS * M * TMX_MAX_RPAD);
    const int seg_end[3] = {N, N, N};
    const int rc = qlinear_wide_lora(st, x, K, qweight, scales, lora ? lora_a_t : nullptr, lora_b, r, lora_scale,
                                     seg_end, y, t_part, t16, M, K, N, G, r_pad);
    if (rc != TMX_ERR_UNSUPPORTED) return rc;
  }
  int rc = qlinear_base(st, x, K, qweight, scales, lora ? lora_a_t : nullptr, nullptr, y_part, t_part,
                        TMX_MAX_RPAD, M, K, N, G, r_pad, ns);
  if (rc != TMX_OK) return rc;
  hipLaunchKernelGGL(lora_apply_kernel, dim3((N + 255) / 256, M), dim3(256), 0, st, (uint16_t*)y, y_part,
                     ns, lora ? t_part : nullptr, qlinear_num_lora_splits(K, N), TMX_MAX_RPAD,
                     (const uint16_t*)lora_b, r, lora_scale,
                     (const uint16_t*)residual, M, N);
  return check_launch();
}

// ---------------------------------------------------------------------------
// tmx_qlora_linear for callers that may not allocate (HIP graph capture, serving loops): the
// K-slice planes and LoRA planes live in a file-scope device array instead of a caller workspace.
// Every GPU holds its own copy of the array at its own address; the address is looked up once per
// device, with that device current, and host code only ever uses that pointer (the array's name
// is a host-side stand-in, not a device address).
constexpr size_t kStaticScratchBytes = TMX_STATIC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

static int static_scratch(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return TMX_ERR_LAUNCH;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
      (void)hipGetLastError();
      return TMX_ERR_LAUNCH;
    }
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // racing first calls store the same address
  }
  *out = p;
  return TMX_OK;
}

extern "C" size_t tmx_qlora_linear_noalloc_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int tmx_qlora_linear_noalloc(void* stream, const void* x, const void* qweight, const void* scales,
                                        const void* lora_a_t, const void* lora_b, const void* residual,
                                        void* y, int M, int K, int N, int G, int r, int r_pad,
                                        float lora_scale) {
  if (M <= 0 || K <= 0 || N <= 0) return TMX_ERR_SHAPE;
  if (tmx_qlora_linear_workspace_bytes(M, K, N) > kStaticScratchBytes) return TMX_ERR_SCRATCH;
  void* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc != TMX_OK) return rc;
  // every plane element a consumer reads is written by the projection launch of the same call,
  // so nothing in the array has to start at zero
  return tmx_qlora_linear(stream, x, qweight, scales, lora_a_t, lora_b, residual, y, ws, M, K, N, G, r, r_pad,
                          lora_scale);
}

extern "C" size_t tmx_qlora_gate_up_swiglu_handover_bytes(int M, int K, int F, int r) {
  return qlinear_gate_up_handover_bytes(M, K, F, r);
}

extern "C" int tmx_qlora_gate_up_swiglu_handover(void* stream, const void* x, const void* qweight, const void* scales,
                                                 const void* lora_a_t, const void* lora_b, void* act, void* workspace,
                                                 int M, int K, int F, int G, int r, float lora_scale) {
  if (!lora_a_t || !lora_b || !workspace) return TMX_ERR_ARG;
  if (qlinear_gate_up_handover_bytes(M, K, F, r) == 0) return TMX_ERR_UNSUPPORTED;
  int rc = zero_words((hipStream_t)stream, (uint32_t*)workspace, 64);
  if (rc != TMX_OK) return rc;
  return qlinear_gate_up_swiglu((hipStream_t)stream, x, K, qweight, scales, lora_a_t, lora_b, r, lora_scale, act,
                                M, K, F, G, workspace, (uint32_t*)workspace + kHandoverStatusWord);
}

extern "C" int tmx_qlora_gate_up_swiglu(void* stream, const void* x, const void* qweight, const void* scales,
                                        const void* lora_a_t, const void* lora_b, void* act, int M, int K,
                                        int F, int G, int r, float lora_scale) {
  return qlinear_gate_up_swiglu((hipStream_t)stream, x, K, qweight, scales, lora_a_t, lora_b, r, lora_scale, act,
                                M, K, F, G, nullptr);
}
