// Final projection to the vocabulary fused with log-softmax statistics and token
// selection, so the [B, V] logits never travel through HBM.
//
// Replaces the tail of the model call and Sampler._sample:
//   logits = bf16(x . head) -> f32      tunix/models/llama3/model.py:688-697, :244-246
//                                       tunix/models/qwen3/model.py:1422-1442, :425-429
//   forbidden ids -> -inf               tunix/generate/sampler.py:536-537
//   greedy: argmax, first index on ties tunix/generate/sampler.py:158-168
//   top_p mode with top_p >= 1, no top_k: z = logits / T, token = categorical(
//     fold_in(seed, step), z), logprob = log_softmax(z)[token]
//                                       tunix/generate/sampler.py:112-134, :562
//   token / logprob scatter, done |= isin(token, eos)   tunix/generate/sampler.py:575-581
//
// categorical(key, z) = argmax(z + gumbel), gumbel from threefry2x32 bits over
// the linear index b * V + v (jax's partitionable bit generation).
//
// Mapping: the head matrix [V, D] (bf16, the tied embedding table or the
// transposed lm_head) is the A operand of v_mfma_f32_32x32x16_bf16, the hidden
// states the B operand, so a lane's accumulator registers are 16 vocabulary rows
// of ONE sequence: max / sum-exp / arg-best run down the registers without
// cross-lane traffic.  Workgroup partials are merged by a second tiny kernel.
#include "tmx_kernels.h"
#include "tmx_sampling.h"

namespace tmx {

template <int V>
struct HIC { static constexpr int value = V; };
constexpr int kHXStride = 72;  // bf16 elements per LDS row of the activation tile (64 + 8 pad)

// Scoring (tunix/rl/common.py:217-221, selective_log_softmax): a NaN logit counts as -1e9 and
// the others are clipped to [-1e9, 1e9] before the log-softmax, so the result is always finite.
__device__ __forceinline__ float score_clip(float z) {
  return z != z ? -1e9f : fminf(fmaxf(z, -1e9f), 1e9f);
}

// Workgroup = 4 waves x 32 vocabulary rows.  The hidden-state k-tile x[0:M, 64 kb : 64 kb + 64]
// is fetched once per workgroup, double-buffered in LDS and shared by the waves (MFMA B
// fragments); head rows stream HBM -> registers through a ring of 4 k-tiles per wave.  Lane
// (row, h) reads the 64 contiguous bytes k = 32 h .. 32 h + 31 of its row, so a k-tile of a row
// is one 128-byte line split between two lanes; MFMA step t pairs them with x[.., 32 h + 8 t ..].
// TILED: the same 16-byte pieces from the tile copy of the matrix (head_tiles_kernel), where the
// piece of (k-tile, step t, lane) sits at ((k-tile * 4 + t) * 64 + lane) * 16 of its row tile:
// a wave's load is 1 KiB of consecutive bytes and its whole share of the matrix one contiguous
// stream, read once (non-temporal).  Row-major, one load touches 32 lines of 32 different DRAM
// pages; measured on the 1.05 GB head at 64 rows: 252 us row-major, 190 us from tiles.
template <int MT, bool TILED>
__global__ __launch_bounds__(256, MT == 4 ? 1 : 2) void head_kernel(HeadArgs a) {
  __shared__ __align__(16) uint16_t xs[2][MT * 32][kHXStride];
  __shared__ float s_f[4][MT * 32][4];
  __shared__ int s_i[4][MT * 32];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int h = lane >> 5, nl = lane & 31;
  const int tile = blockIdx.x * 4 + wave;
  const bool live = tile * 32 < a.V;
  const int v0 = live ? tile * 32 : a.V - 32;  // dead waves recompute the last tile (dropped)
  const int KT = a.D >> 6;

  f32x16_t acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[m][r] = 0.f;

  const u32x4_t* wsrc = TILED ? reinterpret_cast<const u32x4_t*>(a.w_tiles + (size_t)v0 * a.D) + lane
                              : reinterpret_cast<const u32x4_t*>(a.w + (size_t)(v0 + nl) * a.D + h * 32);
  const uint16_t* xsrc[MT];
  int xrow_l[MT], xcol_l[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int c = tid + 256 * i;
    xrow_l[i] = c >> 3;
    xcol_l[i] = (c & 7) * 8;
    const int row = xrow_l[i] < a.M ? xrow_l[i] : a.M - 1;
    xsrc[i] = a.x + (size_t)row * a.D + xcol_l[i];
  }
  constexpr int P = 4;
  u32x4_t wring[P][4];
  u32x4_t xring[P][MT];
  const int klast = KT - 1;
  auto load_w = [&](int kb, auto pc) __attribute__((always_inline)) {
    constexpr int p = decltype(pc)::value;
    kb = kb < klast ? kb : klast;
#pragma unroll
    for (int t = 0; t < 4; ++t)
      wring[p][t] = TILED ? __builtin_nontemporal_load(wsrc + (size_t)kb * 256 + t * 64) : wsrc[(size_t)kb * 8 + t];
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
  auto tile_step = [&](int kb, auto pc) __attribute__((always_inline)) {
    constexpr int p = decltype(pc)::value;
    constexpr int p1 = (p + 1) % P;
    bf16x8_t xf[MT][4];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        xf[m][t] = *reinterpret_cast<const bf16x8_t*>(&xs[p & 1][m * 32 + nl][h * 32 + t * 8]);
    u32x4_t wc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) wc[t] = wring[p][t];
    load_w(kb + P, pc);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int m = 0; m < MT; ++m)
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wc[t]), xf[m][t],
                                                         acc[m], 0, 0, 0);
    stash_x((p + 1) & 1, HIC<p1>{});
    load_x(kb + 1 + P, HIC<p1>{});
    __syncthreads();
  };
  load_x(0, HIC<0>{}); load_x(1, HIC<1>{}); load_x(2, HIC<2>{}); load_x(3, HIC<3>{});
  load_w(0, HIC<0>{}); load_w(1, HIC<1>{}); load_w(2, HIC<2>{}); load_w(3, HIC<3>{});
  stash_x(0, HIC<0>{});
  load_x(P, HIC<0>{});
  __syncthreads();
  const int ngroups = KT / P;
  for (int g = 0; g < ngroups; ++g) {
    const int kb = g * P;
    tile_step(kb + 0, HIC<0>{}); tile_step(kb + 1, HIC<1>{});
    tile_step(kb + 2, HIC<2>{}); tile_step(kb + 3, HIC<3>{});
  }
  {
    const int kb = ngroups * P, rem = KT - ngroups * P;
    if (rem > 0) tile_step(kb + 0, HIC<0>{});
    if (rem > 1) tile_step(kb + 1, HIC<1>{});
    if (rem > 2) tile_step(kb + 2, HIC<2>{});
  }

  // per-step key = fold_in(seed, step)
  uint32_t key0 = 0, key1 = 0;
  if (a.mode == TMX_SAMPLE_TOP_P) threefry2x32(a.k0, a.k1, 0u, (uint32_t)*a.step, key0, key1);
  const bool score = a.mode == TMX_SAMPLE_SCORE;

  int target[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    const int row = m * 32 + nl;
    const int tpp = a.tpp > 0 ? a.tpp : 1;
    const int prow = a.row_base + row;  // row of the pass
    target[m] = (score && row < a.M)
                    ? a.token_buffer[(size_t)(prow / tpp) * a.buf_len + min(*a.step + prow % tpp + 1, a.buf_len - 1)] : -1;
  }
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    const int row = m * 32 + nl;
    float mx = kNegBig, se = 0.f;
    Best best = {-INFINITY, -INFINITY, 0x7FFFFFFF};
    if (live && row < a.M) {
      uint64_t packed = 0;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int v = v0 + acc_row(r, lane);
        float logit = rbf(acc[m][r]);
        if (a.logits_out) a.logits_out[(size_t)row * a.V + v] = logit;
        for (int f = 0; f < a.n_forbidden; ++f)
          if (a.forbidden[f] == v) logit = -INFINITY;
        float z = logit, key = logit;
        if (score) {
          // the "best" candidate is the given next token: its z is what the log-prob needs
          z = score_clip(rbf(logit / a.temperature));  // bf16 logits divided in place stay bf16 (rl/common.py:591-592)
          key = (v == target[m]) ? 0.f : -INFINITY;
        } else if (a.mode == TMX_SAMPLE_TOP_P) {
          z = logit / a.temperature;
          if (a.sort_keys) {
            // 16-bit key whose ascending order is the descending order of the logit (= of z, T > 0;
            // -0 counts as +0): non-negative values count down from 0x7FFF, negative ones up from 0x8000
            const uint32_t zb = __float_as_uint(logit + 0.0f) >> 16;
            // registers 4 q .. 4 q + 3 hold four consecutive vocabulary rows: one 8-byte store
            packed |= (uint64_t)((zb & 0x8000u) ? zb : (~zb & 0x7FFFu)) << (16 * (r & 3));
            if ((r & 3) == 3) {
              *reinterpret_cast<uint64_t*>(a.sort_keys + (size_t)row * a.V + v - 3) = packed;
              packed = 0;
            }
            key = z;
          } else {
            uint32_t o0, o1;
            threefry2x32(key0, key1, 0u, (uint32_t)(a.row_off + row) * (uint32_t)a.V + (uint32_t)v, o0, o1);
            key = z + gumbel_from_bits(o0 ^ o1);
          }
        }
        if (z > mx) {
          se = se * expf(mx - z) + 1.f;
          mx = z;
        } else {
          se += expf(z - mx);
        }
        Best c = {key, z, v};
        best_merge(best, c);
      }
    }
    // the other half-wave holds the other 16 vocabulary rows of the same sequence
    {
      const float mx2 = __shfl_xor(mx, 32, 64), se2 = __shfl_xor(se, 32, 64);
      Best o = {__shfl_xor(best.key, 32, 64), __shfl_xor(best.z, 32, 64), __shfl_xor(best.idx, 32, 64)};
      lse_merge(mx, se, mx2, se2);
      best_merge(best, o);
    }
    if (h == 0) {
      s_f[wave][row][0] = mx;
      s_f[wave][row][1] = se;
      s_f[wave][row][2] = best.key;
      s_f[wave][row][3] = best.z;
      s_i[wave][row] = best.idx;
    }
  }
  __syncthreads();
  for (int row = threadIdx.x; row < MT * 32; row += 256) {
    if (row >= a.M) continue;
    float mx = s_f[0][row][0], se = s_f[0][row][1];
    Best best = {s_f[0][row][2], s_f[0][row][3], s_i[0][row]};
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      lse_merge(mx, se, s_f[w][row][0], s_f[w][row][1]);
      Best o = {s_f[w][row][2], s_f[w][row][3], s_i[w][row]};
      best_merge(best, o);
    }
    float* pf = a.part_f + ((size_t)row * a.nwg + blockIdx.x) * 4;
    pf[0] = mx; pf[1] = se; pf[2] = best.key; pf[3] = best.z;
    a.part_i[(size_t)row * a.nwg + blockIdx.x] = best.idx;
  }
}

// The tile copy of the head matrix: row tile vt (32 vocabulary rows) x k-tile kt (64 columns) is 4 KiB at
// (vt * D / 64 + kt) * 4 KiB, and in it the 16 bytes W[32 vt + nl][64 kt + 32 h + 8 t .. + 7] sit at
// (t * 64 + 32 h + nl) * 16: what lane (nl, h) of head_kernel feeds to MFMA step t.  One workgroup per tile.
__global__ __launch_bounds__(256) void head_tiles_kernel(const uint16_t* __restrict__ w, uint16_t* __restrict__ tiles,
                                                         int D) {
  const int kt = blockIdx.x, vt = blockIdx.y, KT = D >> 6;
  const int t = threadIdx.x >> 6, lane = threadIdx.x & 63, h = lane >> 5, nl = lane & 31;
  const u32x4_t v = *reinterpret_cast<const u32x4_t*>(w + (size_t)(32 * vt + nl) * D + 64 * kt + 32 * h + 8 * t);
  reinterpret_cast<u32x4_t*>(tiles)[((size_t)vt * KT + kt) * 256 + t * 64 + lane] = v;
}

int head_tiles_pack(hipStream_t st, const uint16_t* w, uint16_t* tiles, int V, int D) {
  if (V <= 0 || D <= 0 || V % 32 || D % 64 || V / 32 > 65535) return TMX_ERR_SHAPE;
  hipLaunchKernelGGL(head_tiles_kernel, dim3(D / 64, V / 32), dim3(256), 0, st, w, tiles, D);
  return check_launch();
}

// One workgroup per sequence: merge the vocabulary-tile partials, emit the token
// and its log-probability into column step + 1, update `done`.
__global__ __launch_bounds__(256) void head_finalize_kernel(HeadArgs a) {
  __shared__ float s_f[4][4];
  __shared__ int s_i[4];
  const int row = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float mx = kNegBig, se = 0.f;
  Best best = {-INFINITY, -INFINITY, 0x7FFFFFFF};
  for (int i = threadIdx.x; i < a.nwg; i += 256) {
    const float* pf = a.part_f + ((size_t)row * a.nwg + i) * 4;
    lse_merge(mx, se, pf[0], pf[1]);
    Best o = {pf[2], pf[3], a.part_i[(size_t)row * a.nwg + i]};
    best_merge(best, o);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float mx2 = __shfl_xor(mx, off, 64), se2 = __shfl_xor(se, off, 64);
    Best o = {__shfl_xor(best.key, off, 64), __shfl_xor(best.z, off, 64), __shfl_xor(best.idx, off, 64)};
    lse_merge(mx, se, mx2, se2);
    best_merge(best, o);
  }
  if (lane == 0) {
    s_f[wave][0] = mx; s_f[wave][1] = se; s_f[wave][2] = best.key; s_f[wave][3] = best.z;
    s_i[wave] = best.idx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    mx = s_f[0][0]; se = s_f[0][1];
    best = {s_f[0][2], s_f[0][3], s_i[0]};
    for (int w = 1; w < 4; ++w) {
      lse_merge(mx, se, s_f[w][0], s_f[w][1]);
      Best o = {s_f[w][2], s_f[w][3], s_i[w]};
      best_merge(best, o);
    }
    if (a.mode == TMX_SAMPLE_SCORE) {  // teacher forcing: the token stays, only its log-prob is written
      const int tpp = a.tpp > 0 ? a.tpp : 1;
      const int prow = a.row_base + row;
      // selective_log_softmax: logit - logsumexp, with logsumexp = max + log(sum exp(z - max))
      const int scol = *a.step + prow % tpp + 1;
      if (a.logprobs && scol < a.buf_len)
        a.logprobs[(size_t)(prow / tpp) * a.buf_len + scol] = best.z - (mx + logf(se));
      return;
    }
    const int col = *a.step + 1;
    if (col >= a.buf_len) return;  // a caller that steps past the buffer gets no write instead of a stray one
    const int tok = best.idx;
    a.token_buffer[(size_t)row * a.buf_len + col] = tok;
    if (a.logprobs) a.logprobs[(size_t)row * a.buf_len + col] = (best.z - mx) - logf(se);
    bool hit = false;
    for (int e = 0; e < a.n_eos; ++e) hit = hit || (a.eos[e] == tok);
    if (hit) a.done[row] = 1;
  }
}

// ---------------------------------------------------------------------------
// Many rows (scoring passes over whole sequences, decode steps of more than 128 sequences): the same
// product as a matrix-pipe-bound kernel.  A workgroup multiplies 256 vocabulary rows by 256 sequence rows:
// the vocabulary rows are the A operand and come through a double-buffered LDS slab filled by
// direct-to-LDS loads (256-byte rows of a 128-wide k-step, chunks XOR-swizzled by row % 16);
// wave w owns sequence rows 32 w .. 32 w + 31 as the B operand, read straight from global
// memory, 64 contiguous bytes per lane and k-tile (lane (row, h) holds k = 32 h .. 32 h + 31 of
// the tile, MFMA step t pairs k = 32 h + 8 t .. with the same k of the vocabulary rows).  A lane's
// 128 accumulator registers are 128 vocabulary rows of ONE sequence row, so max / sum-exp / the
// target's z run down the registers.  LDS reads of fragment group g + 1 and the refill of the
// B registers are pinned between the MFMAs of group g.  Consecutive workgroups take the
// sequence-row blocks of one vocabulary block, so the head matrix leaves HBM once.
struct HW {
  static constexpr int MT = 8, ROWS = 256, TS = 2, XS = 128;
  static constexpr size_t LDS = (size_t)2 * ROWS * XS * 2;  // 128 KiB
};

template <int MODE>  // TMX_SAMPLE_*: the epilogue is compiled per mode
__global__ __launch_bounds__(512, 1) void head_wide_kernel(HeadArgs a, int tok_blocks, int voc_blocks) {
  extern __shared__ __align__(16) uint16_t smem[];
  constexpr int MT = HW::MT, TS = HW::TS, XS = HW::XS, ROWS = HW::ROWS;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, nl = lane & 31;
  const int vb = (int)blockIdx.x / tok_blocks, tb = (int)blockIdx.x % tok_blocks;
  if (vb >= voc_blocks) return;
  const int v0 = vb * ROWS;
  const int vrows = a.V - v0 < ROWS ? a.V - v0 : ROWS;
  const int tok = tb * 256 + wave * 32 + nl;       // sequence row of this lane's accumulator column
  const int tok_l = tok < a.M ? tok : a.M - 1;
  const int nsteps = a.D >> 7, last_step = nsteps - 1;

  const __amdgpu_buffer_rsrc_t rw = make_rsrc(a.w + (size_t)v0 * a.D, (uint32_t)vrows * a.D * 2u);
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(a.x, (uint32_t)a.M * a.D * 2u);
  constexpr int XR = ROWS / 32;
  int woff[XR];  // slab transfer: load i moves vocabulary rows 4 wave + 32 i .. + 3, 16 lanes each
#pragma unroll
  for (int i = 0; i < XR; ++i) {
    const int row_l = 4 * wave + 32 * i + (lane >> 4);
    woff[i] = (row_l < vrows ? row_l : vrows - 1) * a.D * 2 + (((lane & 15) ^ (row_l & 15)) * 16);
  }
  const int xv = tok_l * a.D * 2 + h * 64;

  f32x16_t acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[m][r] = 0.f;
  u32x4_t breg[4 * TS];  // B fragments of the 8 groups of a step, refilled for the next step after use

  auto load_b = [&](int step, auto gc) __attribute__((always_inline)) {
    constexpr int g = decltype(gc)::value;
    step = step < last_step ? step : last_step;
    breg[g] = __builtin_amdgcn_raw_buffer_load_b128(rx, xv + (g & 3) * 16, (step * TS + (g >> 2)) * 128, 0);
  };
  auto dma_w = [&](int step, int buf) __attribute__((always_inline)) {
    step = step < last_step ? step : last_step;
    uint16_t* base = smem + (size_t)buf * ROWS * XS + wave * 4 * XS;
#pragma unroll
    for (int i = 0; i < XR; ++i) load_row_to_lds_nt(rw, base + i * 32 * XS, woff[i], step * (TS * 128));
  };
  constexpr int kYounger = 4 * TS;
  auto wait_slab = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0F70 | (kYounger & 15) | ((kYounger >> 4) << 14));
    __syncthreads();
  };
  auto step_math = [&](int step, int buf) __attribute__((always_inline)) {
    const uint16_t* wb = smem + (size_t)buf * ROWS * XS + nl * XS;
    bf16x8_t wq[2][MT];
    {
      // group g = 4 j + t needs k = 64 j + 32 h + 8 t ..: chunk 8 j + 4 h + t of the slab row
      const int slot = ((4 * h) ^ (nl & 15)) * 8;
#pragma unroll
      for (int m = 0; m < MT; ++m) wq[0][m] = *reinterpret_cast<const bf16x8_t*>(wb + m * 32 * XS + slot);
    }
    __builtin_amdgcn_sched_barrier(0);
    static_for<4 * TS>([&](auto gc) __attribute__((always_inline)) {
      constexpr int g = decltype(gc)::value, cur = g & 1, nxt = cur ^ 1;
      constexpr bool more = g + 1 < 4 * TS;
      constexpr int gn = g + 1;
      const int slot = ((8 * (gn >> 2) + 4 * h + (gn & 3)) ^ (nl & 15)) * 8;
      const bf16x8_t b = __builtin_bit_cast(bf16x8_t, breg[g]);
      static_for<MT>([&](auto mc) __attribute__((always_inline)) {
        constexpr int m = decltype(mc)::value;
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wq[cur][m], b, acc[m], 0, 0, 0);
        if constexpr (more) {
          wq[nxt][m] = *reinterpret_cast<const bf16x8_t*>(wb + m * 32 * XS + slot);
          __builtin_amdgcn_sched_barrier(0);
        }
      });
      load_b(step + 1, gc);  // fragment consumed: refill it for the next step
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  dma_w(0, 0);
  static_for<4 * TS>([&](auto gc) __attribute__((always_inline)) { load_b(0, gc); });
  wait_slab();
  for (int step = 0; step < nsteps; ++step) {
    const int buf = step & 1;
    dma_w(step + 1, buf ^ 1);
    __builtin_amdgcn_sched_barrier(0);
    step_math(step, buf);
    wait_slab();
  }

  // per sequence row: running max and sum of exp over this block's vocabulary rows and the best
  // candidate by key, as in head_kernel: greedy key = logit; sampling key = z + Gumbel noise of the
  // counter row * V + v; scoring: the given next token (key 0 marks it)
  constexpr bool score = MODE == TMX_SAMPLE_SCORE, sampling = MODE == TMX_SAMPLE_TOP_P;
  uint32_t key0 = 0, key1 = 0;
  if (sampling) threefry2x32(a.k0, a.k1, 0u, (uint32_t)*a.step, key0, key1);
  const int tpp = a.tpp > 0 ? a.tpp : 1;
  const int target = score ? a.token_buffer[(size_t)(tok_l / tpp) * a.buf_len + min(*a.step + tok_l % tpp + 1, a.buf_len - 1)] : -1;
  float mx = kNegBig, se = 0.f;
  Best best = {-INFINITY, -INFINITY, 0x7FFFFFFF};
  uint64_t packed = 0;  // sorting branch: the 16-bit keys of four consecutive vocabulary rows
  const bool keys_out = sampling && a.sort_keys != nullptr && tok < a.M;
  // (unrolled by construction: a loop the compiler declines to unroll would index the accumulators
  // dynamically and move them to scratch memory)
  static_for<MT * 16>([&](auto ic) __attribute__((always_inline)) {
      constexpr int m = decltype(ic)::value / 16, r = decltype(ic)::value % 16;
      const int v = v0 + m * 32 + acc_row(r, lane);
      if (v >= a.V) return;  // (V % 32 == 0 where keys are written: a group of four rows is in or out as one)
      const float logit = rbf(acc[m][r]);
      float z = logit, key = logit;
      if (score) {
        z = score_clip(rbf(logit / a.temperature));  // bf16 logits divided in place stay bf16 (rl/common.py:591-592)
        key = (v == target) ? 0.f : -INFINITY;
      } else if (sampling) {
        z = logit / a.temperature;
        if (a.sort_keys) {
          // the same 16-bit descending key as head_kernel writes (selection happens in nucleus.hip)
          if (keys_out) {
            const uint32_t zb = __float_as_uint(logit + 0.0f) >> 16;
            packed |= (uint64_t)((zb & 0x8000u) ? zb : (~zb & 0x7FFFu)) << (16 * (r & 3));
            if constexpr ((r & 3) == 3) {
              *reinterpret_cast<uint64_t*>(a.sort_keys + (size_t)tok * a.V + v - 3) = packed;
              packed = 0;
            }
          }
          key = z;
        } else {
          uint32_t o0, o1;
          threefry2x32(key0, key1, 0u, (uint32_t)tok_l * (uint32_t)a.V + (uint32_t)v, o0, o1);
          key = z + gumbel_from_bits(o0 ^ o1);
        }
      }
      if (z > mx) {
        se = se * expf(mx - z) + 1.f;
        mx = z;
      } else {
        se += expf(z - mx);
      }
      if (score) {
        if (v == target) best = {0.f, z, v};  // at most one vocabulary row is the target
      } else {
        Best c = {key, z, v};
        best_merge(best, c);
      }
  });
  {
    const float mx2 = __shfl_xor(mx, 32, 64), se2 = __shfl_xor(se, 32, 64);
    Best o = {__shfl_xor(best.key, 32, 64), __shfl_xor(best.z, 32, 64), __shfl_xor(best.idx, 32, 64)};
    lse_merge(mx, se, mx2, se2);
    best_merge(best, o);
  }
  if (h == 0 && tok < a.M) {
    float* pf = a.part_f + ((size_t)tok * a.nwg + vb) * 4;
    pf[0] = mx; pf[1] = se; pf[2] = best.key; pf[3] = best.z;
    a.part_i[(size_t)tok * a.nwg + vb] = best.idx;
  }
}

// M rows (any count) with the wide kernel + the finalize kernel: greedy, sampling without the sorting
// branch, or scoring; the caller has checked: no forbidden ids, no logits output, D % 128 == 0.
template <int MODE>
static int launch_head_wide(hipStream_t st, const HeadArgs& a, int tok_blocks, int voc_blocks) {
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(&head_wide_kernel<MODE>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)HW::LDS);
  if (attr != hipSuccess) return TMX_ERR_LAUNCH;
  hipLaunchKernelGGL(head_wide_kernel<MODE>, dim3(tok_blocks * voc_blocks), dim3(512), HW::LDS, st, a, tok_blocks,
                     voc_blocks);
  return TMX_OK;
}

bool head_wide_ok(const HeadArgs& a) {
  return a.D % 128 == 0 && a.M > 0 && (size_t)a.M * a.D * 2 < (1u << 31) && (size_t)256 * a.D * 2 < (1u << 31) &&
         a.n_forbidden == 0 && !a.logits_out;
}

// The wide kernel alone: partials (and, in the sorting branch, keys) of every row; sets a.nwg.
int head_wide_logits(hipStream_t st, HeadArgs& a) {
  if (!head_wide_ok(a)) return TMX_ERR_SHAPE;
  const int tok_blocks = (a.M + 255) / 256, voc_blocks = (a.V + HW::ROWS - 1) / HW::ROWS;
  a.nwg = voc_blocks;
  a.row_base = 0;
  int lrc;
  if (a.mode == TMX_SAMPLE_SCORE) lrc = launch_head_wide<TMX_SAMPLE_SCORE>(st, a, tok_blocks, voc_blocks);
  else if (a.mode == TMX_SAMPLE_TOP_P) lrc = launch_head_wide<TMX_SAMPLE_TOP_P>(st, a, tok_blocks, voc_blocks);
  else lrc = launch_head_wide<TMX_SAMPLE_GREEDY>(st, a, tok_blocks, voc_blocks);
  if (lrc != TMX_OK) return lrc;
  return check_launch();
}

int head_wide(hipStream_t st, HeadArgs a) {
  int rc = head_wide_logits(st, a);
  if (rc != TMX_OK) return rc;
  hipLaunchKernelGGL(head_finalize_kernel, dim3(a.M), dim3(256), 0, st, a);
  return check_launch();
}

int head_logits(hipStream_t st, HeadArgs& a) {
  if (a.V % 32 || a.D % 64 || a.M <= 0 || a.M > TMX_MAX_FILL_ROWS) return TMX_ERR_SHAPE;
  a.nwg = (a.V + 127) / 128;
  // Rows go through the 32- or 64-row kernel in chunks of 64: one pass over the head matrix per chunk.
  // (A 128-row instantiation ran 0.87 ms on a 1 GB head against 2 x 0.27 ms: one workgroup per CU, its
  // x tile and weight ring no longer hide the latencies.)  The partials of every chunk sit where one
  // finalize launch over all rows expects them.
  for (int r0 = 0; r0 < a.M; r0 += 64) {
    HeadArgs c = a;
    c.M = a.M - r0 < 64 ? a.M - r0 : 64;
    c.x = a.x + (size_t)r0 * a.D;
    c.row_base = a.row_base + r0;
    c.row_off = a.row_off + r0;
    if (a.logits_out) c.logits_out = a.logits_out + (size_t)r0 * a.V;
    if (a.sort_keys) c.sort_keys = a.sort_keys + (size_t)r0 * a.V;
    c.part_f = a.part_f + (size_t)r0 * a.nwg * 4;
    c.part_i = a.part_i + (size_t)r0 * a.nwg;
    if (c.w_tiles) {
      if (c.M <= 32) hipLaunchKernelGGL((head_kernel<1, true>), dim3(a.nwg), dim3(256), 0, st, c);
      else hipLaunchKernelGGL((head_kernel<2, true>), dim3(a.nwg), dim3(256), 0, st, c);
    } else {
      if (c.M <= 32) hipLaunchKernelGGL((head_kernel<1, false>), dim3(a.nwg), dim3(256), 0, st, c);
      else hipLaunchKernelGGL((head_kernel<2, false>), dim3(a.nwg), dim3(256), 0, st, c);
    }
  }
  return check_launch();
}

int head_sample(hipStream_t st, HeadArgs a) {
  int rc = head_logits(st, a);
  if (rc != TMX_OK) return rc;
  hipLaunchKernelGGL(head_finalize_kernel, dim3(a.M), dim3(256), 0, st, a);
  return check_launch();
}

size_t head_partial_bytes(int M, int V) {
  const size_t nwg = (V + 127) / 128;
  return (size_t)M * nwg * 5 * sizeof(float);
}

}  // namespace tmx

using namespace tmx;

extern "C" size_t tmx_head_sample_workspace_bytes(int M, int V) { return head_partial_bytes(M, V); }

static int head_sample_entry(void* stream, const void* x, const void* head_w, const void* head_tiles, int M, int D,
                             int V, int mode, float temperature, uint32_t seed_hi, uint32_t seed_lo,
                             const int32_t* step, const int32_t* forbidden, int n_forbidden,
                             const int32_t* eos, int n_eos, int32_t* token_buffer, float* logprobs,
                             uint8_t* done, int buf_len, float* logits_out, void* workspace) {
  if (!x || (!head_w && !head_tiles) || !step || !token_buffer || !done || !workspace) return TMX_ERR_ARG;
  if ((n_forbidden > 0 && !forbidden) || (n_eos > 0 && !eos)) return TMX_ERR_ARG;
  if (mode != TMX_SAMPLE_GREEDY && mode != TMX_SAMPLE_TOP_P && mode != TMX_SAMPLE_SCORE) return TMX_ERR_UNSUPPORTED;
  HeadArgs a = {};
  a.x = (const uint16_t*)x;
  a.w = (const uint16_t*)head_w;
  a.w_tiles = (const uint16_t*)head_tiles;
  a.M = M; a.D = D; a.V = V;
  a.mode = mode;
  a.temperature = temperature;
  a.k0 = seed_hi; a.k1 = seed_lo;
  a.step = step;
  a.forbidden = forbidden; a.n_forbidden = n_forbidden;
  a.logits_out = logits_out;
  const size_t nwg = (V + 127) / 128;
  a.part_f = (float*)workspace;
  a.part_i = (int32_t*)((float*)workspace + (size_t)M * nwg * 4);
  a.token_buffer = token_buffer;
  a.logprobs = logprobs;
  a.done = done;
  a.eos = eos; a.n_eos = n_eos;
  a.buf_len = buf_len;
  return head_sample((hipStream_t)stream, a);
}

extern "C" int tmx_head_sample(void* stream, const void* x, const void* head_w, int M, int D, int V,
                               int mode, float temperature, uint32_t seed_hi, uint32_t seed_lo,
                               const int32_t* step, const int32_t* forbidden, int n_forbidden,
                               const int32_t* eos, int n_eos, int32_t* token_buffer, float* logprobs,
                               uint8_t* done, int buf_len, float* logits_out, void* workspace) {
  return head_sample_entry(stream, x, head_w, nullptr, M, D, V, mode, temperature, seed_hi, seed_lo, step, forbidden,
                           n_forbidden, eos, n_eos, token_buffer, logprobs, done, buf_len, logits_out, workspace);
}

extern "C" int tmx_head_sample_tiles(void* stream, const void* x, const void* head_tiles, int M, int D, int V,
                                     int mode, float temperature, uint32_t seed_hi, uint32_t seed_lo,
                                     const int32_t* step, const int32_t* forbidden, int n_forbidden,
                                     const int32_t* eos, int n_eos, int32_t* token_buffer, float* logprobs,
                                     uint8_t* done, int buf_len, float* logits_out, void* workspace) {
  if (!head_tiles) return TMX_ERR_ARG;
  return head_sample_entry(stream, x, nullptr, head_tiles, M, D, V, mode, temperature, seed_hi, seed_lo, step,
                           forbidden, n_forbidden, eos, n_eos, token_buffer, logprobs, done, buf_len, logits_out,
                           workspace);
}

extern "C" int tmx_head_tiles_pack(void* stream, const void* head_w, void* head_tiles, int V, int D) {
  if (!head_w || !head_tiles) return TMX_ERR_ARG;
  return head_tiles_pack((hipStream_t)stream, (const uint16_t*)head_w, (uint16_t*)head_tiles, V, D);
}
