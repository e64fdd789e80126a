// GQA decode attention over the KV cache: one query token per sequence.
//
// Replaces, for T = 1, tunix/models/llama3/model.py:379-396 and
// tunix/models/qwen3/model.py:776-793 together with the decode mask of
// tunix/generate/utils.py:35-59: position j may be attended iff j <= step and
// input_mask[b, j].  The reference evaluates a masked softmax over the whole
// cache_size; masked scores there are K_MASK and contribute exp(K_MASK - max) = 0,
// so reading only j <= step gives the same probabilities.
//
// Mapping: a workgroup (4 waves) owns one (sequence, kv head, split) and streams
// K and V rows of 2*H bytes straight from HBM into registers: H/8 lanes share a
// row (16 bytes per lane), so one wave-wide load covers 64/(H/8) positions and
// every row is a fully coalesced 128- or 256-byte segment.  All G = N/Kh query
// heads of the group reuse the K/V registers.  Scores are reduced across the
// lanes of a row with DPP adds; every lane group keeps its own online-softmax
// state (max, sum, output slice) and the states are merged once at the end.
#include "tmx_kernels.h"

namespace tmx {

constexpr int kMaxPrefixSplits = 4;  // splits of the slots that a group of sequences shares

// waves per workgroup: fewer for wide groups so the merge buffers stay under 64 KiB
template <int G>
struct AttnWaves { static constexpr int value = G > 4 ? 2 : 4; };

// LDS of the one-token walk: merge buffers of the NG lane groups of a workgroup
template <int H, int G>
struct DecodeLds {
  static constexpr int NW = AttnWaves<G>::value;
  static constexpr int NG = NW * (64 / (H / 8));
  float m[NG][G], l[NG][G];
  float acc[NG][G][H];
};

template <int H, int G>
__device__ __forceinline__ void gqa_decode_walk(const AttnArgs& a, DecodeLds<H, G>& lds, const int kvh, const int b,
                                                const int split) {
  constexpr int NW = AttnWaves<G>::value;
  constexpr int LPP = H / 8;     // lanes per position row
  constexpr int PPW = 64 / LPP;  // positions per wave-wide load
  constexpr int U = 4;           // positions per lane group per iteration
  constexpr int NG = NW * PPW;   // lane groups per workgroup
  auto& s_m = lds.m;
  auto& s_l = lds.l;
  auto& s_acc = lds.acc;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pg = lane / LPP, dl = lane % LPP;  // lane group, 8-element slice index
  const int tpp = a.tpp > 0 ? a.tpp : 1;
  const int seq = b / tpp;                    // b: query row of this pass
  // newest valid slot; clamped into the cache and the mask row so that a caller that oversteps reads in bounds
  const int step = min(*a.step + b % tpp, min(a.C, a.buf_len) - 1);
  // the splits share the VALID positions base .. step (not the cache size) in chunks of whole
  // 32 positions, so that every split has work at any context length; base > 0: the slots below it
  // are shared by a group of sequences and walked once per group by the tile walk (gqa_shared_kernel)
  const int base = a.share_gs > 1 ? min(a.share_len, step + 1) : 0;
  const int chunk = (((step - base + a.nsplit) / a.nsplit) + 31) & ~31;
  const int s_begin = base + split * chunk;
  int s_end = s_begin + chunk;
  if (s_end > step + 1) s_end = step + 1;
  const int nparts = a.nsplit + a.psplits;  // partial results per row to be merged

  // query fragments for the G heads of this kv head: 8 bf16 = 4 packed pairs each
  uint32_t qf[G][4];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const uint4 v = *reinterpret_cast<const uint4*>(a.q + ((size_t)b * a.N + kvh * G + g) * H + dl * 8);
    qf[g][0] = v.x; qf[g][1] = v.y; qf[g][2] = v.z; qf[g][3] = v.w;
  }
  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -1e30f;
    l[g] = 0.f;
#pragma unroll
    for (int d = 0; d < 8; ++d) acc[g][d] = 0.f;
  }
  const size_t row_stride = (size_t)a.Kh * H;  // elements between consecutive positions
  const uint16_t* kbase = a.kcache + ((size_t)seq * a.C * a.Kh + kvh) * H + dl * 8;
  const uint16_t* vbase = a.vcache + ((size_t)seq * a.C * a.Kh + kvh) * H + dl * 8;
  const uint8_t* mrow = a.input_mask + (size_t)seq * a.buf_len;

  // lane group (wave, pg) takes positions s_begin + (it * NG + wave * PPW + pg) * U + u
  for (int p0 = s_begin + (wave * PPW + pg) * U; p0 < s_end; p0 += NG * U) {
    uint4 kr[U], vr[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = p0 + u;
      ok[u] = p < s_end;
      const int pc = ok[u] ? p : p0;
      // K/V rows are read once per step: non-temporal loads (measured: a plain streaming read reaches
      // 5.6-6.2 TB/s on this part, a non-temporal one 6.3-7.0)
      const u32x4_t k4 = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(kbase + (size_t)pc * row_stride));
      const u32x4_t v4 = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(vbase + (size_t)pc * row_stride));
      kr[u] = make_uint4(k4.x, k4.y, k4.z, k4.w);
      vr[u] = make_uint4(v4.x, v4.y, v4.z, v4.w);
      ok[u] = ok[u] && mrow[pc] != 0;
    }
    float sc[U][G];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t kw[4] = {kr[u].x, kr[u].y, kr[u].z, kr[u].w};
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float d = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, qf[g][j]),
                                              __builtin_bit_cast(bf16x2_t, kw[j]), d, false);
        d = group_sum<LPP>(d);
        sc[u][g] = ok[u] ? d * a.scale : -1e30f;
      }
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float mn = m[g];
#pragma unroll
      for (int u = 0; u < U; ++u) mn = fmaxf(mn, sc[u][g]);
      const float alpha = __expf(m[g] - mn);
      m[g] = mn;
      float pw[U], ps = 0.f;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        pw[u] = ok[u] ? __expf(sc[u][g] - mn) : 0.f;
        ps += pw[u];
      }
      l[g] = l[g] * alpha + ps;
#pragma unroll
      for (int d = 0; d < 8; ++d) acc[g][d] *= alpha;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t vw[4] = {vr[u].x, vr[u].y, vr[u].z, vr[u].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[g][2 * j] = fmaf(pw[u], bf_lo(vw[j]), acc[g][2 * j]);
          acc[g][2 * j + 1] = fmaf(pw[u], bf_hi(vw[j]), acc[g][2 * j + 1]);
        }
      }
    }
  }

  // merge the NG lane-group states
  const int gi = wave * PPW + pg;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    if (dl == 0) {
      s_m[gi][g] = m[g];
      s_l[gi][g] = l[g];
    }
#pragma unroll
    for (int d = 0; d < 8; ++d) s_acc[gi][g][dl * 8 + d] = acc[g][d];
  }
  __syncthreads();
  for (int e = threadIdx.x; e < G * H; e += NW * 64) {
    const int g = e / H, d = e % H;
    float mm = -1e30f;
#pragma unroll
    for (int i = 0; i < NG; ++i) mm = fmaxf(mm, s_m[i][g]);
    float ls = 0.f, o = 0.f;
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const float w = __expf(s_m[i][g] - mm);
      ls += s_l[i][g] * w;
      o += s_acc[i][g][d] * w;
    }
    if (nparts == 1) {
      a.out[((size_t)b * a.N + kvh * G + g) * H + d] = f2bf(ls > 0.f ? o / ls : 0.f);
    } else {
      float* pr = a.partial + ((((size_t)b * a.Kh + kvh) * nparts + split) * G + g) * (H + 2);
      pr[d] = o;
      if (d == 0) {
        pr[H] = mm;
        pr[H + 1] = ls;
      }
    }
  }
}

template <int H, int G>
__global__ __launch_bounds__(AttnWaves<G>::value * 64, 4) void gqa_decode_kernel(AttnArgs a) {
  __shared__ DecodeLds<H, G> lds;
  gqa_decode_walk<H, G>(a, lds, blockIdx.x, blockIdx.y, blockIdx.z);
}

template <int H, int G>
__global__ __launch_bounds__(H) void gqa_combine_kernel(AttnArgs a) {
  const int kvh = blockIdx.x, b = blockIdx.y, g = blockIdx.z, d = threadIdx.x;
  const int nparts = a.nsplit + a.psplits;
  const float* pr = a.partial + (((size_t)b * a.Kh + kvh) * nparts * G + g) * (H + 2);
  const size_t sstride = (size_t)G * (H + 2);
  // the parts are requested eight at a time (clamped indices), so that a row costs one memory round trip and not
  // one per part; merged in ascending order
  float mm = -1e30f, ls = 0.f, o = 0.f;
  for (int s0 = 0; s0 < nparts; s0 += 8) {
    float pm[8], pl[8], po[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const float* q = pr + (size_t)min(s0 + u, nparts - 1) * sstride;
      pm[u] = s0 + u < nparts ? q[H] : -1e30f;
      pl[u] = q[H + 1];
      po[u] = q[d];
    }
    float mn = mm;
#pragma unroll
    for (int u = 0; u < 8; ++u) mn = fmaxf(mn, pm[u]);
    const float alpha = __expf(mm - mn);
    ls *= alpha;
    o *= alpha;
    mm = mn;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (s0 + u < nparts) {
        const float w = __expf(pm[u] - mm);
        ls += pl[u] * w;
        o += po[u] * w;
      }
    }
  }
  a.out[((size_t)b * a.N + kvh * G + g) * H + d] = f2bf(ls > 0.f ? o / ls : 0.f);
}

// ---------------------------------------------------------------------------
// The one-token walk on the matrix pipe (gqa_tile_kernel).  The queries of a workgroup are the 32 columns of an
// MFMA tile: scores^T [position, query] = K . Q^T and out^T [hidden, query] += V^T . P^T as in the many-tokens
// kernel below, with the four waves of a workgroup taking different blocks of 32 positions and meeting through
// LDS at the end.  K rows go from global memory straight into the A operand (lane (position, h) owns one half
// of its row), the V tile of a wave goes global -> LDS by direct loads and is read transposed
// (ds_read_b64_tr_b16: 16 reads per 32 positions where 16-bit gathers took 64 reads and 32 merges), the query
// fragments wait in LDS.  Per 32 positions a wave issues 8 + 32 MFMAs and about 120 VALU instructions, against
// 527 VALU instructions per 16 positions of gqa_decode_walk at 4 query heads (about 1400 at 8), whose dot
// products and reductions run on the vector ALU; it takes the launch wherever its workgroups (three per CU:
// LDS and registers) are all resident at once.
//
// Two kinds of query block share the launch:
//  * a row: the G query heads of one sequence (the first G columns of the tile) over that sequence's own slots;
//  * a group: prompt slots shared by a group of sequences.  A GRPO rollout decodes the samples of every prompt
//    as consecutive rows (tunix/rl/rl_learner.py:432-435 repeats each prompt num_generations times), so the
//    K / V rows of the prompt slots are the same in the share_gs caches of a group, and so are their input_mask
//    entries.  Those slots are walked once per (group, kv head), from the group's first sequence, for the
//    32 / G sequences x G query heads of a query block; every row keeps its own slots share_len .. *step.
// A query block with one split writes its output directly; otherwise every walk writes an (out, max, sum) part
// and gqa_combine_kernel merges the parts of a row: the same softmax over the same positions either way (f32
// throughout, probabilities enter the V product as bf16 hi + lo); only the order of the f32 sums differs.

template <int H>
struct PrefixLds {
  // the V tiles [4 waves][32 positions][H] bf16 are reused after the walk for the waves' accumulators
  // [2][H / 32][16][64] f32 (two of the four waves at a time)
  static constexpr int kTileBytes = 4 * 32 * H * 2;
  static constexpr int kMergeBytes = 2 * (H / 32) * 16 * 64 * 4;
  __attribute__((aligned(16))) unsigned char tiles[kTileBytes > kMergeBytes ? kTileBytes : kMergeBytes];
  __attribute__((aligned(16))) uint16_t q[32 * H];  // query fragments [H / 8 chunks][32 queries][8]
  float m[2][32], l[2][32];
};

// What one workgroup of the tile walk does.
struct TileJob {
  int kv_row;      // sequence whose cache rows and mask entries are read
  int row0, nrows; // query rows row0 .. row0 + nrows - 1 (nrows <= 32 / G), all heads of the kv head
  int pbeg, pend;  // positions [pbeg, pend)
  int split, nsp;  // this workgroup takes split `split` of nsp splits of the blocks of 32 positions
  int part;        // index of the part it writes when a row has several (nparts > 1)
  int nparts;
};

template <int H, int G>
__device__ __forceinline__ void gqa_tile_walk(const AttnArgs& a, PrefixLds<H>& lds, const int kvh, const TileJob j) {
  constexpr int KS = H / 16;        // MFMA k-steps of the score product
  constexpr int CPR = H / 8;        // 16-byte chunks per cache row
  constexpr int RPD = 64 / CPR;     // rows per 1 KiB direct-to-LDS load
  constexpr int NLD = 32 / RPD;     // loads per wave and V tile
  constexpr int HT = H / 32;        // hidden tiles of the output
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int h = lane >> 5, qi = lane & 31;
  const int lead = j.kv_row;
  const int plen = j.pend - j.pbeg;  // positions are counted from pbeg below
  const int nblk = plen > 0 ? (plen + 31) >> 5 : 0;
  const int bps = (nblk + j.nsp - 1) / j.nsp;
  const int b_end = min((j.split + 1) * bps, nblk);

  // query fragments of the block into LDS: thread (query, chunk) copies 16 bytes; columns past the block's
  // rows repeat its last row (their results are not stored)
  for (int e = threadIdx.x; e < 32 * CPR; e += 256) {
    const int q = e / CPR, c = e % CPR;
    const int lr = min(q / G, j.nrows - 1);
    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(a.q + ((size_t)(j.row0 + lr) * a.N + kvh * G + q % G) * H + c * 8);
    *reinterpret_cast<u32x4_t*>(lds.q + (c * 32 + q) * 8) = v;
  }
  __syncthreads();

  const uint32_t row_bytes = (uint32_t)a.Kh * H * 2;
  const uint32_t span = ((uint32_t)(a.C - 1) * a.Kh + 1) * H * 2;  // rows past the cache read zero
  const __amdgpu_buffer_rsrc_t rk = make_rsrc(a.kcache + ((size_t)lead * a.C * a.Kh + kvh) * H, span);
  const __amdgpu_buffer_rsrc_t rv = make_rsrc(a.vcache + ((size_t)lead * a.C * a.Kh + kvh) * H, span);
  uint16_t* vt = reinterpret_cast<uint16_t*>(lds.tiles) + wave * 32 * H;
  // V tile transfer: load i moves rows i RPD .. i RPD + RPD - 1 of the block, the 16-byte chunks of row r
  // XOR-swizzled by r % CPR.  Row i RPD + lane / CPR has r % CPR = (i RPD) % CPR ^ lane / CPR, so the per-lane
  // part of the swizzle is one word and the rest a constant per load; the offsets are formed at the transfer
  // (kept in registers over the loop they would be spilled)
  const int vrow = (lane / CPR) * row_bytes, vswz = (lane % CPR) ^ (lane / CPR);
  auto dma_v = [&](int blk) __attribute__((always_inline)) {
    int sw = vswz;
    asm volatile("" : "+v"(sw));
#pragma unroll
    for (int i = 0; i < NLD; ++i)
      load_row_to_lds(rv, vt + i * RPD * H, vrow + ((sw ^ ((i * RPD) % CPR)) << 4), (j.pbeg + blk * 32 + i * RPD) * row_bytes);
  };
  // K fragments of a block: lane (position qi, h) reads the half h of its row, 16 bytes per MFMA step
  const int koff = qi * row_bytes + h * H;
  u32x4_t kf[KS];
  auto load_k = [&](int blk) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < KS; ++t)
      kf[t] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rk, koff + t * 16, (j.pbeg + blk * 32) * row_bytes, 0));
  };
  const uint8_t* mrow = a.input_mask + (size_t)lead * a.buf_len;
  auto mask_byte = [&](int blk) __attribute__((always_inline)) {
    const int p = j.pbeg + blk * 32 + qi;
    return (h == 0 && p < a.buf_len) ? mrow[p] : (uint8_t)0;
  };

  f32x16_t o[HT];
#pragma unroll
  for (int c = 0; c < HT; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[c][r] = 0.f;
  float m = -1e30f, l = 0.f;

  int blk = j.split * bps + wave;
  uint8_t mb = 0;
  if (blk < b_end) {
    mb = mask_byte(blk);
    load_k(blk);
    dma_v(blk);
  }
  for (; blk < b_end; blk += 4) {
    const bool more = blk + 4 < b_end;
    const uint32_t mbits = (uint32_t)__ballot(mb != 0);
    // scores^T: rows = positions of the block, column = this lane's query
    f32x16_t sacc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
#pragma unroll
    for (int t = 0; t < KS; ++t) {
      const bf16x8_t qf = *reinterpret_cast<const bf16x8_t*>(lds.q + ((KS * h + t) * 32 + qi) * 8);
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kf[t]), qf, sacc, 0, 0, 0);
    }
    float sc[16];
    float mn = m;
    // accumulator register r holds position 8 (r / 4) + 4 h + r % 4 of the block: with the lane's half folded
    // into the mask word and the limit, the per-register part is a compile-time constant
    const uint32_t mb2 = mbits >> (4 * h);
    const int lim = plen - blk * 32 - 4 * h;  // plen: positions of this walk, counted from pbeg
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int pc = (r >> 2) * 8 + (r & 3);
      const bool ok = pc < lim && ((mb2 >> pc) & 1u);
      sc[r] = ok ? sacc[r] * a.scale : -1e30f;
      mn = fmaxf(mn, sc[r]);
    }
    mn = fmaxf(mn, __shfl_xor(mn, 32, 64));
    const float alpha = __expf(m - mn);
    m = mn;
    float psum = 0.f;
    uint32_t pk[8], pl2[8];
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const float p0 = sc[r] > -1e29f ? __expf(sc[r] - mn) : 0.f;
      const float p1 = sc[r + 1] > -1e29f ? __expf(sc[r + 1] - mn) : 0.f;
      pk[r >> 1] = pack_bf2(p0, p1);
      pl2[r >> 1] = pack_bf2(p0 - bf_lo(pk[r >> 1]), p1 - bf_hi(pk[r >> 1]));
      psum += p0 + p1;
    }
    l = l * alpha + psum;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int c = 0; c < HT; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[c][r] *= alpha;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this block's V tile has landed
    // out^T += V^T . P^T, 16 positions (accumulator registers 8 kb .. 8 kb + 7) per MFMA.  The V^T fragment of
    // lane (hidden 32 c + qi, h) is positions acc_row(8 kb + j, lane) = 16 kb + 8 (j / 4) + 4 h + j % 4, j = 0..7:
    // two runs of four consecutive rows of one column of the tile, which the transposing LDS read delivers
    // directly (ds_read_b64_tr_b16: in every 16 lanes, lane 4 k + q supplies the address of four consecutive
    // 16-bit elements M[4 k + q][0..3] and lane 4 q' + c' receives M[4 k + q'][c'], k = 0..3).  So lane
    // (k4, q4) of a group points at row run + 4 h + k4, columns 32 c + 16 (group % 2) + 4 q4 .. + 3, and a read
    // returns the four rows of the lane's own column.  Chunk (column / 8) of row r sits at chunk ^ r % CPR; the
    // lane's share of that XOR is one word (lsw), the rest a constant per read.
    {
      const int k4 = (lane & 15) >> 2, q4 = lane & 3, g2 = (lane >> 4) & 1;
      int lsw = (2 * g2 + (q4 >> 1)) ^ (4 * h + k4), lbase = (4 * h + k4) * H + 4 * (q4 & 1);
      asm volatile("" : "+v"(lsw), "+v"(lbase));
      typedef short s16x4_t __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int kb2 = 0; kb2 < 2; ++kb2) {
        const u32x4_t pf = {pk[4 * kb2], pk[4 * kb2 + 1], pk[4 * kb2 + 2], pk[4 * kb2 + 3]};
        const u32x4_t pg = {pl2[4 * kb2], pl2[4 * kb2 + 1], pl2[4 * kb2 + 2], pl2[4 * kb2 + 3]};
#pragma unroll
        for (int c = 0; c < HT; ++c) {
          s16x4_t run[2];
#pragma unroll
          for (int a2 = 0; a2 < 2; ++a2) {
            const int row0 = 16 * kb2 + 8 * a2;  // the run without the lane's 4 h + k4
            const uint16_t* src = vt + lbase + row0 * H + ((lsw ^ (4 * c) ^ (row0 % CPR)) << 3);
            run[a2] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) s16x4_t*)(src));
          }
          uint32_t vw[4];
          __builtin_memcpy(&vw[0], &run[0], 8);
          __builtin_memcpy(&vw[2], &run[1], 8);
          const u32x4_t vf = {vw[0], vw[1], vw[2], vw[3]};
          o[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vf),
                                                         __builtin_bit_cast(bf16x8_t, pf), o[c], 0, 0, 0);
          o[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vf),
                                                         __builtin_bit_cast(bf16x8_t, pg), o[c], 0, 0, 0);
        }
      }
    }
    // the tile's reads are complete before the next transfer overwrites it.  The next block's K rows are
    // requested only now (not under the softmax): 32 more live registers would not fit three workgroups per CU,
    // and the other eleven waves of the CU cover the round trip.
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (more) {
      mb = mask_byte(blk + 4);
      load_k(blk + 4);
      dma_v(blk + 4);
    }
  }
  l += __shfl_xor(l, 32, 64);

  // merge the four waves in two rounds through LDS: waves 2, 3 hand their state to waves 0, 1, then wave 1 to
  // wave 0.  The accumulator layout is the same in every wave, so the merge is per lane.
  float* mb_f = reinterpret_cast<float*>(lds.tiles);
  auto put = [&](int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int c = 0; c < HT; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) mb_f[(((slot * HT + c) * 16 + r) << 6) + lane] = o[c][r];
    if (h == 0) {
      lds.m[slot][qi] = m;
      lds.l[slot][qi] = l;
    }
  };
  auto take = [&](int slot) __attribute__((always_inline)) {
    const float m2 = lds.m[slot][qi], l2 = lds.l[slot][qi];
    const float mm = fmaxf(m, m2);
    const float w1 = __expf(m - mm), w2 = __expf(m2 - mm);
#pragma unroll
    for (int c = 0; c < HT; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[c][r] = o[c][r] * w1 + mb_f[(((slot * HT + c) * 16 + r) << 6) + lane] * w2;
    l = l * w1 + l2 * w2;
    m = mm;
  };
  __syncthreads();  // every wave is done with its V tile
  if (wave >= 2) put(wave - 2);
  __syncthreads();
  if (wave < 2) take(wave);
  __syncthreads();
  if (wave == 1) put(0);
  __syncthreads();
  if (wave != 0) return;
  take(0);
  // wave 0 holds out^T [hidden, query] for the block's queries
  const int lr = qi / G, g = qi % G;
  if (lr >= j.nrows) return;
  const int row = j.row0 + lr;
  if (j.nparts == 1) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    uint16_t* dst = a.out + ((size_t)row * a.N + kvh * G + g) * H;
#pragma unroll
    for (int c = 0; c < HT; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint2 w;
        w.x = pack_bf2(o[c][4 * i] * inv, o[c][4 * i + 1] * inv);
        w.y = pack_bf2(o[c][4 * i + 2] * inv, o[c][4 * i + 3] * inv);
        *reinterpret_cast<uint2*>(dst + 32 * c + 8 * i + 4 * h) = w;
      }
    return;
  }
  float* pr = a.partial + ((((size_t)row * a.Kh + kvh) * j.nparts + j.part) * G + g) * (H + 2);
#pragma unroll
  for (int c = 0; c < HT; ++c)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // accumulator registers 4 i .. 4 i + 3 of tile c: hidden values 32 c + 8 i + 4 h .. + 3 (a part is H + 2
      // floats: 8-byte aligned pieces)
      float* d = pr + 32 * c + 8 * i + 4 * h;
      *reinterpret_cast<f32x2_t*>(d) = f32x2_t{o[c][4 * i], o[c][4 * i + 1]};
      *reinterpret_cast<f32x2_t*>(d + 2) = f32x2_t{o[c][4 * i + 2], o[c][4 * i + 3]};
    }
  if (h == 0) {
    pr[H] = m;
    pr[H + 1] = l;
  }
}

// The job of workgroup (y, z) of a launch whose first n_group_y y-indices are (group, query block) pairs of the
// shared slots and whose other y-indices are rows; false: nothing to do.
template <int G>
__device__ __forceinline__ bool tile_job(const AttnArgs& a, int n_group_y, int y, int z, bool rows_too, TileJob& j) {
  constexpr int RPB = 32 / G;  // sequences per query block
  // newest valid slot; clamped into the cache and the mask row so that a caller that oversteps reads in bounds
  const int step = min(*a.step, min(a.C, a.buf_len) - 1);
  const int shared_end = a.share_gs > 1 ? min(a.share_len, step + 1) : 0;
  j.nparts = a.nsplit + a.psplits;
  j.split = z;
  if (y < n_group_y) {
    if (z >= a.psplits) return false;
    const int qblocks = (a.share_gs + RPB - 1) / RPB;
    const int grp = y / qblocks, qb = y - grp * qblocks;
    j.kv_row = grp * a.share_gs;
    j.row0 = j.kv_row + qb * RPB;
    j.nrows = min(RPB, a.share_gs - qb * RPB);
    j.pbeg = 0; j.pend = shared_end;
    j.nsp = a.psplits;
    j.part = a.nsplit + z;
    return true;
  }
  if (!rows_too || z >= a.nsplit) return false;
  j.kv_row = j.row0 = y - n_group_y;
  j.nrows = 1;
  j.pbeg = shared_end; j.pend = step + 1;
  j.nsp = a.nsplit;
  j.part = z;
  return true;
}

// grid (Kh, group query blocks + rows, splits): every workgroup runs the tile walk (the groups' workgroups first
// in dispatch order).  Three workgroups per CU (LDS and registers).
template <int H, int G>
__global__ __launch_bounds__(256, 3) void gqa_tile_kernel(AttnArgs a, int n_group_y) {
  __shared__ PrefixLds<H> lds;
  TileJob j;
  if (tile_job<G>(a, n_group_y, blockIdx.y, blockIdx.z, true, j)) gqa_tile_walk<H, G>(a, lds, blockIdx.x, j);
}

// The same grid with the rows' own slots on the vector-ALU walk (gqa_decode_walk) and only the shared slots on
// the tile walk: up to four query heads per kv head the vector walk streams cold cache rows faster (whole rows
// in coalesced non-temporal loads; the tile walk fetches K in 16-byte pieces per lane): measured on the 8B
// rollout shape, 64 sequences at context 512, per decode step: 3.997 ms this way, 4.098 ms all on the tile
// walk, 4.176 ms without sharing.
template <int H, int G>
__global__ __launch_bounds__(256, 3) void gqa_shared_kernel(AttnArgs a, int n_group_y) {
  union Lds {
    DecodeLds<H, G> d;
    PrefixLds<H> p;
  };
  __shared__ Lds lds;
  if ((int)blockIdx.y < n_group_y) {
    TileJob j;
    if (tile_job<G>(a, n_group_y, blockIdx.y, blockIdx.z, false, j)) gqa_tile_walk<H, G>(a, lds.p, blockIdx.x, j);
    return;
  }
  if ((int)blockIdx.z < a.nsplit) gqa_decode_walk<H, G>(a, lds.d, blockIdx.x, (int)blockIdx.y - n_group_y, blockIdx.z);
}

// ---------------------------------------------------------------------------
// Many tokens per sequence (cache fill and scoring passes): a workgroup owns one (sequence, kv
// head) and a block of consecutive query tokens, and walks the cache once for all of them, 32
// positions at a time, on the matrix pipe.  Wave w holds 32 query rows (32 / G tokens x G heads)
// as the B operand; the K tile [32 positions, H] and the V tile go global -> LDS by direct loads
// (16-byte chunks XOR-swizzled by row) and are shared by the four waves.
//   scores^T [position, query] = K . Q^T : lane (query, h) keeps 16 positions of ONE query in its
//     accumulator, so mask, max, exp and sum run down the registers (one shuffle joins the halves);
//   out^T [hidden, query] += V^T . P^T  : the B operand is the lane's own 8 probabilities of a
//     16-position block (positions are consumed in accumulator order, which V^T follows: its
//     fragment comes from the V tile by transposing LDS reads), and the rescale by
//     exp(old max - new max) is per lane.
// Probabilities enter the product as two bf16 terms (hi + lo), i.e. with 16 mantissa bits.
constexpr int kFillMinTokens = 4;  // tokens per sequence and pass from which the fill kernel is used

template <int H, int G>
__global__ __launch_bounds__(256) void gqa_fill_kernel(AttnArgs a) {
  constexpr int KS = H / 16;        // MFMA k-steps of the score product
  constexpr int CPR = H / 8;        // 16-byte chunks per cache row
  constexpr int RPD = 64 / CPR;     // rows per 1 KiB direct-to-LDS load
  constexpr int NLD = 32 / RPD / 4; // loads per wave and tile
  constexpr int HT = H / 32;        // hidden tiles of the output
  constexpr int TPW = 32 / G, TQ = 4 * TPW;  // tokens per wave / workgroup
  __shared__ __align__(16) uint16_t kt[2][32 * H], vt[2][32 * H];
  const int kvh = blockIdx.x, seq = blockIdx.y, tblk = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int h = lane >> 5, qi = lane & 31;
  const int T = a.tpp, step0 = max(min(*a.step, min(a.C, a.buf_len) - T), 0);  // clamped: every slot read lies in the cache
  const int tok = tblk * TQ + wave * TPW + qi / G, g = qi % G;
  const int tok_l = tok < T ? tok : T - 1;
  const int limit = step0 + tok_l;  // newest slot this query sees
  const int last_tok = tblk * TQ + TQ - 1 < T - 1 ? tblk * TQ + TQ - 1 : T - 1;
  const int nblk = (step0 + last_tok + 32) >> 5;  // blocks of 32 positions up to the newest slot of the block

  const size_t qoff = ((size_t)(seq * T + tok_l) * a.N + kvh * G + g) * H;
  u32x4_t qf[KS];
#pragma unroll
  for (int t = 0; t < KS; ++t) qf[t] = *reinterpret_cast<const u32x4_t*>(a.q + qoff + (H / 2) * h + 8 * t);

  const uint32_t row_bytes = (uint32_t)a.Kh * H * 2;
  const uint32_t span = ((uint32_t)(a.C - 1) * a.Kh + 1) * H * 2;  // rows past the cache read zero
  const __amdgpu_buffer_rsrc_t rk = make_rsrc(a.kcache + ((size_t)seq * a.C * a.Kh + kvh) * H, span);
  const __amdgpu_buffer_rsrc_t rv = make_rsrc(a.vcache + ((size_t)seq * a.C * a.Kh + kvh) * H, span);
  int toff[NLD];  // tile transfer: load i of this wave moves rows (wave + 4 i) RPD .. + RPD - 1
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int row_l = (wave + 4 * i) * RPD + lane / CPR;
    toff[i] = row_l * row_bytes + (((lane % CPR) ^ (row_l % CPR)) * 16);
  }
  auto dma_tile = [&](int blk, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      load_row_to_lds(rk, &kt[buf][(wave + 4 * i) * RPD * H], toff[i], blk * 32 * row_bytes);
      load_row_to_lds(rv, &vt[buf][(wave + 4 * i) * RPD * H], toff[i], blk * 32 * row_bytes);
    }
  };
  // input mask of a block: lane p of the lower half fetches the byte of position 32 blk + p early,
  // the ballot that turns the bytes into a bit per position runs when the block is needed
  const uint8_t* mrow = a.input_mask + (size_t)seq * a.buf_len;
  auto mask_byte = [&](int blk) __attribute__((always_inline)) {
    const int p = blk * 32 + qi;
    return (h == 0 && p < a.buf_len) ? mrow[p] : (uint8_t)0;
  };
  f32x16_t o[HT];
#pragma unroll
  for (int c = 0; c < HT; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[c][r] = 0.f;
  float m = -1e30f, l = 0.f;

  uint8_t mb = mask_byte(0);
  dma_tile(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  for (int blk = 0; blk < nblk; ++blk) {
    const int buf = blk & 1;
    const uint32_t mbits = (uint32_t)__ballot(mb != 0);
    mb = mask_byte(blk + 1);  // requested before the tile so that the tile's loads stay the youngest
    if (blk + 1 < nblk) dma_tile(blk + 1, buf ^ 1);
    // scores^T: rows = positions of the block, column = this lane's query
    f32x16_t sacc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
    const uint16_t* kb = &kt[buf][qi * H];
#pragma unroll
    for (int t = 0; t < KS; ++t) {
      const int slot = ((KS * h + t) ^ (qi % CPR)) * 8;  // lane (position, h) multiplies k = (H / 2) h + 8 t ..
      const bf16x8_t kf = *reinterpret_cast<const bf16x8_t*>(kb + slot);
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, __builtin_bit_cast(bf16x8_t, qf[t]), sacc, 0, 0, 0);
    }
    float sc[16];
    float mn = m;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int pl = acc_row(r, lane), p = blk * 32 + pl;
      const bool ok = p <= limit && ((mbits >> pl) & 1u);
      sc[r] = ok ? sacc[r] * a.scale : -1e30f;
      mn = fmaxf(mn, sc[r]);
    }
    mn = fmaxf(mn, __shfl_xor(mn, 32, 64));
    const float alpha = __expf(m - mn);
    m = mn;
    // probabilities as bf16 pairs hi + lo (16 mantissa bits between them), so that the product
    // keeps the precision of the one-token kernel's f32 probabilities and a scoring pass
    // reproduces the log-probs of the rollout that generated the tokens
    float ps = 0.f;
    uint32_t pk[8], pl2[8];
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const float p0 = sc[r] > -1e29f ? __expf(sc[r] - mn) : 0.f;
      const float p1 = sc[r + 1] > -1e29f ? __expf(sc[r + 1] - mn) : 0.f;
      pk[r >> 1] = pack_bf2(p0, p1);
      pl2[r >> 1] = pack_bf2(p0 - bf_lo(pk[r >> 1]), p1 - bf_hi(pk[r >> 1]));
      ps += p0 + p1;
    }
    l = l * alpha + ps;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int c = 0; c < HT; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[c][r] *= alpha;
    }
    // out^T += V^T . P^T, 16 positions (accumulator registers 8 kb .. 8 kb + 7) per MFMA
#pragma unroll
    for (int kb2 = 0; kb2 < 2; ++kb2) {
      const u32x4_t pf = {pk[4 * kb2], pk[4 * kb2 + 1], pk[4 * kb2 + 2], pk[4 * kb2 + 3]};
      const u32x4_t pg = {pl2[4 * kb2], pl2[4 * kb2 + 1], pl2[4 * kb2 + 2], pl2[4 * kb2 + 3]};
#pragma unroll
      for (int c = 0; c < HT; ++c) {
        // V^T fragment: two runs of four consecutive rows of the lane's column, by the transposing LDS read
        // (see gqa_tile_walk): lane (k4, q4) of a group of 16 points at row run + 4 h + k4, columns
        // 32 c + 16 (group % 2) + 4 q4 .. + 3
        typedef short s16x4_t __attribute__((ext_vector_type(4)));
        const int k4 = (lane & 15) >> 2, q4 = lane & 3, g2 = (lane >> 4) & 1;
        s16x4_t run[2];
#pragma unroll
        for (int a2 = 0; a2 < 2; ++a2) {
          const int row = 16 * kb2 + 8 * a2 + 4 * h + k4;
          const int chunk = 4 * c + 2 * g2 + (q4 >> 1);
          run[a2] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(
              &vt[buf][row * H + ((chunk ^ (row % CPR)) * 8) + 4 * (q4 & 1)]));
        }
        uint32_t vw[4];
        __builtin_memcpy(&vw[0], &run[0], 8);
        __builtin_memcpy(&vw[2], &run[1], 8);
        const u32x4_t vf = {vw[0], vw[1], vw[2], vw[3]};
        o[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vf),
                                                       __builtin_bit_cast(bf16x8_t, pf), o[c], 0, 0, 0);
        o[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vf),
                                                       __builtin_bit_cast(bf16x8_t, pg), o[c], 0, 0, 0);
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // the next tile has landed
    __syncthreads();
  }
  l += __shfl_xor(l, 32, 64);
  if (tok >= T) return;
  const float inv = l > 0.f ? 1.f / l : 0.f;
  uint16_t* dst = a.out + qoff;
#pragma unroll
  for (int c = 0; c < HT; ++c)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint2 w;
      w.x = pack_bf2(o[c][4 * i] * inv, o[c][4 * i + 1] * inv);
      w.y = pack_bf2(o[c][4 * i + 2] * inv, o[c][4 * i + 3] * inv);
      *reinterpret_cast<uint2*>(dst + 32 * c + 8 * i + 4 * h) = w;
    }
}

template <int H, int G>
static int launch_fill(hipStream_t st, const AttnArgs& a) {
  const int nseq = a.B / a.tpp, tq = 4 * (32 / G);
  hipLaunchKernelGGL((gqa_fill_kernel<H, G>), dim3(a.Kh, nseq, (a.tpp + tq - 1) / tq), dim3(256), 0, st, a);
  return check_launch();
}

template <int H, int G>
static int launch_attn(hipStream_t st, const AttnArgs& a) {
  hipLaunchKernelGGL((gqa_decode_kernel<H, G>), dim3(a.Kh, a.B, a.nsplit), dim3(AttnWaves<G>::value * 64), 0, st, a);
  int rc = check_launch();
  if (rc != TMX_OK || a.nsplit == 1) return rc;
  hipLaunchKernelGGL((gqa_combine_kernel<H, G>), dim3(a.Kh, a.B, G), dim3(H), 0, st, a);
  return check_launch();
}

// Number of sequence splits of the vector-ALU walk that brings the grid to roughly two workgroups per CU
// (more splits cost more in partial sums and the combine launch than they gain at rollout batch sizes).
// Mid-sized grids (65 to 256 (sequence, kv head) pairs, the 30B-A3B shape at 32 sequences) run
// fastest at four workgroups per CU with chunks down to 128 positions (measured).
int attn_num_splits(int B, int Kh, int C) {
  const int pairs = B * Kh;
  const bool mid = pairs > 64 && pairs <= 256;
  int ns = (mid ? 1024 : 512) / pairs;
  if (ns < 1) ns = 1;
  const int per = mid ? 128 : 256;
  const int max_by_len = (C + per - 1) / per;
  if (ns > max_by_len) ns = max_by_len;
  if (ns > 32) ns = 32;
  return ns;
}

// The shared walk serves one token per sequence, up to 128 sequences in whole groups, the head dimensions and
// group widths of the tile walk, and 32-bit byte offsets per cache.
bool attn_share_ok(int B, int N, int Kh, int H, int C, int share_gs, int share_len) {
  if (share_gs <= 1 || share_len < 32 || share_len > C || B <= 0 || B > 128 || B % share_gs) return false;
  if (Kh <= 0 || N % Kh || (H != 64 && H != 128)) return false;
  const int G = N / Kh;
  if (G != 1 && G != 2 && G != 4 && G != 8) return false;
  return (size_t)C * Kh * H * 2 < (1u << 31);
}

// Which kernel walks the cache of a one-token step, and in how many splits.
struct AttnPlan {
  bool tile;    // gqa_tile_kernel (matrix pipe) or gqa_decode_kernel (vector ALU)
  bool shared;  // tile only: prompt slots once per group
  int nsplit;   // splits of a row's own slots
  int psplits;  // splits of the shared slots
};

static AttnPlan plan_attention(int B, int N, int Kh, int H, int C, int share_gs, int share_len) {
  AttnPlan p = {false, false, attn_num_splits(B, Kh, C), 0};
  const int G = Kh > 0 && N % Kh == 0 ? N / Kh : 0;
  if ((H != 64 && H != 128) || (G != 1 && G != 2 && G != 4 && G != 8) || (size_t)C * Kh * H * 2 >= (1u << 31)) return p;
  // Launches with tile-walk workgroups hold three per CU and want them all resident at once (measured at 128
  // sequences x 8 kv heads = 1024 workgroups: 108 against 98 us for the vector-ALU walk, four of whose workgroups
  // fit a CU); with shared prompt slots a launch reads fewer cache rows and may take two rounds.
  const long slots = 3L * device_cus(), pairs = (long)B * Kh;
  p.shared = attn_share_ok(B, N, Kh, H, C, share_gs, share_len);
  // Rows' own slots: the tile walk for 8 query heads per kv head (measured on the 30B-A3B shape, 32 sequences at
  // context 512: 10.7 + 3.0 us for walk and combine against 21.7 + 3.9 us; the vector walk's work per cache row
  // grows with the heads); up to 2 heads, and 4 heads behind shared slots, the vector walk (see gqa_shared_kernel).
  p.tile = G == 8 && pairs <= (p.shared ? 2 * slots : slots);
  // 4 heads per kv head without shared slots: the tile walk as well, since its V^T fragments come from the
  // transposing LDS read (measured on the 8B shape, 64 sequences, whole rollout: 4.158 -> 4.109 ms per step; with
  // shared slots the rows stay on the vector walk: 3.941 against 3.953)
  if (G == 4 && !p.shared && pairs <= slots) p.tile = true;
  if (G == 8 && !p.tile) p.shared = false;
  if (p.shared && pairs > 2 * slots) p.shared = false;
  long group_wgs = 0;
  if (p.shared) {
    const int rpb = 32 / G, qblocks = (share_gs + rpb - 1) / rpb;
    group_wgs = (long)(B / share_gs) * qblocks * Kh;
    // splits of the shared slots: a block of 32 positions for every other wave, while the launch stays resident
    // (measured on 256 shared slots at 64 sequences of the 8B shape: 1, 2, 4 splits -> 23.9, 22.1, 21.2 us)
    const int nblk = (share_len + 31) / 32;
    p.psplits = nblk / 2 < 1 ? 1 : (nblk / 2 > kMaxPrefixSplits ? kMaxPrefixSplits : nblk / 2);
    while (p.psplits > 1 && pairs + group_wgs * p.psplits > slots) --p.psplits;
  }
  if (p.tile) {
    // fill the slots that are left, at least 8 blocks of 32 positions per split
    long ns = (slots - group_wgs * p.psplits) / pairs;
    const int by_len = (C + 255) / 256;
    if (ns > by_len) ns = by_len;
    if (ns > 8) ns = 8;
    p.nsplit = ns < 1 ? 1 : (int)ns;
  } else if (p.shared) {
    p.nsplit = 1;  // the vector walk behind shared slots: one split per row (more did not pay, see above)
  }
  return p;
}

size_t attn_partial_bytes(int B, int N, int Kh, int H, int C) {
  const AttnPlan p = plan_attention(B, N, Kh, H, C, 0, 0);
  // rows of two or three tokens per pass take the vector-ALU walk whatever the plan says
  const int ns = p.nsplit > attn_num_splits(B, Kh, C) ? p.nsplit : attn_num_splits(B, Kh, C);
  return ns == 1 ? 0 : (size_t)B * N * ns * (H + 2) * sizeof(float);
}

// room for every plan of this shape, shared slots included
size_t attn_shared_partial_bytes(int B, int N, int Kh, int H, int C) {
  const int nv = attn_num_splits(B, Kh, C);
  const int ns = nv > 8 ? nv : 8;
  return (size_t)B * N * (ns + kMaxPrefixSplits) * (H + 2) * sizeof(float);
}

template <int H, int G>
static int launch_tile(hipStream_t st, const AttnArgs& a, bool rows_on_tile) {
  int n_group_y = 0;
  if (a.share_gs > 1) {
    const int rpb = 32 / G, qblocks = (a.share_gs + rpb - 1) / rpb;
    n_group_y = (a.B / a.share_gs) * qblocks;
  }
  const int nz = a.nsplit > a.psplits ? a.nsplit : a.psplits;
  const dim3 grid(a.Kh, n_group_y + a.B, nz);
  if (rows_on_tile) hipLaunchKernelGGL((gqa_tile_kernel<H, G>), grid, dim3(256), 0, st, a, n_group_y);
  else if constexpr (G <= 4) hipLaunchKernelGGL((gqa_shared_kernel<H, G>), grid, dim3(256), 0, st, a, n_group_y);
  else return TMX_ERR_UNSUPPORTED;
  int rc = check_launch();
  if (rc != TMX_OK || a.nsplit + a.psplits == 1) return rc;
  hipLaunchKernelGGL((gqa_combine_kernel<H, G>), dim3(a.Kh, a.B, G), dim3(H), 0, st, a);
  return check_launch();
}

int gqa_decode(hipStream_t st, AttnArgs a, int H) {
  const int G = a.N / a.Kh;
  if (a.N % a.Kh) return TMX_ERR_SHAPE;
  if (a.tpp <= 1) {
    const AttnPlan p = plan_attention(a.B, a.N, a.Kh, H, a.C, a.share_gs, a.share_len);
    if (p.tile || p.shared) {
      a.nsplit = p.nsplit;
      a.psplits = p.shared ? p.psplits : 0;
      if (!p.shared) a.share_gs = a.share_len = 0;
      if (a.nsplit + a.psplits > 1 && !a.partial) return TMX_ERR_ARG;
#define TMX_TILE_CASE(HH, GG) \
  if (H == HH && G == GG) return launch_tile<HH, GG>(st, a, p.tile);
      TMX_TILE_CASE(64, 1)
      TMX_TILE_CASE(64, 2)
      TMX_TILE_CASE(64, 4)
      TMX_TILE_CASE(64, 8)
      TMX_TILE_CASE(128, 1)
      TMX_TILE_CASE(128, 2)
      TMX_TILE_CASE(128, 4)
      TMX_TILE_CASE(128, 8)
#undef TMX_TILE_CASE
    }
  }
  a.nsplit = attn_num_splits(a.B, a.Kh, a.C);
  a.share_gs = a.share_len = a.psplits = 0;
  if (a.nsplit > 1 && !a.partial) return TMX_ERR_ARG;
  // several tokens per sequence: one walk over the cache for a block of them (MFMA kernel)
  if (a.tpp >= kFillMinTokens && a.B % a.tpp == 0 && (size_t)a.C * a.Kh * H * 2 < (1u << 31)) {
#define TMX_FILL_CASE(HH, GG) \
  if (H == HH && G == GG) return launch_fill<HH, GG>(st, a);
    TMX_FILL_CASE(64, 1)
    TMX_FILL_CASE(64, 2)
    TMX_FILL_CASE(64, 4)
    TMX_FILL_CASE(128, 1)
    TMX_FILL_CASE(128, 2)
    TMX_FILL_CASE(128, 4)
    TMX_FILL_CASE(128, 8)
#undef TMX_FILL_CASE
  }
#define TMX_ATTN_CASE(HH, GG) \
  if (H == HH && G == GG) return launch_attn<HH, GG>(st, a);
  TMX_ATTN_CASE(64, 1)
  TMX_ATTN_CASE(64, 2)
  TMX_ATTN_CASE(64, 4)
  TMX_ATTN_CASE(128, 1)
  TMX_ATTN_CASE(128, 2)
  TMX_ATTN_CASE(128, 4)
  TMX_ATTN_CASE(128, 8)
#undef TMX_ATTN_CASE
  return TMX_ERR_UNSUPPORTED;
}

}  // namespace tmx

using namespace tmx;

extern "C" size_t tmx_gqa_decode_workspace_bytes(int B, int N, int Kh, int H, int C) {
  return attn_partial_bytes(B, N, Kh, H, C);
}

extern "C" int tmx_gqa_decode_attention(void* stream, const void* q, const void* kcache,
                                        const void* vcache, const uint8_t* input_mask,
                                        const int32_t* step, int buf_len, void* out, void* workspace,
                                        int B, int N, int Kh, int H, int C) {
  if (!q || !kcache || !vcache || !input_mask || !step || !out) return TMX_ERR_ARG;
  if (B <= 0 || N <= 0 || Kh <= 0 || C <= 0) return TMX_ERR_SHAPE;
  AttnArgs a = {};
  a.q = (const uint16_t*)q;
  a.kcache = (const uint16_t*)kcache;
  a.vcache = (const uint16_t*)vcache;
  a.input_mask = input_mask;
  a.step = step;
  a.buf_len = buf_len;
  a.out = (uint16_t*)out;
  a.partial = (float*)workspace;
  a.B = B; a.N = N; a.Kh = Kh; a.C = C;
  a.scale = 1.0f / sqrtf((float)H);
  return gqa_decode((hipStream_t)stream, a, H);
}

extern "C" size_t tmx_gqa_decode_shared_workspace_bytes(int B, int N, int Kh, int H, int C) {
  return attn_shared_partial_bytes(B, N, Kh, H, C);
}

extern "C" int tmx_gqa_decode_attention_shared(void* stream, const void* q, const void* kcache, const void* vcache,
                                               const uint8_t* input_mask, const int32_t* step, int buf_len,
                                               void* out, void* workspace, int B, int N, int Kh, int H, int C,
                                               int share_group, int share_len) {
  if (!q || !kcache || !vcache || !input_mask || !step || !out || !workspace) return TMX_ERR_ARG;
  if (B <= 0 || N <= 0 || Kh <= 0 || C <= 0) return TMX_ERR_SHAPE;
  if (!plan_attention(B, N, Kh, H, C, share_group, share_len).shared) return TMX_ERR_UNSUPPORTED;
  AttnArgs a = {};
  a.q = (const uint16_t*)q;
  a.kcache = (const uint16_t*)kcache;
  a.vcache = (const uint16_t*)vcache;
  a.input_mask = input_mask;
  a.step = step;
  a.buf_len = buf_len;
  a.out = (uint16_t*)out;
  a.partial = (float*)workspace;
  a.B = B; a.N = N; a.Kh = Kh; a.C = C;
  a.share_gs = share_group; a.share_len = share_len;
  a.scale = 1.0f / sqrtf((float)H);
  return gqa_decode((hipStream_t)stream, a, H);
}

extern "C" int tmx_gqa_attention_rows(void* stream, const void* q, const void* kcache, const void* vcache,
                                      const uint8_t* input_mask, const int32_t* step, int buf_len, void* out,
                                      void* workspace, int n_seq, int T, int N, int Kh, int H, int C) {
  if (!q || !kcache || !vcache || !input_mask || !step || !out) return TMX_ERR_ARG;
  if (n_seq <= 0 || T <= 0 || N <= 0 || Kh <= 0 || C <= 0) return TMX_ERR_SHAPE;
  AttnArgs a = {};
  a.q = (const uint16_t*)q;
  a.kcache = (const uint16_t*)kcache;
  a.vcache = (const uint16_t*)vcache;
  a.input_mask = input_mask;
  a.step = step;
  a.buf_len = buf_len;
  a.out = (uint16_t*)out;
  a.partial = (float*)workspace;
  a.B = n_seq * T; a.N = N; a.Kh = Kh; a.C = C;
  a.tpp = T;
  a.scale = 1.0f / sqrtf((float)H);
  return gqa_decode((hipStream_t)stream, a, H);
}
