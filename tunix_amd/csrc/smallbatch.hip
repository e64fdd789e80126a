// The decode step for one to four sequences (single-sequence latency regime): five launches per
// layer instead of eight.
//
// At this size a projection is a matrix-vector product: the activations of all rows are a few KiB,
// so every workgroup keeps ALL of them in LDS and can afford to redo the cheap row work itself.
// That removes the launches whose only job was a cross-workgroup reduction:
//   * RMSNorm (tunix/models/llama3/model.py:290-297) runs in the prologue of the projection that
//     consumes it (q|k|v and gate|up): every workgroup normalises the residual stream itself;
//   * the LoRA projection t = x . A (qwix LoRA on tunix/models/llama3/model.py:216-218, :461-487)
//     is computed by every workgroup over the full K (A comes from L2), so the delta
//     bf16(bf16(t . B) * alpha / r) and, for o and down, the residual add
//     (llama3/model.py:546-564) happen in the projection's own epilogue; for the down projection
//     t comes from partial products the gate|up workgroups leave behind (each owns 32 hidden units);
//   * SwiGLU (llama3/model.py:489-496) is the epilogue of gate|up (a workgroup owns a gate tile and
//     the matching up tile);
//   * RoPE and the KV-cache write (llama3/model.py:249-270, :367-377) are the prologue of the
//     attention kernel, and the merge of its context splits is the prologue of the o projection.
// Weights stream HBM -> registers in the packed tile format (one coalesced 1 KiB load per tile and
// wave), every tile load of a wave is issued before the first use, dequantisation is the same
// bit-exact bf16((u - 8) * s), and the product runs on v_mfma_f32_32x32x16_bf16 with the rows
// beyond the batch ignored: at one row the VALU dequantisation, not the matrix pipe, is what a
// tile costs.  A workgroup is 8 waves = column tiles x K-slices; the K-slices meet in LDS.
#include "tmx_kernels.h"

namespace tmx {

constexpr int kSbThreads = 512, kSbWaves = 8;
constexpr int kSbMaxRows = 4;
constexpr int kSbMaxTiles = 8;   // k-tiles per wave requested at once

enum { SB_PRO_PLAIN = 0, SB_PRO_NORM = 1, SB_PRO_ATTN = 2 };
enum { SB_EPI_PLAIN = 0, SB_EPI_RESIDUAL = 1, SB_EPI_SWIGLU = 2 };

// LDS carve of sb_linear_kernel (bytes): x [M][K + 8] bf16 | red [8 waves][4][32] f32 |
// red_t [8][4][64] f32 | t [4][64] f32 | act [4][32] f32 | row scratch [4 + 8 * 4] f32
__host__ __device__ inline size_t sb_x_bytes(int M, int K) { return ((size_t)M * (K + 8) * 2 + 15) & ~(size_t)15; }
constexpr size_t kSbTailFloats = kSbWaves * kSbMaxRows * 32 + kSbWaves * kSbMaxRows * 64 + kSbMaxRows * 64 +
                                 kSbMaxRows * 32 + 4 + kSbWaves * 4;

template <int PRO, int EPI>
__global__ __launch_bounds__(kSbThreads) void sb_linear_kernel(SbLinearArgs a) {
  extern __shared__ __align__(16) unsigned char sb_smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, nl = lane & 31;
  const int M = a.M, K = a.K, KT = K >> 6, XS = K + 8;
  constexpr int CT = EPI == SB_EPI_SWIGLU ? 2 : 1;  // column tiles per workgroup
  constexpr int KS = kSbWaves / CT;                  // K-slices
  const int c = wave % CT, s = wave / CT;
  uint16_t* xs = reinterpret_cast<uint16_t*>(sb_smem);
  float* red = reinterpret_cast<float*>(sb_smem + sb_x_bytes(M, K));
  float* red_t = red + kSbWaves * kSbMaxRows * 32;
  float* t_s = red_t + kSbWaves * kSbMaxRows * 64;
  float* act_s = t_s + kSbMaxRows * 64;
  float* rms_s = act_s + kSbMaxRows * 32;  // [4] + per-wave sums [8][4]

  // column tile of this wave; its first weight tiles and scales are requested before anything else
  const int nb = EPI == SB_EPI_SWIGLU ? (int)blockIdx.x + c * a.pair_off : (int)blockIdx.x;
  const int per = (KT + KS - 1) / KS;  // k-tiles per slice
  const int kt0 = s * per, kt1 = min(kt0 + per, KT);
  const int gs = __builtin_ctz(a.G >> 6), KG = K / a.G;
  const u32x4_t* wsrc = reinterpret_cast<const u32x4_t*>(a.qw) + (size_t)nb * KT * 64 + lane;
  const uint16_t* ssrc = a.scales + (size_t)nb * KG * 32 + nl;
  u32x4_t wr[kSbMaxTiles];
  uint16_t sr[kSbMaxTiles];
#pragma unroll
  for (int i = 0; i < kSbMaxTiles; ++i) {
    if (i < per) {
      const int kt = min(kt0 + i, KT - 1);
      wr[i] = __builtin_nontemporal_load(wsrc + (size_t)kt * 64);  // every tile is read once, by this wave
      sr[i] = ssrc[(size_t)(kt >> gs) * 32];
    }
  }
  // Everything the epilogue needs that depends on no other launch is requested now as well, so that its
  // latency hides behind the weight stream: the B values of this thread's column(s) (rows 0..15 of B; a
  // larger rank reads the rest in the epilogue), the residual, and the rows of the next projection's A.
  const bool epi_thread = tid < kSbMaxRows * 32 && (tid >> 5) < M;
  const int em = tid >> 5, ej = tid & 31;
  uint16_t breg[CT][16];
  uint16_t res_v = 0;
  uint4 anx[EPI == SB_EPI_SWIGLU ? 4 : 1];  // A_next[32 blockIdx.x + 8 u .. + 7][ej], u = 0..3
  if (epi_thread) {
    if (a.lora_b) {
#pragma unroll
      for (int q = 0; q < CT; ++q) {
        const int n = ((int)blockIdx.x + q * (EPI == SB_EPI_SWIGLU ? a.pair_off : 0)) * 32 + ej;
#pragma unroll
        for (int rr = 0; rr < 16; ++rr) breg[q][rr] = a.lora_b[(size_t)min(rr, a.lora_r - 1) * a.N + n];
      }
    }
    if constexpr (EPI == SB_EPI_RESIDUAL) res_v = a.residual[(size_t)em * a.ldy + blockIdx.x * 32 + ej];
    if constexpr (EPI == SB_EPI_SWIGLU) {
      if (a.a_next) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          // rows k .. k + 7 of column ej are 8 consecutive values in fragment order (r_pad 32):
          // ((kb * 4 + t) * 64 + 32 h + ej) * 8 with k = 64 kb + 16 t + 8 h
          const int k = blockIdx.x * 32 + u * 8;
          const int kb = k >> 6, rem = k & 63, t = rem >> 4, hh = (rem >> 3) & 1;
          anx[u] = *reinterpret_cast<const uint4*>(a.a_next + ((((size_t)kb * 4 + t) * 64) + 32 * hh + ej) * 8);
        }
      }
    }
  }
  // t handed over by the previous launch as parts (down projection): thread (group, row, column) adds a
  // contiguous run of parts, 16 loads in flight; the runs meet in LDS in run order
  if (a.t_parts) {
    const int lanes_per = 32 * M, groups = kSbThreads / lanes_per;
    const int grp = tid / lanes_per, rest = tid - grp * lanes_per;
    if (grp < groups) {
      const int run = (a.t_nparts + groups - 1) / groups;
      const int p0 = grp * run, p1 = min(p0 + run, a.t_nparts);
      float t = 0.f;
      for (int pb = p0; pb < p1; pb += 16) {
        float pv[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) pv[u] = a.t_parts[(size_t)min(pb + u, a.t_nparts - 1) * lanes_per + rest];
#pragma unroll
        for (int u = 0; u < 16; ++u) t += (pb + u < p1) ? pv[u] : 0.f;
      }
      red_t[grp * lanes_per + rest] = t;  // [group][m][32]
    }
  }

  // ---- prologue: the activations of every row into LDS ----
  if constexpr (PRO == SB_PRO_ATTN) {
    // merge of the context splits of the attention kernel: out = sum_s o_s exp(m_s - m) / sum_s l_s exp(m_s - m)
    const int NH = a.attn_kh * a.attn_g * a.attn_h;  // == K
    for (int e = tid; e < M * NH; e += kSbThreads) {
      const int m = e / NH, rest = e - m * NH, head = rest / a.attn_h, d = rest - head * a.attn_h;
      const int kvh = head / a.attn_g, g = head - kvh * a.attn_g;
      const float* pr = a.attn_part + ((((size_t)m * a.attn_kh + kvh) * a.attn_ns) * a.attn_g + g) * (a.attn_h + 2);
      const size_t sstride = (size_t)a.attn_g * (a.attn_h + 2);
      float pm[8], pl[8], po[8];  // up to 8 splits, every load requested before the first use
#pragma unroll
      for (int sp = 0; sp < 8; ++sp) {
        const size_t o = (size_t)min(sp, a.attn_ns - 1) * sstride;
        pm[sp] = pr[o + a.attn_h];
        pl[sp] = pr[o + a.attn_h + 1];
        po[sp] = pr[o + d];
      }
      float mm = -1e30f;
#pragma unroll
      for (int sp = 0; sp < 8; ++sp) mm = fmaxf(mm, sp < a.attn_ns ? pm[sp] : -1e30f);
      float ls = 0.f, o = 0.f;
#pragma unroll
      for (int sp = 0; sp < 8; ++sp) {
        const float w = sp < a.attn_ns ? __expf(pm[sp] - mm) : 0.f;
        ls += pl[sp] * w;
        o += po[sp] * w;
      }
      xs[m * XS + rest] = f2bf(ls > 0.f ? o / ls : 0.f);
    }
  } else if constexpr (PRO == SB_PRO_PLAIN) {
    const int nchunks = M * (K >> 3), cpr = K >> 3;
    for (int ch = tid; ch < nchunks; ch += kSbThreads) {
      const int m = ch / cpr, cc = ch - m * cpr;
      *reinterpret_cast<uint4*>(xs + m * XS + cc * 8) = *reinterpret_cast<const uint4*>(a.x + (size_t)m * a.ldx + cc * 8);
    }
  } else {
    // RMSNorm of every row: up to 4 chunks of 8 elements per thread (M K <= 16384)
    const int nchunks = M * (K >> 3), cpr = K >> 3;
    float v[4][8];
    float ss[kSbMaxRows] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ch = tid + kSbThreads * i;
      if (ch < nchunks) {
        const int m = ch / cpr, cc = ch - m * cpr;
        const uint4 q = *reinterpret_cast<const uint4*>(a.x + (size_t)m * a.ldx + cc * 8);
        v[i][0] = bf_lo(q.x); v[i][1] = bf_hi(q.x); v[i][2] = bf_lo(q.y); v[i][3] = bf_hi(q.y);
        v[i][4] = bf_lo(q.z); v[i][5] = bf_hi(q.z); v[i][6] = bf_lo(q.w); v[i][7] = bf_hi(q.w);
        float sq = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) sq += v[i][e] * v[i][e];
#pragma unroll
        for (int r = 0; r < kSbMaxRows; ++r) ss[r] += (m == r) ? sq : 0.f;
      }
    }
    // sum of squares of each row over the workgroup, in a fixed order
#pragma unroll
    for (int r = 0; r < kSbMaxRows; ++r) ss[r] = wave_sum(ss[r]);
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < kSbMaxRows; ++r) rms_s[4 + wave * 4 + r] = ss[r];
    }
    __syncthreads();
    if (tid < kSbMaxRows) {
      float t = 0.f;
      for (int w = 0; w < kSbWaves; ++w) t += rms_s[4 + w * 4 + tid];
      rms_s[tid] = sqrtf(t / (float)K + a.eps);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ch = tid + kSbThreads * i;
      if (ch < nchunks) {
        const int m = ch / cpr, cc = ch - m * cpr;
        const float rms = rms_s[m];
        const uint4 wq = *reinterpret_cast<const uint4*>(a.norm_w + cc * 8);
        const float w[8] = {bf_lo(wq.x), bf_hi(wq.x), bf_lo(wq.y), bf_hi(wq.y),
                            bf_lo(wq.z), bf_hi(wq.z), bf_lo(wq.w), bf_hi(wq.w)};
        float o[8];
#pragma unroll
        for (int e = 0; e < 8; ++e)
          o[e] = a.family == TMX_FAMILY_LLAMA3 ? rbf(w[e] * v[i][e]) / rms : w[e] * (v[i][e] / rms);
        uint4 pk;
        pk.x = pack_bf2(o[0], o[1]); pk.y = pack_bf2(o[2], o[3]);
        pk.z = pack_bf2(o[4], o[5]); pk.w = pack_bf2(o[6], o[7]);
        *reinterpret_cast<uint4*>(xs + m * XS + cc * 8) = pk;
      }
    }
  }
  __syncthreads();

  // ---- the K-slice of this wave: its column tile, and its share of x . A ----
  const int xrow = min(nl, M - 1);  // rows beyond the batch repeat the last one (their results are dropped)
  const uint16_t* xb = xs + xrow * XS + h * 8;
  f32x16_t acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  const bool lora_here = a.a_t != nullptr;
  const int RT = a.Rpad >> 5;  // 32-column tiles of A (<= 2)
  // the epilogue uses the t columns of its own segment(s) only: the tiles of A that hold them
  int q0 = 0, q1 = RT - 1;
  if (CT == 1 && lora_here) {
    const int n0 = blockIdx.x * 32;
    const int seg = n0 >= a.seg_end[0] ? (n0 >= a.seg_end[1] ? 2 : 1) : 0;
    q0 = (seg * a.lora_r) >> 5;
    q1 = min(((seg + 1) * a.lora_r - 1) >> 5, RT - 1);
  }
  f32x16_t tacc[2];
#pragma unroll
  for (int q = 0; q < 2; ++q)
#pragma unroll
    for (int r = 0; r < 16; ++r) tacc[q][r] = 0.f;
  // x . A: wave w takes the w-th eighth of K, i.e. the c-th part of its own slice, so the x fragments are
  // the ones it reads anyway.  The A tiles of a k-tile are requested one k-tile ahead.
  const int lpart = (per + CT - 1) / CT;
  auto mine = [&](int i) { return lora_here && i >= c * lpart && i < (c + 1) * lpart && kt0 + i < kt1; };
  u32x4_t ab[2][2][4];  // [parity of the k-tile][tile of A][step]
  auto load_a = [&](int i, auto pc) __attribute__((always_inline)) {
    constexpr int p = decltype(pc)::value;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      if (q < q0 || q > q1) continue;
      const u32x4_t* ap = reinterpret_cast<const u32x4_t*>(a.a_t) + ((size_t)((kt0 + i) * RT + q) * 4) * 64 + lane;
#pragma unroll
      for (int t = 0; t < 4; ++t) ab[p][q][t] = ap[t * 64];
    }
  };
  if (mine(0)) load_a(0, IC<0>{});
  for (int base = 0; base < per; base += kSbMaxTiles) {
    static_for<kSbMaxTiles>([&](auto ic) __attribute__((always_inline)) {
      constexpr int i = decltype(ic)::value;
      const int kt = kt0 + base + i;
      if (kt < kt1) {
        if (mine(base + i + 1)) load_a(base + i + 1, IC<(i + 1) & 1>{});
        bf16x8_t xa[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) xa[t] = *reinterpret_cast<const bf16x8_t*>(xb + kt * 64 + t * 16);
        const float sc = bf2f(sr[i]), m8s = -8.f * sc;
        const uint32_t wd[4] = {wr[i].x, wr[i].y, wr[i].z, wr[i].w};
        if (base + i + kSbMaxTiles < per) {  // slot consumed: refill it for the tile 8 further on
          const int ktn = min(kt + kSbMaxTiles, KT - 1);
          wr[i] = __builtin_nontemporal_load(wsrc + (size_t)ktn * 64);
          sr[i] = ssrc[(size_t)(ktn >> gs) * 32];
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[t], dequant_word<true>(wd[t], sc, m8s), acc, 0, 0, 0);
        if (mine(base + i)) {
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            if (q < q0 || q > q1) continue;
#pragma unroll
            for (int t = 0; t < 4; ++t)
              tacc[q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[t], __builtin_bit_cast(bf16x8_t, ab[i & 1][q][t]), tacc[q], 0, 0, 0);
          }
        }
      }
    });
  }
  // rows 0..3 of a tile are accumulator registers 0..3 of the lanes with h == 0
  if (h == 0) {
#pragma unroll
    for (int r = 0; r < kSbMaxRows; ++r) {
      red[(wave * kSbMaxRows + r) * 32 + nl] = acc[r];
      if (!a.t_parts) {
        red_t[(wave * kSbMaxRows + r) * 64 + nl] = tacc[0][r];
        red_t[(wave * kSbMaxRows + r) * 64 + 32 + nl] = tacc[1][r];
      }
    }
  }
  __syncthreads();
  // t = bf16(sum over the waves, in wave order), or bf16(sum of the runs of handed-over parts, in run order)
  if (tid < kSbMaxRows * 64) {
    const int m = tid >> 6, cc = tid & 63;
    float t = 0.f;
    if (m < M) {
      if (a.t_parts) {
        const int lanes_per = 32 * M, groups = kSbThreads / lanes_per;
        if (cc < 32)
          for (int g = 0; g < groups; ++g) t += red_t[g * lanes_per + m * 32 + cc];
      } else if (lora_here) {
        for (int w = 0; w < kSbWaves; ++w) t += red_t[(w * kSbMaxRows + m) * 64 + cc];
      }
    }
    t_s[m * 64 + cc] = rbf(t);
  }
  __syncthreads();

  // ---- epilogue: thread (row m, column j of the tile) ----
  const bool lora = a.lora_b != nullptr;
  if (epi_thread) {
    const int m = em, j = ej;
    float yv[CT];
#pragma unroll
    for (int q = 0; q < CT; ++q) {
      const int tile = EPI == SB_EPI_SWIGLU ? (int)blockIdx.x + q * a.pair_off : (int)blockIdx.x;
      const int n = tile * 32 + j;
      float b = 0.f;
      for (int sl = 0; sl < KS; ++sl) b += red[((sl * CT + q) * kSbMaxRows + m) * 32 + j];
      b = rbf(b);
      if (lora) {
        const int seg = n >= a.seg_end[0] ? (n >= a.seg_end[1] ? 2 : 1) : 0;
        const float* tp = t_s + m * 64 + seg * a.lora_r;
        float d = 0.f;
#pragma unroll
        for (int rr = 0; rr < 16; ++rr) d = fmaf(rr < a.lora_r ? tp[rr] : 0.f, bf2f(breg[q][rr]), d);
        for (int rr = 16; rr < a.lora_r; ++rr) d = fmaf(tp[rr], bf2f(a.lora_b[(size_t)rr * a.N + n]), d);
        b = rbf(b + rbf(rbf(d) * a.lora_ls));
      }
      yv[q] = b;
    }
    if constexpr (EPI == SB_EPI_SWIGLU) {
      const float g = yv[0], u = yv[CT - 1];
      const float sg = rbf(1.f / (1.f + expf(-g)));
      const float av = rbf(rbf(g * sg) * u);
      a.y[(size_t)m * a.ldy + blockIdx.x * 32 + j] = f2bf(av);
      act_s[m * 32 + j] = av;
    } else {
      const int n = blockIdx.x * 32 + j;
      float v = yv[0];
      if constexpr (EPI == SB_EPI_RESIDUAL) v = rbf(v + bf2f(res_v));
      a.y[(size_t)m * a.ldy + n] = f2bf(v);
    }
  }
  if constexpr (EPI == SB_EPI_SWIGLU) {
    if (a.a_next) {
      // this workgroup's 32 hidden units times their rows of the next projection's A: one part of its t
      __syncthreads();
      if (epi_thread) {
        float t = 0.f;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const uint32_t w[4] = {anx[u].x, anx[u].y, anx[u].z, anx[u].w};
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
            t = fmaf(act_s[em * 32 + u * 8 + 2 * jj], bf_lo(w[jj]), t);
            t = fmaf(act_s[em * 32 + u * 8 + 2 * jj + 1], bf_hi(w[jj]), t);
          }
        }
        a.t_parts_out[((size_t)blockIdx.x * M + em) * 32 + ej] = t;
      }
    }
  }
}

size_t sb_linear_lds(int M, int K) { return sb_x_bytes(M, K) + kSbTailFloats * 4; }

template <int PRO, int EPI>
static int launch_sb(hipStream_t st, const SbLinearArgs& a, int blocks) {
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(&sb_linear_kernel<PRO, EPI>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
  if (attr != hipSuccess) return TMX_ERR_LAUNCH;
  hipLaunchKernelGGL((sb_linear_kernel<PRO, EPI>), dim3(blocks), dim3(kSbThreads), sb_linear_lds(a.M, a.K), st, a);
  return check_launch();
}

bool sb_linear_ok(int M, int K, int N, int G, int rank, int rpad, bool norm) {
  if (M < 1 || M > kSbMaxRows || K % 64 || N % 32 || G % 64 || (G & (G - 1)) || K % G) return false;
  if ((size_t)M * K > (norm ? 16384u : 32768u) || sb_linear_lds(M, K) > 96 * 1024) return false;
  if (rpad > 64 || rank > 32) return false;
  return true;
}

int sb_linear(hipStream_t st, const SbLinearArgs& a, int pro, int epi) {
  if (!a.qw || !a.scales || !a.y) return TMX_ERR_ARG;
  if (!sb_linear_ok(a.M, a.K, a.N, a.G, a.lora_r, a.Rpad, pro == SB_PRO_NORM)) return TMX_ERR_SHAPE;
  if (epi == SB_EPI_SWIGLU) {
    if (pro != SB_PRO_NORM || a.N % 64) return TMX_ERR_UNSUPPORTED;
    return launch_sb<SB_PRO_NORM, SB_EPI_SWIGLU>(st, a, a.N / 64);
  }
  const int blocks = a.N / 32;
  if (pro == SB_PRO_NORM && epi == SB_EPI_PLAIN) return launch_sb<SB_PRO_NORM, SB_EPI_PLAIN>(st, a, blocks);
  if (pro == SB_PRO_ATTN && epi == SB_EPI_RESIDUAL) return launch_sb<SB_PRO_ATTN, SB_EPI_RESIDUAL>(st, a, blocks);
  if (pro == SB_PRO_PLAIN && epi == SB_EPI_RESIDUAL) return launch_sb<SB_PRO_PLAIN, SB_EPI_RESIDUAL>(st, a, blocks);
  if (pro == SB_PRO_PLAIN && epi == SB_EPI_PLAIN) return launch_sb<SB_PRO_PLAIN, SB_EPI_PLAIN>(st, a, blocks);
  return TMX_ERR_UNSUPPORTED;
}

// ---------------------------------------------------------------------------
// Attention of the small-batch step: gqa_decode_kernel's walk over the cache with RoPE and the
// cache write in front.  Workgroup (kv head, row, context split); the q | k | v row comes from the
// projection with its LoRA deltas applied.  Every workgroup rotates the G query heads of its kv
// head into LDS; the one whose split ends at the newest slot also rotates k, writes k and v into
// that slot and reads them back after a barrier with the rest of its positions.  Every split
// leaves (unnormalised output, max, sum) for the o projection's prologue to merge.
template <int H, int G>
__global__ __launch_bounds__(256) void sb_attn_kernel(SbAttnArgs a) {
  constexpr int NW = 4, LPP = H / 8, PPW = 64 / LPP, U = 4, NG = NW * PPW;
  __shared__ float s_m[NG][G], s_l[NG][G];
  __shared__ float s_acc[NG][G][H];
  __shared__ __align__(16) uint16_t q_s[G][H];
  const int kvh = blockIdx.x, b = blockIdx.y, split = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int pg = lane / LPP, dl = lane % LPP;
  const int step = min(*a.step, min(a.C, a.buf_len) - 1);
  const int chunk = (((step + a.nsplit) / a.nsplit) + 31) & ~31;
  const int s_begin = split * chunk;
  int s_end = s_begin + chunk;
  if (s_end > step + 1) s_end = step + 1;
  constexpr int half = H / 2;
  const int ntot = (a.N + 2 * a.Kh) * H;
  const uint16_t* row = a.qkv + (size_t)b * ntot;
  const float* tab = a.rope_tab + (size_t)b * half * 2;
  // Per-head RMSNorm (Qwen3 q_norm / k_norm: f32 with one cast, qwen3/model.py:478-484) of a head vector held as
  // one (x1, x2) pair per lane by `half` consecutive lanes, then the rotation: f32 throughout with one cast for
  // Llama3 (llama3/model.py:249-270); sin / cos and every product rounded to bf16 for Qwen3 (qwen3/model.py:432-453).
  const bool qwen = a.family == TMX_FAMILY_QWEN3;
  auto norm_rotate = [&](float x1, float x2, const uint16_t* nw, int i, float& o1, float& o2) __attribute__((always_inline)) {
    if (nw) {
      float ss = x1 * x1 + x2 * x2;
#pragma unroll
      for (int off = half / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
      const float rms = sqrtf(ss / (float)H + a.eps);
      x1 = rbf(bf2f(nw[i]) * (x1 / rms));
      x2 = rbf(bf2f(nw[i + half]) * (x2 / rms));
    }
    float sn = tab[i * 2], cs = tab[i * 2 + 1];
    if (qwen) {
      sn = rbf(sn);
      cs = rbf(cs);
      o1 = rbf(x1 * cs) - rbf(x2 * sn);
      o2 = rbf(x2 * cs) + rbf(x1 * sn);
    } else {
      o1 = x1 * cs - x2 * sn;
      o2 = x2 * cs + x1 * sn;
    }
  };
  static_assert(G * (H / 2) <= 256, "one (x1, x2) pair of the query heads per thread");
  {  // the G query heads: thread (g, i); the `half` lanes of a head are consecutive and aligned
    const bool act = tid < G * half;
    const int g = act ? tid / half : 0, i = tid % half;
    const uint16_t* qh = row + (size_t)(kvh * G + g) * H;
    float o1, o2;
    norm_rotate(act ? bf2f(qh[i]) : 0.f, act ? bf2f(qh[i + half]) : 0.f, a.q_norm_w, i, o1, o2);
    if (act) {
      q_s[g][i] = f2bf(o1);
      q_s[g][i + half] = f2bf(o2);
    }
  }
  uint16_t* kc = a.kcache + ((size_t)b * a.C * a.Kh + kvh) * H;
  uint16_t* vc = a.vcache + ((size_t)b * a.C * a.Kh + kvh) * H;
  const size_t row_stride = (size_t)a.Kh * H;
  if (s_begin <= step && step < s_end) {  // this split holds the newest slot: write it
    const int slot = step % a.C;
    if (tid < half) {
      const uint16_t* kh = row + (size_t)(a.N + kvh) * H;
      float o1, o2;
      norm_rotate(bf2f(kh[tid]), bf2f(kh[tid + half]), a.k_norm_w, tid, o1, o2);
      kc[(size_t)slot * row_stride + tid] = f2bf(o1);
      kc[(size_t)slot * row_stride + tid + half] = f2bf(o2);
    } else if (tid >= 128 && tid < 128 + H) {
      vc[(size_t)slot * row_stride + (tid - 128)] = row[(size_t)(a.N + a.Kh + kvh) * H + (tid - 128)];
    }
  }
  __syncthreads();  // q in LDS; the new cache row is visible to this workgroup's loads

  uint32_t qf[G][4];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const uint4 v = *reinterpret_cast<const uint4*>(&q_s[g][dl * 8]);
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
  const uint16_t* kbase = kc + dl * 8;
  const uint16_t* vbase = vc + dl * 8;
  const uint8_t* mrow = a.input_mask + (size_t)b * a.buf_len;
  for (int p0 = s_begin + (wave * PPW + pg) * U; p0 < s_end; p0 += NG * U) {
    uint4 kr[U], vr[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = p0 + u;
      ok[u] = p < s_end;
      const int pc = ok[u] ? p : p0;
      kr[u] = *reinterpret_cast<const uint4*>(kbase + (size_t)pc * row_stride);
      vr[u] = *reinterpret_cast<const uint4*>(vbase + (size_t)pc * row_stride);
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
  for (int e = tid; e < G * H; e += 256) {
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
    float* pr = a.partial + ((((size_t)b * a.Kh + kvh) * a.nsplit + split) * G + g) * (H + 2);
    pr[d] = o;
    if (d == 0) {
      pr[H] = mm;
      pr[H + 1] = ls;
    }
  }
}

int sb_attn_splits(int B, int Kh, int C) {
  // enough workgroups to spread the cache walk, few enough parts for the o projection to merge
  int ns = 64 / (B * Kh);
  const int by_len = (C + 127) / 128;
  if (ns > by_len) ns = by_len;
  if (ns > 8) ns = 8;
  return ns < 1 ? 1 : ns;
}

size_t sb_attn_partial_bytes(int B, int N, int Kh, int H, int C) {
  return (size_t)B * N * sb_attn_splits(B, Kh, C) * (H + 2) * sizeof(float);
}

bool sb_attn_ok(int N, int Kh, int H) {
  const int G = Kh > 0 ? N / Kh : 0;
  return Kh > 0 && N % Kh == 0 && (H == 64 || H == 128) && (G == 1 || G == 2 || G == 4);
}

int sb_attn(hipStream_t st, SbAttnArgs a, int H) {
  if (!a.qkv || !a.rope_tab || !a.kcache || !a.vcache || !a.input_mask || !a.step || !a.partial) return TMX_ERR_ARG;
  if (!sb_attn_ok(a.N, a.Kh, H)) return TMX_ERR_UNSUPPORTED;
  const int G = a.N / a.Kh;
  const dim3 grid(a.Kh, a.B, a.nsplit);
#define TMX_SB_ATTN_CASE(HH, GG) \
  if (H == HH && G == GG) { hipLaunchKernelGGL((sb_attn_kernel<HH, GG>), grid, dim3(256), 0, st, a); return check_launch(); }
  TMX_SB_ATTN_CASE(64, 1)
  TMX_SB_ATTN_CASE(64, 2)
  TMX_SB_ATTN_CASE(64, 4)
  TMX_SB_ATTN_CASE(128, 1)
  TMX_SB_ATTN_CASE(128, 2)
  TMX_SB_ATTN_CASE(128, 4)
#undef TMX_SB_ATTN_CASE
  return TMX_ERR_UNSUPPORTED;
}

}  // namespace tmx

using namespace tmx;

extern "C" int tmx_small_linear(void* stream, const void* x, const void* norm_w, float eps, int family,
                                const void* qweight, const void* scales, const void* lora_a_t, const void* lora_b,
                                const void* residual, void* y, int M, int K, int N, int G, int r, int r_pad,
                                float lora_scale, int swiglu) {
  if (!x || !qweight || !scales || !y) return TMX_ERR_ARG;
  if (lora_a_t && (!lora_b || r <= 0 || r_pad < r)) return TMX_ERR_ARG;
  if (swiglu && (!norm_w || residual || (lora_a_t && (r_pad != 32 || 2 * r > 32)))) return TMX_ERR_UNSUPPORTED;
  if (norm_w && residual) return TMX_ERR_UNSUPPORTED;
  SbLinearArgs a = {};
  a.M = M;
  a.x = (const uint16_t*)x; a.ldx = K;
  a.norm_w = (const uint16_t*)norm_w; a.eps = eps; a.family = family;
  a.qw = (const uint4*)qweight; a.scales = (const uint16_t*)scales;
  a.K = K; a.N = N; a.G = G;
  a.seg_end[0] = swiglu ? N / 2 : N; a.seg_end[1] = a.seg_end[2] = N;
  if (lora_a_t) {
    a.a_t = (const uint16_t*)lora_a_t; a.Rpad = r_pad;
    a.lora_b = (const uint16_t*)lora_b; a.lora_r = r; a.lora_ls = lora_scale;
  }
  a.residual = (const uint16_t*)residual;
  a.y = (uint16_t*)y;
  a.ldy = swiglu ? N / 2 : N;
  a.pair_off = swiglu ? N / 64 : 0;
  return sb_linear((hipStream_t)stream, a, norm_w ? 1 : 0, swiglu ? 2 : (residual ? 1 : 0));
}
