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


// waves per workgroup: fewer for wide groups so the merge buffers stay under 64 KiB
template <int G>
struct AttnWaves { static constexpr int value = G > 4 ? 2 : 4; };

template <int H, int G>
__global__ __launch_bounds__(AttnWaves<G>::value * 64) void gqa_decode_kernel(AttnArgs a) {
  constexpr int NW = AttnWaves<G>::value;
  constexpr int LPP = H / 8;     // lanes per position row
  constexpr int PPW = 64 / LPP;  // positions per wave-wide load
  constexpr int U = 4;           // positions per lane group per iteration
  constexpr int NG = NW * PPW;   // lane groups per workgroup
  __shared__ float s_m[NG][G], s_l[NG][G];
  __shared__ float s_acc[NG][G][H];

  const int kvh = blockIdx.x, b = blockIdx.y, split = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pg = lane / LPP, dl = lane % LPP;  // lane group, 8-element slice index
  const int tpp = a.tpp > 0 ? a.tpp : 1;
  const int seq = b / tpp;                    // b: query row of this pass
  const int step = *a.step + b % tpp;
  // the splits share the VALID positions 0 .. step (not the cache size) in chunks of whole
  // 32 positions, so that every split has work at any context length
  const int chunk = (((step + a.nsplit) / a.nsplit) + 31) & ~31;
  const int s_begin = split * chunk;
  int s_end = s_begin + chunk;
  if (s_end > step + 1) s_end = step + 1;

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
    if (a.nsplit == 1) {
      a.out[((size_t)b * a.N + kvh * G + g) * H + d] = f2bf(ls > 0.f ? o / ls : 0.f);
    } else {
      float* pr = a.partial + ((((size_t)b * a.Kh + kvh) * a.nsplit + split) * G + g) * (H + 2);
      pr[d] = o;
      if (d == 0) {
        pr[H] = mm;
        pr[H + 1] = ls;
      }
    }
  }
}

template <int H, int G>
__global__ __launch_bounds__(H) void gqa_combine_kernel(AttnArgs a) {
  const int kvh = blockIdx.x, b = blockIdx.y, g = blockIdx.z, d = threadIdx.x;
  const float* pr = a.partial + (((size_t)b * a.Kh + kvh) * a.nsplit * G + g) * (H + 2);
  const size_t sstride = (size_t)G * (H + 2);
  float mm = -1e30f;
  for (int s = 0; s < a.nsplit; ++s) mm = fmaxf(mm, pr[s * sstride + H]);
  float ls = 0.f, o = 0.f;
  for (int s = 0; s < a.nsplit; ++s) {
    const float w = __expf(pr[s * sstride + H] - mm);
    ls += pr[s * sstride + H + 1] * w;
    o += pr[s * sstride + d] * w;
  }
  a.out[((size_t)b * a.N + kvh * G + g) * H + d] = f2bf(ls > 0.f ? o / ls : 0.f);
}

template <int H, int G>
static int launch_attn(hipStream_t st, const AttnArgs& a) {
  hipLaunchKernelGGL((gqa_decode_kernel<H, G>), dim3(a.Kh, a.B, a.nsplit), dim3(AttnWaves<G>::value * 64), 0, st, a);
  int rc = check_launch();
  if (rc != TMX_OK || a.nsplit == 1) return rc;
  hipLaunchKernelGGL((gqa_combine_kernel<H, G>), dim3(a.Kh, a.B, G), dim3(H), 0, st, a);
  return check_launch();
}

// Number of sequence splits that brings the grid to roughly two workgroups per CU (more splits
// cost more in partial sums and the combine launch than they gain at rollout batch sizes).
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

size_t attn_partial_bytes(int B, int N, int Kh, int H, int C) {
  const int ns = attn_num_splits(B, Kh, C);
  return ns == 1 ? 0 : (size_t)B * N * ns * (H + 2) * sizeof(float);
}

int gqa_decode(hipStream_t st, AttnArgs a, int H) {
  a.nsplit = attn_num_splits(a.B, a.Kh, a.C);
  if (a.nsplit > 1 && !a.partial) return TMX_ERR_ARG;
  const int G = a.N / a.Kh;
  if (a.N % a.Kh) return TMX_ERR_SHAPE;
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
