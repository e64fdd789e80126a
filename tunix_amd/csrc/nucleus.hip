// Nucleus (top-p) and top-k token selection: the branch of sample_top_p that sorts.
//
// Replaces tunix/generate/sampler.py:136-153:
//   logits_sorted, indices = lax.top_k(z, k)         (descending, lower index first on ties)
//   probs = softmax(logits_sorted); cum = cumsum(probs)
//   logits_sorted[cum - probs > top_p] = -inf
//   token = indices[categorical(key, logits_sorted)]
//   logprob = log_softmax(z)[token]                   (full vocabulary, not renormalised)
//
// The head kernel writes one 64-bit sort key per logit, (row << 32) | ~ordered(z), so one
// device-wide ascending radix sort (rocPRIM, the only library routine of this path) orders every
// row by descending z with ties in index order.  nucleus_select_kernel then walks a row's sorted
// keys in rank order: softmax denominator over the k candidates, running cumulative
// probability, Gumbel-max over the ranks that survive the cut.  The Gumbel noise of rank i of
// row b is drawn at linear index b * k + i (categorical over a [B, k] array).
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/iterator/counting_iterator.hpp>

#include "tmx_kernels.h"
#include "tmx_sampling.h"

namespace tmx {

constexpr int kSelThreads = 1024;
constexpr int kSelItems = 4;

// The key's low word orders the bf16 logit (its low 16 bits only repeat the sign, so the sort
// skips them); z = logit / T is the same f32 division the head kernel makes.
__device__ __forceinline__ float z_of_key(uint64_t key, float temperature) {
  const uint32_t o = ~(uint32_t)key;
  return __uint_as_float((o & 0x80000000u) ? (o ^ 0x80000000u) : ~o) / temperature;
}

__global__ __launch_bounds__(kSelThreads) void nucleus_select_kernel(NucleusArgs a) {
  __shared__ float s_w[16];
  __shared__ float s_f[16][4];
  __shared__ int s_i[16];
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const size_t base = (size_t)row * a.V;
  const int k = a.k;
  const float z0 = z_of_key(a.keys[base], a.temperature);

  // full-vocabulary log-sum-exp from the head kernel's per-workgroup partials
  float mx = kNegBig, se = 0.f;
  for (int i = tid; i < a.nwg; i += kSelThreads) {
    const float* pf = a.part_f + ((size_t)row * a.nwg + i) * 4;
    lse_merge(mx, se, pf[0], pf[1]);
  }
  // softmax denominator over the k candidates
  float s = 0.f;
  for (int i = tid; i < k; i += kSelThreads) s += expf(z_of_key(a.keys[base + i], a.temperature) - z0);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    lse_merge(mx, se, __shfl_xor(mx, off, 64), __shfl_xor(se, off, 64));
    s += __shfl_xor(s, off, 64);
  }
  if (lane == 0) { s_f[wave][0] = mx; s_f[wave][1] = se; s_f[wave][2] = s; }
  __syncthreads();
  mx = s_f[0][0]; se = s_f[0][1];
  float denom = s_f[0][2];
  for (int w = 1; w < 16; ++w) {
    lse_merge(mx, se, s_f[w][0], s_f[w][1]);
    denom += s_f[w][2];
  }
  __syncthreads();

  uint32_t key0, key1;
  threefry2x32(a.k0, a.k1, 0u, (uint32_t)*a.step, key0, key1);

  float carry = 0.f;
  Best best = {-INFINITY, -INFINITY, 0x7FFFFFFF};
  for (int c0 = 0; c0 < k; c0 += kSelThreads * kSelItems) {
    const int i0 = c0 + tid * kSelItems;
    float p[kSelItems], z[kSelItems];
    float t = 0.f;
#pragma unroll
    for (int j = 0; j < kSelItems; ++j) {
      const int i = i0 + j;
      z[j] = i < k ? z_of_key(a.keys[base + i], a.temperature) : -INFINITY;
      p[j] = i < k ? expf(z[j] - z0) / denom : 0.f;
      t += p[j];
    }
    float inc = t;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float v = __shfl_up(inc, off, 64);
      if (lane >= off) inc += v;
    }
    if (lane == 63) s_w[wave] = inc;
    __syncthreads();
    float wpre = 0.f, total = 0.f;
    for (int w = 0; w < 16; ++w) {
      if (w < wave) wpre += s_w[w];
      total += s_w[w];
    }
    float cs = carry + wpre + (inc - t);
    bool cut = false;
#pragma unroll
    for (int j = 0; j < kSelItems; ++j) {
      const int i = i0 + j;
      cs += p[j];
      const bool masked = (cs - p[j]) > a.top_p;
      if (i < k) {
        cut = cut || masked;
        if (!masked) {
          uint32_t o0, o1;
          threefry2x32(key0, key1, 0u, (uint32_t)row * (uint32_t)k + (uint32_t)i, o0, o1);
          Best c = {z[j] + gumbel_from_bits(o0 ^ o1), z[j], i};
          best_merge(best, c);
        }
      }
    }
    carry += total;
    // cum - p never decreases along the ranks, so nothing after a cut survives
    if (__syncthreads_or(cut ? 1 : 0)) break;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    Best o = {__shfl_xor(best.key, off, 64), __shfl_xor(best.z, off, 64), __shfl_xor(best.idx, off, 64)};
    best_merge(best, o);
  }
  if (lane == 0) { s_f[wave][2] = best.key; s_f[wave][3] = best.z; s_i[wave] = best.idx; }
  __syncthreads();
  if (tid == 0) {
    best = {s_f[0][2], s_f[0][3], s_i[0]};
    for (int w = 1; w < 16; ++w) {
      Best o = {s_f[w][2], s_f[w][3], s_i[w]};
      best_merge(best, o);
    }
    const int tok = (int)(a.vals[base + best.idx] - (uint32_t)base);
    const int col = *a.step + 1;
    if (col >= a.buf_len) return;
    a.token_buffer[(size_t)row * a.buf_len + col] = tok;
    if (a.logprobs) a.logprobs[(size_t)row * a.buf_len + col] = (best.z - mx) - logf(se);
    bool hit = false;
    for (int e = 0; e < a.n_eos; ++e) hit = hit || (a.eos[e] == tok);
    if (hit) a.done[row] = 1;
  }
}

static int row_bits(int M) {
  int b = 0;
  while ((1 << b) < M) ++b;
  return b;
}

static hipError_t sort_rows(void* tmp, size_t& tmp_bytes, const uint64_t* kin, uint64_t* kout,
                            uint32_t* vout, int M, int V, hipStream_t st) {
  return rocprim::radix_sort_pairs(tmp, tmp_bytes, kin, kout, rocprim::counting_iterator<uint32_t>(0),
                                   vout, (size_t)M * V, 16u, (unsigned)(32 + row_bits(M)), st, false);
}

// keys in | keys out | values out | sort scratch
struct NucleusCarve {
  uint64_t *kin, *kout;
  uint32_t* vout;
  void* tmp;
  size_t tmp_bytes, total;
};
static NucleusCarve nucleus_carve(int M, int V, char* base, size_t sort_tmp) {
  NucleusCarve c;
  size_t off = 0;
  auto take = [&](size_t n) { char* p = base ? base + off : nullptr; off += (n + 255) & ~(size_t)255; return p; };
  const size_t n = (size_t)M * V;
  c.kin = (uint64_t*)take(n * 8);
  c.kout = (uint64_t*)take(n * 8);
  c.vout = (uint32_t*)take(n * 4);
  c.tmp = take(sort_tmp);
  c.tmp_bytes = sort_tmp;
  c.total = off;
  return c;
}

size_t nucleus_bytes(int M, int V) {
  if (M <= 0 || V <= 0 || (size_t)M * V >= (1ull << 32)) return 0;
  size_t sort_tmp = 0;
  if (sort_rows(nullptr, sort_tmp, nullptr, nullptr, nullptr, M, V, nullptr) != hipSuccess) return 0;
  return nucleus_carve(M, V, nullptr, sort_tmp).total;
}

int head_sample_nucleus(hipStream_t st, HeadArgs a, float top_p, int top_k, void* ws, size_t ws_bytes) {
  if (a.V % 32 || a.D % 64 || a.M <= 0 || a.M > TMX_MAX_FILL_ROWS) return TMX_ERR_SHAPE;
  if (!ws || !(top_p >= 0.f)) return TMX_ERR_ARG;
  size_t sort_tmp = 0;
  if (sort_rows(nullptr, sort_tmp, nullptr, nullptr, nullptr, a.M, a.V, st) != hipSuccess)
    return TMX_ERR_LAUNCH;
  const NucleusCarve c = nucleus_carve(a.M, a.V, (char*)ws, sort_tmp);
  if (c.total > ws_bytes) return TMX_ERR_SHAPE;
  a.mode = TMX_SAMPLE_TOP_P;
  a.sort_keys = c.kin;
  int rc = head_logits(st, a);
  if (rc != TMX_OK) return rc;
  size_t tb = c.tmp_bytes;
  if (sort_rows(c.tmp, tb, c.kin, c.kout, c.vout, a.M, a.V, st) != hipSuccess) return TMX_ERR_LAUNCH;
  NucleusArgs n = {};
  n.keys = c.kout; n.vals = c.vout;
  n.M = a.M; n.V = a.V;
  n.k = (top_k > 0 && top_k < a.V) ? top_k : a.V;
  n.top_p = top_p;
  n.temperature = a.temperature;
  n.k0 = a.k0; n.k1 = a.k1;
  n.step = a.step;
  n.part_f = a.part_f; n.nwg = a.nwg;
  n.token_buffer = a.token_buffer; n.logprobs = a.logprobs; n.done = a.done;
  n.eos = a.eos; n.n_eos = a.n_eos; n.buf_len = a.buf_len;
  hipLaunchKernelGGL(nucleus_select_kernel, dim3(a.M), dim3(kSelThreads), 0, st, n);
  return check_launch();
}

}  // namespace tmx

using namespace tmx;

extern "C" size_t tmx_nucleus_workspace_bytes(int M, int V) { return nucleus_bytes(M, V); }

extern "C" int tmx_head_sample_nucleus(void* stream, const void* x, const void* head_w, int M, int D, int V,
                                       float temperature, float top_p, int top_k, uint32_t seed_hi,
                                       uint32_t seed_lo, const int32_t* step, const int32_t* forbidden,
                                       int n_forbidden, const int32_t* eos, int n_eos, int32_t* token_buffer,
                                       float* logprobs, uint8_t* done, int buf_len, void* workspace,
                                       void* nucleus_workspace, size_t nucleus_workspace_bytes) {
  if (!x || !head_w || !step || !token_buffer || !done || !workspace || !nucleus_workspace) return TMX_ERR_ARG;
  if ((n_forbidden > 0 && !forbidden) || (n_eos > 0 && !eos)) return TMX_ERR_ARG;
  HeadArgs a = {};
  a.x = (const uint16_t*)x;
  a.w = (const uint16_t*)head_w;
  a.M = M; a.D = D; a.V = V;
  a.temperature = temperature;
  a.k0 = seed_hi; a.k1 = seed_lo;
  a.step = step;
  a.forbidden = forbidden; a.n_forbidden = n_forbidden;
  const size_t nwg = (V + 127) / 128;
  a.part_f = (float*)workspace;
  a.part_i = (int32_t*)((float*)workspace + (size_t)M * nwg * 4);
  a.token_buffer = token_buffer;
  a.logprobs = logprobs;
  a.done = done;
  a.eos = eos; a.n_eos = n_eos;
  a.buf_len = buf_len;
  return head_sample_nucleus((hipStream_t)stream, a, top_p, top_k, nucleus_workspace, nucleus_workspace_bytes);
}
