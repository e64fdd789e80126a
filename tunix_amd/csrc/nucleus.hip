// Nucleus (top-p) and top-k token selection: the branch of sample_top_p that sorts.
//
// Replaces tunix/generate/sampler.py:136-153:
//   logits_sorted, indices = lax.top_k(z, k)         (descending, lower index first on ties)
//   probs = softmax(logits_sorted); cum = cumsum(probs)
//   logits_sorted[cum - probs > top_p] = -inf
//   token = indices[categorical(key, logits_sorted)]
//   logprob = log_softmax(z)[token]                   (full vocabulary, not renormalised)
//
// No sort is needed.  The logits are bf16 values, so a row holds at most 65 536 distinct ones:
// the head kernel writes one 16-bit ordered key per logit (ascending key = descending logit) and
// everything the rule needs follows from the per-row COUNT of every key value:
//   * the rank of the first candidate of a value = number of candidates with a larger value;
//     equal values rank in index order, so the e-th occurrence of a value (in index order) has
//     rank base + e;
//   * every candidate of a value has the same probability, so the cumulative probability in front
//     of rank base + e is (mass in front of the value + e * exp(z - max)) / denominator;
//   * the Gumbel noise of a candidate depends on its rank alone (categorical over the [B, k]
//     array of sorted logits draws at linear index b * k + rank), so the winner is found by
//     walking the surviving RANKS, never the elements; only the winner's (value, occurrence) is
//     turned back into a token id, by one scan of the row's keys.
// Three launches: nucleus_hist_kernel (per row and sign half: LDS histogram of 32 768 counters,
// prefix counts and masses of the populated values, compacted), nucleus_eval_kernel (per row and
// slice of the rank range: cut + Gumbel-max over the surviving ranks), nucleus_pick_kernel (per
// row: merge the slices, locate the winner's token, write token / log-prob / done).  Nothing here
// allocates or calls a library, so the step can be recorded into a HIP graph.
#include "tmx_kernels.h"
#include "tmx_sampling.h"

namespace tmx {

constexpr int kNT = 1024;          // threads of every kernel here
constexpr int kHalfBins = 32768;   // key values per sign half
constexpr float kGumbelMax = 16.f; // no draw exceeds it: -log(-log(1 - 2^-23)) = 15.94

// bf16 logit of a 16-bit descending key (see head_kernel: non-negative values count down from
// 0x7FFF, negative ones up from 0x8000), divided by the temperature like the head kernel does.
__device__ __forceinline__ float z_of_dk(uint32_t dk, float temperature) {
  const uint32_t b16 = (dk & 0x8000u) ? dk : (~dk & 0x7FFFu);
  return __uint_as_float(b16 << 16) / temperature;
}

// Entries of one (row, half): populated key values in rank order with the exclusive prefix of
// their counts and of their unnormalised masses count * exp(z - max) inside the half.
struct Entries {
  const uint32_t *key, *cnt, *mass;  // [n]
};
__device__ __forceinline__ Entries entries_of(const uint32_t* ent, int row, int half) {
  const uint32_t* b = ent + ((size_t)row * 2 + half) * 3 * kHalfBins;
  return {b, b + kHalfBins, b + 2 * kHalfBins};
}

// Both halves of a row seen as one list of n0 + n1 values in rank order.
struct RowList {
  Entries e0, e1;
  int n0, n1;
  uint32_t c0, c1;  // candidates per half
  float m0, m1;     // mass per half
  float mx;         // largest z of the row
  __device__ __forceinline__ uint32_t key(int j) const { return j < n0 ? e0.key[j] : e1.key[j - n0]; }
  __device__ __forceinline__ uint32_t base(int j) const {  // rank of the value's first candidate
    return j < n0 ? e0.cnt[j] : (j < n0 + n1 ? c0 + e1.cnt[j - n0] : c0 + c1);
  }
  __device__ __forceinline__ float mass(int j) const {
    return j < n0 ? __uint_as_float(e0.mass[j]) : m0 + __uint_as_float(e1.mass[j - n0]);
  }
  // index of the value that holds rank r (r below the number of candidates); `staged` is an LDS
  // copy of base(0 .. n0 + n1 - 1) made by stage_bases(), or null when the list did not fit
  __device__ __forceinline__ int value_of_rank(uint32_t r, const uint32_t* staged) const {
    int lo = 0, hi = n0 + n1 - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if ((staged ? staged[mid] : base(mid)) <= r) lo = mid; else hi = mid - 1;
    }
    return lo;
  }
};
constexpr int kStageCap = 12288;  // values whose first ranks fit the 48 KiB staging area (three workgroups per CU)
// Copies the first ranks of all values into LDS (every thread of the workgroup calls it); returns
// the LDS array, or null when there are more values than it holds.  Ends with a barrier.
__device__ __forceinline__ const uint32_t* stage_bases(const RowList& l, uint32_t* lds) {
  const int n = l.n0 + l.n1;
  if (n > kStageCap) return nullptr;
  for (int j = threadIdx.x; j < n; j += kNT) lds[j] = l.base(j);
  __syncthreads();
  return lds;
}
__device__ __forceinline__ RowList row_list(const uint32_t* ent, const uint32_t* tot, int row) {
  RowList l;
  l.e0 = entries_of(ent, row, 0);
  l.e1 = entries_of(ent, row, 1);
  const uint32_t* t = tot + (size_t)row * 8;
  l.n0 = (int)t[0]; l.c0 = t[1]; l.m0 = __uint_as_float(t[2]); l.mx = __uint_as_float(t[3]);
  l.n1 = (int)t[4]; l.c1 = t[5]; l.m1 = __uint_as_float(t[6]);
  return l;
}

// Exclusive prefix over the workgroup's threads, in thread order (so float sums are reproducible);
// `total` receives the sum over all threads.  smem: 16 values.
template <class T>
__device__ __forceinline__ T block_excl_scan(T v, T* smem, T& total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  T inc = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const T u = __shfl_up(inc, off, 64);
    if (lane >= off) inc += u;
  }
  __syncthreads();
  if (lane == 63) smem[wave] = inc;
  __syncthreads();
  T pre = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < kNT / 64; ++w) {
    if (w < wave) pre += smem[w];
    tot += smem[w];
  }
  total = tot;
  return pre + inc - v;
}

// grid (2, M): half 0 counts the non-negative logits of a row, half 1 the negative ones.
__global__ __launch_bounds__(kNT) void nucleus_hist_kernel(NucleusArgs a) {
  extern __shared__ uint32_t hist[];  // [kHalfBins]
  __shared__ float s_f[16];
  __shared__ uint32_t s_u[16];
  const int half = blockIdx.x, row = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < kHalfBins; i += kNT) hist[i] = 0;
  // largest z of the row (the softmax reference point) from the head kernel's partials
  float mx = kNegBig;
  for (int i = tid; i < a.nwg; i += kNT) mx = fmaxf(mx, a.part_f[((size_t)row * a.nwg + i) * 4]);
  mx = wave_max(mx);
  if (lane == 0) s_f[wave] = mx;
  __syncthreads();
  mx = s_f[0];
#pragma unroll
  for (int w = 1; w < kNT / 64; ++w) mx = fmaxf(mx, s_f[w]);
  // count this half's keys, 8 per 16-byte load, 8 loads in flight per thread
  const uint4* kp = reinterpret_cast<const uint4*>(a.keys + (size_t)row * a.V);
  const int nvec = a.V >> 3;
  for (int i0 = tid; i0 < nvec; i0 += 8 * kNT) {
    uint4 q[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kNT;
      q[u] = kp[i < nvec ? i : nvec - 1];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (i0 + u * kNT >= nvec) break;
      const uint32_t w[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t k0 = w[j] & 0xFFFFu, k1 = w[j] >> 16;
        if ((int)(k0 >> 15) == half) atomicAdd(&hist[k0 & 0x7FFFu], 1u);
        if ((int)(k1 >> 15) == half) atomicAdd(&hist[k1 & 0x7FFFu], 1u);
      }
    }
  }
  __syncthreads();
  // Populated values are few (bf16 logits of one row: hundreds to thousands of the 32 768), so they are
  // compacted first, in rank order: wave w owns values 2048 w .. 2048 w + 2047, 64 consecutive values
  // per round (lane = value: conflict-free LDS reads), positions from ballots.  The prefix sums then
  // run over the compacted list.
  constexpr int PER_WAVE = kHalfBins / (kNT / 64), ROUNDS = PER_WAVE / 64;
  const uint32_t dk0 = ((uint32_t)half << 15) | (uint32_t)(wave * PER_WAVE);
  uint32_t npop = 0;
  for (int it = 0; it < ROUNDS; ++it)
    npop += (uint32_t)__popcll(__ballot(hist[wave * PER_WAVE + it * 64 + lane] != 0));
  __shared__ uint32_t w_pop[kNT / 64];
  if (lane == 0) w_pop[wave] = npop;
  __syncthreads();
  uint32_t ppre = 0, pop_tot = 0;
  for (int w = 0; w < kNT / 64; ++w) {
    if (w < wave) ppre += w_pop[w];
    pop_tot += w_pop[w];
  }
  uint32_t* eb = a.ent + ((size_t)row * 2 + half) * 3 * kHalfBins;
  for (int it = 0; it < ROUNDS; ++it) {
    const uint32_t c = hist[wave * PER_WAVE + it * 64 + lane];
    const unsigned long long m = __ballot(c != 0);
    if (c) {
      const uint32_t pos = ppre + (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
      eb[pos] = dk0 + it * 64 + lane;
      eb[kHalfBins + pos] = c;  // raw count for now
    }
    ppre += (uint32_t)__popcll(m);
  }
  __syncthreads();  // the list is read back by other threads of this workgroup
  // thread t takes entries t C .. t C + C - 1: exclusive prefixes of counts and masses in entry order
  // (a fixed summation order: the same float sums on every run)
  const uint32_t C = (pop_tot + kNT - 1) / kNT;
  const uint32_t j0 = (uint32_t)tid * C, j1 = j0 + C < pop_tot ? j0 + C : pop_tot;
  uint32_t cnt = 0;
  float mass = 0.f;
  for (uint32_t q = j0; q < j1; ++q) {
    const uint32_t c = eb[kHalfBins + q];
    cnt += c;
    mass += (float)c * expf(z_of_dk(eb[q], a.temperature) - mx);
  }
  uint32_t cnt_tot;
  float mass_tot;
  uint32_t cpre = block_excl_scan<uint32_t>(cnt, s_u, cnt_tot);
  float mpre = block_excl_scan<float>(mass, s_f, mass_tot);
  for (uint32_t q = j0; q < j1; ++q) {
    const uint32_t c = eb[kHalfBins + q];
    eb[kHalfBins + q] = cpre;
    eb[2 * kHalfBins + q] = __float_as_uint(mpre);
    cpre += c;
    mpre += (float)c * expf(z_of_dk(eb[q], a.temperature) - mx);
  }
  if (tid == 0) {
    uint32_t* t = a.tot + (size_t)row * 8 + half * 4;
    t[0] = pop_tot; t[1] = cnt_tot; t[2] = __float_as_uint(mass_tot); t[3] = __float_as_uint(mx);
  }
}

// grid (slices, M): slice s of row b walks ranks [s R, (s + 1) R) of the k candidates.
__global__ __launch_bounds__(kNT) void nucleus_eval_kernel(NucleusArgs a) {
  extern __shared__ uint32_t stage[];  // [kStageCap]
  __shared__ float s_f[16][2];
  __shared__ int s_i[16];
  const int slice = blockIdx.x, row = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const RowList l = row_list(a.ent, a.tot, row);
  const uint32_t* staged = stage_bases(l, stage);
  const uint32_t total = l.c0 + l.c1;
  const uint32_t k = (uint32_t)a.k < total ? (uint32_t)a.k : total;
  // softmax denominator over the k candidates
  float denom = l.m0 + l.m1;
  if (k < total) {
    const int j = l.value_of_rank(k, staged);
    denom = l.mass(j) + (float)(k - l.base(j)) * expf(z_of_dk(l.key(j), a.temperature) - l.mx);
  }
  uint32_t key0, key1;
  threefry2x32(a.k0, a.k1, 0u, (uint32_t)*a.step, key0, key1);

  const uint32_t R = (k + gridDim.x - 1) / gridDim.x;
  const uint32_t s_begin = (uint32_t)slice * R, s_end = s_begin + R < k ? s_begin + R : k;
  Best best = {-INFINITY, -INFINITY, 0x7FFFFFFF};
  if (s_begin < s_end) {
    const uint32_t C = (s_end - s_begin + kNT - 1) / kNT;
    uint32_t r = s_begin + (uint32_t)tid * C;
    const uint32_t r_end = r + C < s_end ? r + C : s_end;
    if (r < r_end) {
      int j = l.value_of_rank(r, staged);
      uint32_t jb = l.base(j), jn = l.base(j + 1);
      float zj = z_of_dk(l.key(j), a.temperature), ej = expf(zj - l.mx), mj = l.mass(j);
      for (; r < r_end; ++r) {
        while (r >= jn) {
          ++j;
          jb = jn; jn = l.base(j + 1);
          zj = z_of_dk(l.key(j), a.temperature); ej = expf(zj - l.mx); mj = l.mass(j);
        }
        // cumulative probability in front of this rank; it never decreases along the ranks
        const float before = (mj + (float)(r - jb) * ej) / denom;
        if (before > a.top_p) break;
        if (zj + kGumbelMax < best.key) continue;  // cannot win whatever its draw
        uint32_t o0, o1;
        threefry2x32(key0, key1, 0u, (uint32_t)row * k + r, o0, o1);
        Best c = {zj + gumbel_from_bits(o0 ^ o1), zj, (int)r};
        best_merge(best, c);
      }
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    Best o = {__shfl_xor(best.key, off, 64), __shfl_xor(best.z, off, 64), __shfl_xor(best.idx, off, 64)};
    best_merge(best, o);
  }
  if (lane == 0) { s_f[wave][0] = best.key; s_f[wave][1] = best.z; s_i[wave] = best.idx; }
  __syncthreads();
  if (tid == 0) {
    best = {s_f[0][0], s_f[0][1], s_i[0]};
    for (int w = 1; w < kNT / 64; ++w) {
      Best o = {s_f[w][0], s_f[w][1], s_i[w]};
      best_merge(best, o);
    }
    float* pb = a.pbest + ((size_t)row * gridDim.x + slice) * 4;
    pb[0] = best.key; pb[1] = best.z; pb[2] = __int_as_float(best.idx);
  }
}

// grid (M): merge the slices' winners, turn (value, occurrence) into the token id, write the outputs.
__global__ __launch_bounds__(kNT) void nucleus_pick_kernel(NucleusArgs a) {
  extern __shared__ uint32_t stage[];  // [kStageCap]
  __shared__ float s_f[16][2];
  __shared__ uint32_t s_u[16];
  __shared__ int s_tok;
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // full-vocabulary log-sum-exp from the head kernel's per-workgroup partials
  float mx = kNegBig, se = 0.f;
  for (int i = tid; i < a.nwg; i += kNT) {
    const float* pf = a.part_f + ((size_t)row * a.nwg + i) * 4;
    lse_merge(mx, se, pf[0], pf[1]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) lse_merge(mx, se, __shfl_xor(mx, off, 64), __shfl_xor(se, off, 64));
  if (lane == 0) { s_f[wave][0] = mx; s_f[wave][1] = se; }
  if (tid == 0) s_tok = 0;
  __syncthreads();
  mx = s_f[0][0]; se = s_f[0][1];
  for (int w = 1; w < kNT / 64; ++w) lse_merge(mx, se, s_f[w][0], s_f[w][1]);
  // the row's winner (every thread merges the few slices itself)
  Best best = {-INFINITY, -INFINITY, 0x7FFFFFFF};
  for (int s = 0; s < a.ns; ++s) {
    const float* pb = a.pbest + ((size_t)row * a.ns + s) * 4;
    Best o = {pb[0], pb[1], __float_as_int(pb[2])};
    best_merge(best, o);
  }
  const RowList l = row_list(a.ent, a.tot, row);
  const uint32_t* staged = stage_bases(l, stage);
  const uint32_t rank = best.idx == 0x7FFFFFFF ? 0u : (uint32_t)best.idx;  // nothing drawable: the first candidate
  const int j = l.value_of_rank(rank, staged);
  const uint32_t want = l.key(j), occ = rank - l.base(j);
  // The occ-th key equal to `want` in index order.  Wave w scans the w-th sixteenth of the row with
  // coalesced 16-byte loads (8 keys per lane and load); the wave whose piece holds the occurrence
  // walks it again, counting per load instruction with ballots over the bit planes of the lanes'
  // match counts (0..8), so the order (load, lane, key) is the index order.
  const int nvec = a.V >> 3, per_wave = (nvec + kNT / 64 - 1) / (kNT / 64);
  const int wb = wave * per_wave, we = min(wb + per_wave, nvec);
  const uint4* kp = reinterpret_cast<const uint4*>(a.keys + (size_t)row * a.V);
  auto matches = [&](const uint4& q) {
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
    uint32_t m = 0;
#pragma unroll
    for (int t = 0; t < 4; ++t) m += ((w[t] & 0xFFFFu) == want) + ((w[t] >> 16) == want);
    return m;
  };
  uint32_t mine = 0;
  for (int i0 = wb + lane; i0 < we; i0 += 8 * 64) {  // 8 loads in flight
    uint4 q[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) q[u] = kp[min(i0 + u * 64, we - 1)];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (i0 + u * 64 < we) mine += matches(q[u]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mine += __shfl_xor(mine, off, 64);
  if (lane == 0) s_u[wave] = mine;
  __syncthreads();
  uint32_t pre = 0;
  for (int w = 0; w < wave; ++w) pre += s_u[w];
  if (occ >= pre && occ < pre + mine) {  // wave-uniform: this wave's piece holds the winner
    const unsigned long long below = (1ull << lane) - 1ull;
    uint32_t seen = pre;
    bool found = false;
    for (int b0 = wb; b0 < we && !found; b0 += 8 * 64) {
      uint4 q[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) q[u] = kp[min(b0 + u * 64 + lane, we - 1)];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (found) break;
        const int i = b0 + u * 64 + lane;
        const uint32_t m = i < we ? matches(q[u]) : 0u;
        uint32_t tot = 0, lpre = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const unsigned long long plane = __ballot((m >> b) & 1u);
          tot += (uint32_t)__popcll(plane) << b;
          lpre += (uint32_t)__popcll(plane & below) << b;
        }
        if (occ < seen + tot) {
          if (occ >= seen + lpre && occ < seen + lpre + m) {
            uint32_t left = occ - seen - lpre;
            const uint32_t w[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
#pragma unroll
            for (int t = 0; t < 8; ++t) {
              const uint32_t kv = (t & 1) ? (w[t >> 1] >> 16) : (w[t >> 1] & 0xFFFFu);
              if (kv == want && left-- == 0) s_tok = i * 8 + t;
            }
          }
          found = true;
        }
        seen += tot;
      }
    }
  }
  __syncthreads();
  if (tid == 0) {
    const int tok = s_tok;
    const int col = *a.step + 1;
    if (col >= a.buf_len) return;
    a.token_buffer[(size_t)row * a.buf_len + col] = tok;
    if (a.logprobs) a.logprobs[(size_t)row * a.buf_len + col] = (best.z - mx) - logf(se);
    bool hit = false;
    for (int e = 0; e < a.n_eos; ++e) hit = hit || (a.eos[e] == tok);
    if (hit) a.done[row] = 1;
  }
}

// Slices of the rank range per row: enough workgroups to occupy the chip at any row count.
static int nucleus_slices(int M) {
  int ns = 512 / (M > 0 ? M : 1);
  return ns < 1 ? 1 : (ns > 64 ? 64 : ns);
}

// keys | entries | totals | slice winners
struct NucleusCarve {
  uint16_t* keys;
  uint32_t *ent, *tot;
  float* pbest;
  size_t total;
};
static NucleusCarve nucleus_carve(int M, int V, char* base) {
  NucleusCarve c;
  size_t off = 0;
  auto take = [&](size_t n) { char* p = base ? base + off : nullptr; off += (n + 255) & ~(size_t)255; return p; };
  c.keys = (uint16_t*)take((size_t)M * V * 2);
  c.ent = (uint32_t*)take((size_t)M * 2 * 3 * kHalfBins * 4);
  c.tot = (uint32_t*)take((size_t)M * 8 * 4);
  c.pbest = (float*)take((size_t)M * 64 * 4 * 4);
  c.total = off;
  return c;
}

size_t nucleus_bytes(int M, int V) {
  if (M <= 0 || V <= 0 || V % 32 || (size_t)M * V >= (1ull << 32)) return 0;
  return nucleus_carve(M, V, nullptr).total;
}

int head_sample_nucleus(hipStream_t st, HeadArgs a, float top_p, int top_k, void* ws, size_t ws_bytes) {
  if (a.V % 32 || a.D % 64 || a.M <= 0 || a.M > TMX_MAX_FILL_ROWS || (size_t)a.M * a.V >= (1ull << 32))
    return TMX_ERR_SHAPE;
  if (!ws || !(top_p >= 0.f)) return TMX_ERR_ARG;
  const NucleusCarve c = nucleus_carve(a.M, a.V, (char*)ws);
  if (c.total > ws_bytes) return TMX_ERR_SHAPE;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(&nucleus_hist_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kHalfBins * 4);
  static const hipError_t attr2 = hipFuncSetAttribute(
      reinterpret_cast<const void*>(&nucleus_eval_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kStageCap * 4);
  static const hipError_t attr3 = hipFuncSetAttribute(
      reinterpret_cast<const void*>(&nucleus_pick_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kStageCap * 4);
  if (attr != hipSuccess || attr2 != hipSuccess || attr3 != hipSuccess) return TMX_ERR_LAUNCH;
  a.mode = TMX_SAMPLE_TOP_P;
  a.sort_keys = c.keys;
  // more than 64 rows: one pass over the head matrix in 256 x 256 blocks instead of one per 64 rows
  int rc = (a.M > 64 && head_wide_ok(a)) ? head_wide_logits(st, a) : head_logits(st, a);
  if (rc != TMX_OK) return rc;
  NucleusArgs n = {};
  n.keys = c.keys; n.ent = c.ent; n.tot = c.tot; n.pbest = c.pbest;
  n.ns = nucleus_slices(a.M);
  n.M = a.M; n.V = a.V;
  n.k = (top_k > 0 && top_k < a.V) ? top_k : a.V;
  n.top_p = top_p;
  n.temperature = a.temperature;
  n.k0 = a.k0; n.k1 = a.k1;
  n.step = a.step;
  n.part_f = a.part_f; n.nwg = a.nwg;
  n.token_buffer = a.token_buffer; n.logprobs = a.logprobs; n.done = a.done;
  n.eos = a.eos; n.n_eos = a.n_eos; n.buf_len = a.buf_len;
  hipLaunchKernelGGL(nucleus_hist_kernel, dim3(2, a.M), dim3(kNT), kHalfBins * 4, st, n);
  if ((rc = check_launch()) != TMX_OK) return rc;
  hipLaunchKernelGGL(nucleus_eval_kernel, dim3(n.ns, a.M), dim3(kNT), kStageCap * 4, st, n);
  if ((rc = check_launch()) != TMX_OK) return rc;
  hipLaunchKernelGGL(nucleus_pick_kernel, dim3(a.M), dim3(kNT), kStageCap * 4, st, n);
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
