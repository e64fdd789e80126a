// Row-wise kernels between the matrix products of one decode step: embedding
// gather, RMSNorm, residual adds, RoPE + KV-cache write, SwiGLU.  Each one also
// applies the LoRA "B" half of the projection that produced its input
// (delta = bf16(bf16(t . B) * alpha/r)), so the big GEMM launches stay pure.
//
// Reference arithmetic (rounding points reproduced):
//   Embedder.encode        tunix/models/llama3/model.py:238-242, qwen3/model.py:418-423
//   RMSNorm                llama3/model.py:290-297 (w*x in bf16, then / rms);
//                          qwen3/model.py:478-484 (all f32, one cast)
//   apply_rope             llama3/model.py:249-270 (f32 throughout; theta fixed at 1e6 by
//                          the caller :356-365); qwen3/model.py:432-453 (sin/cos cast to
//                          bf16 first)
//   KV write               llama3/model.py:367-377, qwen3/model.py:586-597 (slot = end_index)
//   residual wiring        llama3/model.py:546-564, qwen3/model.py:1268-1289
//   SwiGLU                 llama3/model.py:489-496, qwen3/model.py:1199-1208
#include "tmx_router.h"

namespace tmx {

__device__ __forceinline__ void unpack8(const uint4& v, float* o) {
  o[0] = bf_lo(v.x); o[1] = bf_hi(v.x); o[2] = bf_lo(v.y); o[3] = bf_hi(v.y);
  o[4] = bf_lo(v.z); o[5] = bf_hi(v.z); o[6] = bf_lo(v.w); o[7] = bf_hi(v.w);
}
__device__ __forceinline__ uint4 pack8(const float* o) {
  uint4 v;
  v.x = pack_bf2(o[0], o[1]); v.y = pack_bf2(o[2], o[3]);
  v.z = pack_bf2(o[4], o[5]); v.w = pack_bf2(o[6], o[7]);
  return v;
}

// Sums NS K-slice planes of 8 adjacent f32 values; all 2 * NS loads are issued before the
// first add so that the planes' memory latencies overlap.  Planes are added in ascending
// order whatever NS is, so every code path rounds identically.
template <int NS>
__device__ __forceinline__ void sum_planes8(const float* p, size_t stride, float* o) {
  float4 a[NS], b[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const float4* q = reinterpret_cast<const float4*>(p + (size_t)s * stride);
    a[s] = q[0];
    b[s] = q[1];
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = 0.f;
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    o[0] += a[s].x; o[1] += a[s].y; o[2] += a[s].z; o[3] += a[s].w;
    o[4] += b[s].x; o[5] += b[s].y; o[6] += b[s].z; o[7] += b[s].w;
  }
}
template <int NS>
__device__ __forceinline__ float sum_planes1(const float* p, size_t stride) {
  float v[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) v[s] = p[(size_t)s * stride];
  float t = 0.f;
#pragma unroll
  for (int s = 0; s < NS; ++s) t += v[s];
  return t;
}
__device__ __forceinline__ float sum_planes1_dyn(const float* p, size_t stride, int ns) {
  switch (ns) {
    case 1: return sum_planes1<1>(p, stride);
    case 2: return sum_planes1<2>(p, stride);
    case 4: return sum_planes1<4>(p, stride);
    case 8: return sum_planes1<8>(p, stride);
    case 16: return sum_planes1<16>(p, stride);
    case 32: return sum_planes1<32>(p, stride);
    default: {
      // any other count: batches of 8 loads with clamped (in-bounds) plane indices
      float t = 0.f;
      for (int s0 = 0; s0 < ns; s0 += 8) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = p[(size_t)(s0 + i < ns ? s0 + i : ns - 1) * stride];
#pragma unroll
        for (int i = 0; i < 8; ++i) t += (s0 + i < ns) ? v[i] : 0.f;
      }
      return t;
    }
  }
}

// t_s[rr] = bf16(sum_s t_part[s][m][col0 + rr]) for rr < n, by the first n threads.
__device__ __forceinline__ void stage_t(float* t_s, const LoraIn& l, int m, int M, int col0, int n) {
  if ((int)threadIdx.x < n)
    t_s[threadIdx.x] = rbf(sum_planes1_dyn(l.t_part + (size_t)m * l.ldt + col0 + threadIdx.x,
                                           (size_t)M * l.ldt, l.nsplit));
}

// The same for a whole workgroup: every (plane, column) value is fetched by its own thread
// (one memory latency instead of one per batch of planes), parked in `stage`
// [nsplit][n] floats, then the first n threads add their column's planes in ascending order.
// Ends with a barrier; needs n * nsplit <= the capacity of `stage`.
__device__ __forceinline__ void stage_t_block(float* t_s, float* stage, const LoraIn& l, int m, int M, int col0,
                                              int n) {
  const int total = n * l.nsplit;
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    const int sp = i / n, c = i - sp * n;
    stage[i] = l.t_part[((size_t)sp * M + m) * l.ldt + col0 + c];
  }
  __syncthreads();
  if ((int)threadIdx.x < n) {
    float t = 0.f;
    for (int sp = 0; sp < l.nsplit; ++sp) t += stage[sp * n + threadIdx.x];
    t_s[threadIdx.x] = rbf(t);
  }
  __syncthreads();
}

// 8 adjacent outputs n0..n0+7 of one row: base = bf16(sum of the split planes) or the bf16 tensor.
__device__ __forceinline__ void load_base8(const uint16_t* y_bf16, const float* y_part, int nsplit, int m,
                                           int M, int N, int n0, float* o) {
  if (y_bf16) {
    unpack8(*reinterpret_cast<const uint4*>(y_bf16 + (size_t)m * N + n0), o);
    return;
  }
  const float* p = y_part + (size_t)m * N + n0;
  const size_t stride = (size_t)M * N;
  switch (nsplit) {
    case 1: sum_planes8<1>(p, stride, o); break;
    case 2: sum_planes8<2>(p, stride, o); break;
    case 4: sum_planes8<4>(p, stride, o); break;
    case 8: sum_planes8<8>(p, stride, o); break;
    case 16: sum_planes8<16>(p, stride, o); break;
    default: {
      // any other count: up to 16 planes in flight at once (clamped, in-bounds plane indices),
      // added in ascending order like the fixed counts
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = 0.f;
      for (int s0 = 0; s0 < nsplit; s0 += 16) {
        float4 a[16], b[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float4* q = reinterpret_cast<const float4*>(p + (size_t)(s0 + i < nsplit ? s0 + i : nsplit - 1) * stride);
          a[i] = q[0];
          b[i] = q[1];
        }
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (s0 + i < nsplit) {
            o[0] += a[i].x; o[1] += a[i].y; o[2] += a[i].z; o[3] += a[i].w;
            o[4] += b[i].x; o[5] += b[i].y; o[6] += b[i].z; o[7] += b[i].w;
          }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = rbf(o[e]);
}

// o[e] = bf16(o[e] + bf16(bf16(sum_r t_s[r] B[r][n0 + e]) * ls))
__device__ __forceinline__ void add_lora8(float* o, const float* t_s, const uint16_t* b, int ldb, int n0,
                                          int r, float ls) {
  float d[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
  for (int rr = 0; rr < r; ++rr) {
    float w[8];
    unpack8(*reinterpret_cast<const uint4*>(b + (size_t)rr * ldb + n0), w);
    const float t = t_s[rr];
#pragma unroll
    for (int e = 0; e < 8; ++e) d[e] = fmaf(t, w[e], d[e]);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = rbf(o[e] + rbf(rbf(d[e]) * ls));
}

// One workgroup per row: h = bf16(bf16(y + delta) + residual); xn = RMSNorm(h).
// In embedding mode it also fills this step's RoPE sin/cos table row.
template <int CPT>  // 8-element chunks per thread, D <= 4096 * CPT
__global__ __launch_bounds__(512) void row_norm_kernel(RowNormArgs a) {
  extern __shared__ __align__(16) float route_sm[];  // moe_router_lds_floats(D, E) floats when the row is routed here, else none
  __shared__ float smem[8];
  __shared__ float t_s[TMX_MAX_RPAD];
  __shared__ float t_stage[TMX_MAX_LORA_SPLITS * 64];
  const int m = blockIdx.x, M = gridDim.x;
  float v[CPT][8];
  float ss = 0.f;
  const uint16_t* src = nullptr;
  if (a.embed) {
    const int tpp = a.tpp > 0 ? a.tpp : 1;
    // column and id are clamped into range like the reference's gathers (jnp indexing clamps), so a
    // caller that oversteps the buffer or feeds an id outside the vocabulary reads a valid row
    const int seq = m / tpp, step = min(*a.step + m % tpp, a.buf_len - 1);
    int tok = a.token_buffer[(size_t)seq * a.buf_len + step];
    if (a.vocab > 0) tok = min(max(tok, 0), a.vocab - 1);
    src = a.embed + (size_t)tok * a.D;
    if (a.rope_tab && (int)threadIdx.x < a.half) {
      const float pos = (float)a.positions[(size_t)seq * a.buf_len + step];
      const float frac = 2.f * (float)threadIdx.x / (float)(2 * a.half);
      const float ang = pos / powf(a.theta, frac);
      a.rope_tab[((size_t)m * a.half + threadIdx.x) * 2] = sinf(ang);
      a.rope_tab[((size_t)m * a.half + threadIdx.x) * 2 + 1] = cosf(ang);
    }
  }
  const int nchunks = a.D >> 3;
  // Everything that does not depend on the row's own sums is requested first and in one go, so
  // that the memory latencies overlap: the LoRA planes' values (one per thread), the rows of B
  // for this thread's columns (16 bytes each; up to 16 rows are kept in registers when every
  // thread owns a single chunk) and the norm weights.  The in-order load counter makes the wait
  // for the planes below cover them all.
  constexpr int kBR = CPT == 1 ? 16 : 1;
  const bool lora = !src && a.lora.t_part;
  const bool b_early = CPT == 1 && lora && a.lora.r <= kBR && (int)threadIdx.x < nchunks;
  uint4 brow[kBR];
  if (b_early) {
#pragma unroll
    for (int rr = 0; rr < kBR; ++rr)
      brow[rr] = *reinterpret_cast<const uint4*>(a.lora.b + (size_t)(rr < a.lora.r ? rr : 0) * a.D + threadIdx.x * 8);
  }
  uint4 nw4[CPT];
  if (a.norm_w) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = threadIdx.x + 512 * i;
      nw4[i] = *reinterpret_cast<const uint4*>(a.norm_w + (c < nchunks ? c : 0) * 8);
    }
  }
  const int t_total = lora ? a.lora.r * a.lora.nsplit : 0;
  const bool t_one = t_total <= 512;  // one value per thread
  float t_val = 0.f;
  if (t_one && (int)threadIdx.x < t_total) {
    const int sp = threadIdx.x / a.lora.r, c = threadIdx.x - sp * a.lora.r;
    t_val = a.lora.t_part[((size_t)sp * M + m) * a.lora.ldt + c];
  }
  // the row's own loads (planes, residual)
  float res8[CPT][8];
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int c = threadIdx.x + 512 * i;
#pragma unroll
    for (int e = 0; e < 8; ++e) { v[i][e] = 0.f; res8[i][e] = 0.f; }
    if (c < nchunks) {
      const int n0 = c * 8;
      if (src) {
        unpack8(*reinterpret_cast<const uint4*>(src + n0), v[i]);
      } else if (a.moe_y) {
        // bf16(sum over the token's experts of weight * expert output), f32 accumulation
        // (eight experts' rows and weights are requested together: one memory round trip per eight, in the
        // experts' order)
        for (int j0 = 0; j0 < a.top_k; j0 += 8) {
          uint4 yr[8];
          float wr[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const size_t p = (size_t)m * a.top_k + min(j0 + u, a.top_k - 1);
            yr[u] = *reinterpret_cast<const uint4*>(a.moe_y + p * a.D + n0);
            wr[u] = j0 + u < a.top_k ? a.moe_w[p] : 0.f;
          }
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            if (j0 + u < a.top_k) {
              float y8[8];
              unpack8(yr[u], y8);
#pragma unroll
              for (int e = 0; e < 8; ++e) v[i][e] = fmaf(wr[u], y8[e], v[i][e]);
            }
          }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] = rbf(v[i][e]);
        if (a.residual) unpack8(*reinterpret_cast<const uint4*>(a.residual + (size_t)m * a.D + n0), res8[i]);
      } else {
        // the residual (and the LoRA delta, when the projection made it) is requested before the planes are waited for
        uint4 r4 = {0, 0, 0, 0}, d4 = {0, 0, 0, 0};
        if (a.residual) r4 = *reinterpret_cast<const uint4*>(a.residual + (size_t)m * a.D + n0);
        if (a.delta) d4 = *reinterpret_cast<const uint4*>(a.delta + (size_t)m * a.D + n0);
        load_base8(a.y_bf16, a.y_part, a.nsplit, m, M, a.D, n0, v[i]);
        if (a.residual) unpack8(r4, res8[i]);
        if (a.delta) {  // bf16(base + delta), delta = bf16(bf16(t . B) * ls)
          float d8[8];
          unpack8(d4, d8);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[i][e] = rbf(v[i][e] + d8[e]);
        }
      }
    }
  }
  if (lora) {
    if (t_one) {
      // t_s[c] = bf16(sum of the planes' values of column c), planes in ascending order
      if ((int)threadIdx.x < t_total) t_stage[threadIdx.x] = t_val;
      __syncthreads();
      if ((int)threadIdx.x < a.lora.r) {
        float t = 0.f;
        for (int sp = 0; sp < a.lora.nsplit; ++sp) t += t_stage[sp * a.lora.r + threadIdx.x];
        t_s[threadIdx.x] = rbf(t);
      }
      __syncthreads();
    } else if (a.lora.r * a.lora.nsplit <= TMX_MAX_LORA_SPLITS * 64) {
      stage_t_block(t_s, t_stage, a.lora, m, M, 0, a.lora.r);
    } else {
      stage_t(t_s, a.lora, m, M, 0, a.lora.r);
      __syncthreads();
    }
  }
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int c = threadIdx.x + 512 * i;
    if (c < nchunks) {
      const int n0 = c * 8;
      if (!src) {
        if (b_early) {
          float d[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int rr = 0; rr < kBR; ++rr) {
            float wv[8];
            unpack8(brow[rr], wv);
            const float t = rr < a.lora.r ? t_s[rr] : 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) d[e] = fmaf(t, wv[e], d[e]);
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) v[i][e] = rbf(v[i][e] + rbf(rbf(d[e]) * a.lora.ls));
        } else if (lora) {
          add_lora8(v[i], t_s, a.lora.b, a.D, n0, a.lora.r, a.lora.ls);
        }
        if (a.residual) {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[i][e] = rbf(v[i][e] + res8[i][e]);
        }
      }
      if (a.x_out) *reinterpret_cast<uint4*>(a.x_out + (size_t)m * a.D + n0) = pack8(v[i]);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += v[i][e] * v[i][e];
    }
  }
  if (!a.norm_w) return;
  ss = block_sum<8>(ss, smem);
  const float rms = sqrtf(ss / (float)a.D + a.eps);
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int c = threadIdx.x + 512 * i;
    if (c < nchunks) {
      const int n0 = c * 8;
      float w[8], o[8];
      unpack8(nw4[i], w);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (a.family == TMX_FAMILY_LLAMA3) o[e] = rbf(w[e] * v[i][e]) / rms;
        else o[e] = w[e] * (v[i][e] / rms);
      }
      *reinterpret_cast<uint4*>(a.xn_out + (size_t)m * a.D + n0) = pack8(o);
      if (a.router.w) {
#pragma unroll
        for (int e = 0; e < 8; ++e) route_sm[n0 + e] = rbf(o[e]);
      }
    }
  }
  if (a.router.w) {
    // MoE layer: the token is routed here, from the normed row this workgroup just made (no router launch, no
    // reload of xn)
    __syncthreads();
    moe_route_token(a.router, route_sm, m);
  }
}

int row_norm(hipStream_t st, const RowNormArgs& a, int M) {
  if (a.D <= 0 || a.D % 8 || a.D > 4096 * 4) return TMX_ERR_SHAPE;
  if (a.lora.t_part && a.lora.r > TMX_MAX_RPAD) return TMX_ERR_SHAPE;
  if (a.rope_tab && a.half > 256) return TMX_ERR_SHAPE;
  size_t lds = 0;
  if (a.router.w) {
    const RouterArgs& r = a.router;
    if (!a.norm_w || !r.expert_of || !r.weight_of || r.D != a.D) return TMX_ERR_ARG;
    if (r.E <= 0 || r.E % 8 || r.top_k <= 0 || r.top_k > 64 || r.top_k > r.E) return TMX_ERR_SHAPE;
    lds = moe_router_lds_floats(a.D, r.E) * sizeof(float);
    if (lds > 60000) return TMX_ERR_SHAPE;
  }
  const int cpt = (a.D / 8 + 511) / 512;
  if (cpt <= 1) hipLaunchKernelGGL(row_norm_kernel<1>, dim3(M), dim3(512), lds, st, a);
  else if (cpt <= 2) hipLaunchKernelGGL(row_norm_kernel<2>, dim3(M), dim3(512), lds, st, a);
  else hipLaunchKernelGGL(row_norm_kernel<4>, dim3(M), dim3(512), lds, st, a);
  return check_launch();
}

// ---------------------------------------------------------------------------
// grid (N + 2 Kh, B), one wave per head vector; lane i owns elements i and i + H/2.
__global__ __launch_bounds__(64) void rope_kvwrite_kernel(RopeArgs a) {
  __shared__ float t_s[64];
  const int head = blockIdx.x, b = blockIdx.y, B = gridDim.y, lane = threadIdx.x;
  const int half = a.H >> 1;
  const int tpp = a.tpp > 0 ? a.tpp : 1;
  const int seq = b / tpp, step = min(*a.step + b % tpp, a.buf_len - 1);  // b: row of this pass (column clamped into the buffer)
  const bool active = lane < half;
  const int ntot = (a.N + 2 * a.Kh) * a.H;
  const int kind = head < a.N ? 0 : (head < a.N + a.Kh ? 1 : 2);  // q, k, v
  const int col0 = head * a.H;
  if (a.lora.t_part) {
    stage_t(t_s, a.lora, b, B, kind * a.lora.r, a.lora.r);
    __syncthreads();
  }
  float x1 = 0.f, x2 = 0.f;
  if (active) {
    const int c1 = col0 + lane, c2 = c1 + half;
    if (a.qkv_bf16) {
      x1 = bf2f(a.qkv_bf16[(size_t)b * ntot + c1]);
      x2 = bf2f(a.qkv_bf16[(size_t)b * ntot + c2]);
    } else {
      x1 = rbf(sum_planes1_dyn(a.qkv_part + (size_t)b * ntot + c1, (size_t)B * ntot, a.nsplit));
      x2 = rbf(sum_planes1_dyn(a.qkv_part + (size_t)b * ntot + c2, (size_t)B * ntot, a.nsplit));
    }
    if (a.lora.t_part) {
      float d1 = 0.f, d2 = 0.f;
#pragma unroll 8
      for (int rr = 0; rr < a.lora.r; ++rr) {
        d1 = fmaf(t_s[rr], bf2f(a.lora.b[(size_t)rr * ntot + c1]), d1);
        d2 = fmaf(t_s[rr], bf2f(a.lora.b[(size_t)rr * ntot + c2]), d2);
      }
      x1 = rbf(x1 + rbf(rbf(d1) * a.lora.ls));
      x2 = rbf(x2 + rbf(rbf(d2) * a.lora.ls));
    }
  }
  const int slot = step % a.C;
  if (kind == 2) {
    if (active) {
      uint16_t* dst = a.vcache + (((size_t)seq * a.C + slot) * a.Kh + (head - a.N - a.Kh)) * a.H;
      dst[lane] = f2bf(x1);
      dst[lane + half] = f2bf(x2);
    }
    return;
  }
  const uint16_t* nw = kind == 0 ? a.q_norm_w : a.k_norm_w;
  if (nw) {  // Qwen3 per-head RMSNorm, f32 with one cast
    const float ss = wave_sum(x1 * x1 + x2 * x2);
    const float rms = sqrtf(ss / (float)a.H + a.eps);
    if (active) {
      x1 = rbf(bf2f(nw[lane]) * (x1 / rms));
      x2 = rbf(bf2f(nw[lane + half]) * (x2 / rms));
    }
  }
  if (active) {
    float sn, cs;
    if (a.rope_tab) {
      sn = a.rope_tab[((size_t)b * half + lane) * 2];
      cs = a.rope_tab[((size_t)b * half + lane) * 2 + 1];
    } else {
      const float pos = (float)a.positions[(size_t)seq * a.buf_len + step];
      const float ang = pos / powf(a.theta, 2.f * (float)lane / (float)a.H);
      sn = sinf(ang);
      cs = cosf(ang);
    }
    float o1, o2;
    if (a.family == TMX_FAMILY_LLAMA3) {
      o1 = x1 * cs - x2 * sn;
      o2 = x2 * cs + x1 * sn;
    } else {
      sn = rbf(sn);
      cs = rbf(cs);
      o1 = rbf(x1 * cs) - rbf(x2 * sn);
      o2 = rbf(x2 * cs) + rbf(x1 * sn);
    }
    uint16_t* dst;
    if (kind == 0) dst = a.q_out + (size_t)b * a.N * a.H + head * a.H;
    else dst = a.kcache + (((size_t)seq * a.C + slot) * a.Kh + (head - a.N)) * a.H;
    dst[lane] = f2bf(o1);
    dst[lane + half] = f2bf(o2);
  }
}

int rope_kvwrite(hipStream_t st, const RopeArgs& a, int B) {
  if (a.H > 128 || a.H % 2) return TMX_ERR_SHAPE;
  if (a.lora.t_part && a.lora.r > 64) return TMX_ERR_SHAPE;
  hipLaunchKernelGGL(rope_kvwrite_kernel, dim3(a.N + 2 * a.Kh, B), dim3(64), 0, st, a);
  return check_launch();
}

// ---------------------------------------------------------------------------
// grid (ceil(F / 2048), M): a thread owns 8 adjacent hidden units of one row.
__global__ __launch_bounds__(256) void swiglu_kernel(SwigluArgs a) {
  __shared__ float t_s[TMX_MAX_RPAD];
  const int m = blockIdx.y, M = gridDim.y;
  const int f0 = (blockIdx.x * 256 + threadIdx.x) * 8;
  const bool mine = f0 < a.F;
  float g[8], u[8], o[8];
  if (mine) {
    load_base8(a.gu_bf16, a.gu_part, a.nsplit, m, M, 2 * a.F, f0, g);
    load_base8(a.gu_bf16, a.gu_part, a.nsplit, m, M, 2 * a.F, a.F + f0, u);
  }
  if (a.lora.t_part) {
    stage_t(t_s, a.lora, m, M, 0, 2 * a.lora.r);
    __syncthreads();
  }
  if (!mine) return;
  if (a.lora.t_part) {
    add_lora8(g, t_s, a.lora.b, 2 * a.F, f0, a.lora.r, a.lora.ls);
    add_lora8(u, t_s + a.lora.r, a.lora.b, 2 * a.F, a.F + f0, a.lora.r, a.lora.ls);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float sg = rbf(1.f / (1.f + expf(-g[e])));
    o[e] = rbf(g[e] * sg) * u[e];
  }
  *reinterpret_cast<uint4*>(a.act + (size_t)m * a.F + f0) = pack8(o);
}

// Many rows (cache fill): grid (ceil(F / 2048), ceil(M / 16)); a thread owns 8 adjacent hidden
// units of 16 rows.  Its columns of B (gate and up, rank <= 16) stay in registers for all 16 rows,
// packed as bf16 pairs along the rank, and the rank sum runs on the packed bf16 dot product
// (two products and the add per instruction; t is bf16 already, so the products are exact and
// only the f32 summation order differs from the one-row kernel).  bf16 input only.
constexpr int kSwigluRows = 16;
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t bf16_of(const uint4& v, int e) {
  const uint32_t w = e < 2 ? v.x : (e < 4 ? v.y : (e < 6 ? v.z : v.w));
  return (e & 1) ? (w >> 16) : (w & 0xFFFFu);
}
__global__ __launch_bounds__(256) void swiglu_rows_kernel(SwigluArgs a, int M) {
  __shared__ uint32_t t_s[kSwigluRows][16];  // [row][gate pairs 0..7 | up pairs 0..7]
  const int m0 = blockIdx.y * kSwigluRows;
  const int rows = M - m0 < kSwigluRows ? M - m0 : kSwigluRows;
  const int f0 = (blockIdx.x * 256 + threadIdx.x) * 8;
  const bool mine = f0 < a.F;
  const int r = a.lora.t_part ? a.lora.r : 0;
  uint32_t pg[8][8], pu[8][8];  // [rank pair][column]: (B[2p][c], B[2p + 1][c])
  if (mine && r) {
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const uint4 z = {0, 0, 0, 0};
      const uint16_t* b0 = a.lora.b + (size_t)(2 * p) * 2 * a.F + f0;
      const uint16_t* b1 = b0 + 2 * a.F;
      const uint4 g0 = 2 * p < r ? *reinterpret_cast<const uint4*>(b0) : z;
      const uint4 g1 = 2 * p + 1 < r ? *reinterpret_cast<const uint4*>(b1) : z;
      const uint4 u0 = 2 * p < r ? *reinterpret_cast<const uint4*>(b0 + a.F) : z;
      const uint4 u1 = 2 * p + 1 < r ? *reinterpret_cast<const uint4*>(b1 + a.F) : z;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        pg[p][e] = bf16_of(g0, e) | (bf16_of(g1, e) << 16);
        pu[p][e] = bf16_of(u0, e) | (bf16_of(u1, e) << 16);
      }
    }
  }
  // t pairs: bf16(sum of the planes' values) of columns x.A_gate | x.A_up, zero past the rank
  if (r) {
    const int row = threadIdx.x >> 4, c = threadIdx.x & 15, half = c >> 3, p = c & 7;
    float t0 = 0.f, t1 = 0.f;
    if (row < rows) {
      const float* q = a.lora.t_part + (size_t)(m0 + row) * a.lora.ldt + half * r + 2 * p;
      for (int sp = 0; sp < a.lora.nsplit; ++sp) {
        if (2 * p < r) t0 += q[(size_t)sp * M * a.lora.ldt];
        if (2 * p + 1 < r) t1 += q[(size_t)sp * M * a.lora.ldt + 1];
      }
    }
    t_s[row][c] = pack_bf2(t0, t1);
  }
  __syncthreads();
  if (!mine) return;
  for (int i = 0; i < rows; ++i) {
    const size_t m = m0 + i;
    float g[8], u[8], o[8];
    unpack8(*reinterpret_cast<const uint4*>(a.gu_bf16 + m * 2 * a.F + f0), g);
    unpack8(*reinterpret_cast<const uint4*>(a.gu_bf16 + m * 2 * a.F + a.F + f0), u);
    if (r) {
      float dg[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, du[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int p = 0; p < 8; ++p) {
        const bf16x2_t tg = __builtin_bit_cast(bf16x2_t, t_s[i][p]), tu = __builtin_bit_cast(bf16x2_t, t_s[i][8 + p]);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          dg[e] = __builtin_amdgcn_fdot2_f32_bf16(tg, __builtin_bit_cast(bf16x2_t, pg[p][e]), dg[e], false);
          du[e] = __builtin_amdgcn_fdot2_f32_bf16(tu, __builtin_bit_cast(bf16x2_t, pu[p][e]), du[e], false);
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        g[e] = rbf(g[e] + rbf(rbf(dg[e]) * a.lora.ls));
        u[e] = rbf(u[e] + rbf(rbf(du[e]) * a.lora.ls));
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float sg = rbf(1.f / (1.f + expf(-g[e])));
      o[e] = rbf(g[e] * sg) * u[e];
    }
    *reinterpret_cast<uint4*>(a.act + m * a.F + f0) = pack8(o);
  }
}

int swiglu(hipStream_t st, const SwigluArgs& a, int M) {
  if (a.F % 8 || (a.lora.t_part && 2 * a.lora.r > TMX_MAX_RPAD)) return TMX_ERR_SHAPE;
  if (M > 128 && a.gu_bf16 && (!a.lora.t_part || a.lora.r <= 16)) {
    hipLaunchKernelGGL(swiglu_rows_kernel, dim3((a.F + 2047) / 2048, (M + kSwigluRows - 1) / kSwigluRows), dim3(256),
                       0, st, a, M);
    return check_launch();
  }
  hipLaunchKernelGGL(swiglu_kernel, dim3((a.F + 2047) / 2048, M), dim3(256), 0, st, a);
  return check_launch();
}

// step += tokens per pass (one thread); keeps the step counter on the device so that a captured
// graph of one decode step can be replayed without host-side parameters.
__global__ void advance_step_kernel(int32_t* step, int by) { *step += by; }

int advance_step(hipStream_t st, int32_t* step, int by) {
  hipLaunchKernelGGL(advance_step_kernel, dim3(1), dim3(1), 0, st, step, by);
  return check_launch();
}

__global__ void zero_words_kernel(uint32_t* p, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0u;
}

int zero_words(hipStream_t st, uint32_t* p, int n) {
  hipLaunchKernelGGL(zero_words_kernel, dim3((n + 255) / 256), dim3(256), 0, st, p, n);
  return check_launch();
}

__global__ void empty_kernel() {}

int empty_launch(hipStream_t st) {
  hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, st);
  return check_launch();
}

}  // namespace tmx

using namespace tmx;

static LoraIn make_lora(const void* t_part, int ldt, int nsplit, const void* b, int r, float ls) {
  // nsplit: number of t planes
  LoraIn l = {};
  l.t_part = (const float*)t_part;
  l.ldt = ldt;
  l.nsplit = nsplit;
  l.b = (const uint16_t*)b;
  l.r = r;
  l.ls = ls;
  return l;
}

extern "C" int tmx_rmsnorm(void* stream, const void* x, const void* w, void* y, int M, int D, float eps,
                           int family) {
  if (!x || !w || !y) return TMX_ERR_ARG;
  if (M <= 0) return TMX_ERR_SHAPE;
  RowNormArgs a = {};
  a.y_bf16 = (const uint16_t*)x;
  a.norm_w = (const uint16_t*)w;
  a.xn_out = (uint16_t*)y;
  a.D = D;
  a.eps = eps;
  a.family = family;
  return row_norm((hipStream_t)stream, a, M);
}

extern "C" int tmx_lora_residual_rmsnorm(void* stream, const void* y_bf16, const float* y_part,
                                         int nsplit, const float* t_part, int t_nsplit, int ldt,
                                         const void* lora_b,
                                         int r, float lora_scale, const void* residual, void* x_out,
                                         const void* norm_w, void* xn_out, int M, int D, float eps,
                                         int family) {
  if ((!y_bf16 && !y_part) || (t_part && (!lora_b || t_nsplit < 1)) || (norm_w && !xn_out)) return TMX_ERR_ARG;
  if (M <= 0 || (!y_bf16 && nsplit < 1)) return TMX_ERR_SHAPE;
  RowNormArgs a = {};
  a.y_bf16 = (const uint16_t*)y_bf16;
  a.y_part = y_part;
  a.nsplit = nsplit;
  a.lora = make_lora(t_part, ldt, t_nsplit, lora_b, r, lora_scale);
  a.residual = (const uint16_t*)residual;
  a.x_out = (uint16_t*)x_out;
  a.norm_w = (const uint16_t*)norm_w;
  a.xn_out = (uint16_t*)xn_out;
  a.D = D;
  a.eps = eps;
  a.family = family;
  return row_norm((hipStream_t)stream, a, M);
}

extern "C" int tmx_rope_kv_write(void* stream, const void* qkv_bf16, const float* qkv_part, int nsplit,
                                 const float* t_part, int t_nsplit, int ldt, const void* lora_b, int r,
                                 float lora_scale, const void* q_norm_w, const void* k_norm_w,
                                 const int32_t* positions, const int32_t* step, int buf_len, void* q_out,
                                 void* kcache, void* vcache, int B, int N, int Kh, int H, int C,
                                 float theta, float eps, int family) {
  if ((!qkv_bf16 && !qkv_part) || !positions || !step || !q_out || !kcache || !vcache ||
      (t_part && (!lora_b || t_nsplit < 1)))
    return TMX_ERR_ARG;
  if (B <= 0 || N <= 0 || Kh <= 0 || C <= 0 || (!qkv_bf16 && nsplit < 1)) return TMX_ERR_SHAPE;
  RopeArgs a = {};
  a.qkv_bf16 = (const uint16_t*)qkv_bf16;
  a.qkv_part = qkv_part;
  a.nsplit = nsplit;
  a.lora = make_lora(t_part, ldt, t_nsplit, lora_b, r, lora_scale);
  a.q_norm_w = (const uint16_t*)q_norm_w;
  a.k_norm_w = (const uint16_t*)k_norm_w;
  a.positions = positions;
  a.step = step;
  a.buf_len = buf_len;
  a.q_out = (uint16_t*)q_out;
  a.kcache = (uint16_t*)kcache;
  a.vcache = (uint16_t*)vcache;
  a.N = N; a.Kh = Kh; a.H = H; a.C = C;
  a.theta = theta; a.eps = eps; a.family = family;
  return rope_kvwrite((hipStream_t)stream, a, B);
}

extern "C" int tmx_swiglu(void* stream, const void* gate_up_bf16, const float* gate_up_part, int nsplit,
                          const float* t_part, int t_nsplit, int ldt, const void* lora_b, int r,
                          float lora_scale,
                          void* act, int M, int F) {
  if ((!gate_up_bf16 && !gate_up_part) || !act || (t_part && (!lora_b || t_nsplit < 1))) return TMX_ERR_ARG;
  if (M <= 0 || F <= 0 || (!gate_up_bf16 && nsplit < 1)) return TMX_ERR_SHAPE;
  SwigluArgs a = {};
  a.gu_bf16 = (const uint16_t*)gate_up_bf16;
  a.gu_part = gate_up_part;
  a.nsplit = nsplit;
  a.lora = make_lora(t_part, ldt, t_nsplit, lora_b, r, lora_scale);
  a.act = (uint16_t*)act;
  a.F = F;
  return swiglu((hipStream_t)stream, a, M);
}
