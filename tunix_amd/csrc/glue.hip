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
#include "tmx_kernels.h"

namespace tmx {

// delta for output column n of row m: bf16(bf16(sum_r t[r] * B[r][n]) * ls)
__device__ __forceinline__ float lora_delta(const uint16_t* __restrict__ t_row,
                                            const uint16_t* __restrict__ b, int ldb, int n, int r,
                                            float ls) {
  float d = 0.f;
  for (int rr = 0; rr < r; ++rr) d = fmaf(bf2f(t_row[rr]), bf2f(b[(size_t)rr * ldb + n]), d);
  return rbf(rbf(d) * ls);
}


// One workgroup per row: h = bf16(bf16(y + delta) + residual); xn = RMSNorm(h).
template <int EPT>  // elements per thread, D <= 256 * EPT
__global__ __launch_bounds__(256) void row_norm_kernel(RowNormArgs a) {
  __shared__ float smem[8];
  const int m = blockIdx.x;
  float v[EPT];
  float ss = 0.f;
  const uint16_t* src = nullptr;
  if (a.embed) {
    const int tok = a.token_buffer[(size_t)m * a.buf_len + *a.step];
    src = a.embed + (size_t)tok * a.D;
  }
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int n = e * 256 + threadIdx.x;
    float x = 0.f;
    if (n < a.D) {
      if (src) {
        x = bf2f(src[n]);
      } else {
        x = bf2f(a.y[(size_t)m * a.D + n]);
        if (a.t) x = rbf(x + lora_delta(a.t + (size_t)m * a.ldt, a.lora_b, a.D, n, a.r, a.ls));
        if (a.residual) x = rbf(x + bf2f(a.residual[(size_t)m * a.D + n]));
      }
      if (a.x_out) a.x_out[(size_t)m * a.D + n] = f2bf(x);
    }
    v[e] = x;
    ss += x * x;
  }
  if (!a.norm_w) return;
  ss = block_sum<4>(ss, smem);
  const float rms = sqrtf(ss / (float)a.D + a.eps);
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int n = e * 256 + threadIdx.x;
    if (n < a.D) {
      const float w = bf2f(a.norm_w[n]);
      float o;
      if (a.family == TMX_FAMILY_LLAMA3) o = rbf(w * v[e]) / rms;
      else o = w * (v[e] / rms);
      a.xn_out[(size_t)m * a.D + n] = f2bf(o);
    }
  }
}

int row_norm(hipStream_t st, const RowNormArgs& a, int M) {
  if (a.D <= 0 || a.D > 256 * 32) return TMX_ERR_SHAPE;
  const int ept = (a.D + 255) / 256;
  if (ept <= 1) hipLaunchKernelGGL(row_norm_kernel<1>, dim3(M), dim3(256), 0, st, a);
  else if (ept <= 4) hipLaunchKernelGGL(row_norm_kernel<4>, dim3(M), dim3(256), 0, st, a);
  else if (ept <= 8) hipLaunchKernelGGL(row_norm_kernel<8>, dim3(M), dim3(256), 0, st, a);
  else if (ept <= 16) hipLaunchKernelGGL(row_norm_kernel<16>, dim3(M), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(row_norm_kernel<32>, dim3(M), dim3(256), 0, st, a);
  return check_launch();
}

// ---------------------------------------------------------------------------

// grid (N + 2 Kh, B), one wave per head vector; lane i owns elements i and i + H/2.
__global__ __launch_bounds__(64) void rope_kvwrite_kernel(RopeArgs a) {
  const int head = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  const int half = a.H >> 1;
  const int step = *a.step;
  const bool active = lane < half;
  const int ntot = (a.N + 2 * a.Kh) * a.H;
  const int kind = head < a.N ? 0 : (head < a.N + a.Kh ? 1 : 2);  // q, k, v
  const int col0 = head * a.H;
  float x1 = 0.f, x2 = 0.f;
  if (active) {
    const size_t base = (size_t)b * ntot + col0;
    x1 = bf2f(a.qkv[base + lane]);
    x2 = bf2f(a.qkv[base + lane + half]);
    if (a.t) {
      const uint16_t* trow = a.t + (size_t)b * a.ldt + kind * a.r;
      x1 = rbf(x1 + lora_delta(trow, a.lora_b, ntot, col0 + lane, a.r, a.ls));
      x2 = rbf(x2 + lora_delta(trow, a.lora_b, ntot, col0 + lane + half, a.r, a.ls));
    }
  }
  const int slot = step % a.C;
  if (kind == 2) {
    if (active) {
      uint16_t* dst = a.vcache + (((size_t)b * a.C + slot) * a.Kh + (head - a.N - a.Kh)) * a.H;
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
  float o1 = 0.f, o2 = 0.f;
  if (active) {
    const float pos = (float)a.positions[(size_t)b * a.buf_len + step];
    const float frac = 2.f * (float)lane / (float)a.H;
    const float timescale = powf(a.theta, frac);
    const float ang = pos / timescale;
    float sn = sinf(ang), cs = cosf(ang);
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
    else dst = a.kcache + (((size_t)b * a.C + slot) * a.Kh + (head - a.N)) * a.H;
    dst[lane] = f2bf(o1);
    dst[lane + half] = f2bf(o2);
  }
}

int rope_kvwrite(hipStream_t st, const RopeArgs& a, int B) {
  if (a.H > 128 || a.H % 2) return TMX_ERR_SHAPE;
  hipLaunchKernelGGL(rope_kvwrite_kernel, dim3(a.N + 2 * a.Kh, B), dim3(64), 0, st, a);
  return check_launch();
}

// ---------------------------------------------------------------------------

__global__ __launch_bounds__(256) void swiglu_kernel(SwigluArgs a) {
  const int f = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
  if (f >= a.F) return;
  float g = bf2f(a.gu[(size_t)m * 2 * a.F + f]);
  float u = bf2f(a.gu[(size_t)m * 2 * a.F + a.F + f]);
  if (a.t) {
    const uint16_t* trow = a.t + (size_t)m * a.ldt;
    g = rbf(g + lora_delta(trow, a.lora_b, 2 * a.F, f, a.r, a.ls));
    u = rbf(u + lora_delta(trow + a.r, a.lora_b, 2 * a.F, a.F + f, a.r, a.ls));
  }
  const float sg = rbf(1.f / (1.f + expf(-g)));
  a.act[(size_t)m * a.F + f] = f2bf(rbf(g * sg) * u);
}

int swiglu(hipStream_t st, const SwigluArgs& a, int M) {
  hipLaunchKernelGGL(swiglu_kernel, dim3((a.F + 255) / 256, M), dim3(256), 0, st, a);
  return check_launch();
}

// step += 1 (one thread); keeps the step counter on the device so that a captured
// graph of one decode step can be replayed without host-side parameters.
__global__ void advance_step_kernel(int32_t* step) { *step += 1; }

int advance_step(hipStream_t st, int32_t* step) {
  hipLaunchKernelGGL(advance_step_kernel, dim3(1), dim3(1), 0, st, step);
  return check_launch();
}

}  // namespace tmx

using namespace tmx;

extern "C" int tmx_rmsnorm(void* stream, const void* x, const void* w, void* y, int M, int D, float eps,
                           int family) {
  if (!x || !w || !y) return TMX_ERR_ARG;
  if (M <= 0) return TMX_ERR_SHAPE;
  RowNormArgs a = {};
  a.y = (const uint16_t*)x;
  a.norm_w = (const uint16_t*)w;
  a.xn_out = (uint16_t*)y;
  a.D = D;
  a.eps = eps;
  a.family = family;
  return row_norm((hipStream_t)stream, a, M);
}

extern "C" int tmx_lora_residual_rmsnorm(void* stream, const void* y, const void* t, int ldt,
                                         const void* lora_b, int r, float lora_scale,
                                         const void* residual, void* x_out, const void* norm_w,
                                         void* xn_out, int M, int D, float eps, int family) {
  if (!y || (t && !lora_b) || (norm_w && !xn_out)) return TMX_ERR_ARG;
  if (M <= 0) return TMX_ERR_SHAPE;
  RowNormArgs a = {};
  a.y = (const uint16_t*)y;
  a.t = (const uint16_t*)t;
  a.ldt = ldt;
  a.lora_b = (const uint16_t*)lora_b;
  a.r = r;
  a.ls = lora_scale;
  a.residual = (const uint16_t*)residual;
  a.x_out = (uint16_t*)x_out;
  a.norm_w = (const uint16_t*)norm_w;
  a.xn_out = (uint16_t*)xn_out;
  a.D = D;
  a.eps = eps;
  a.family = family;
  return row_norm((hipStream_t)stream, a, M);
}

extern "C" int tmx_rope_kv_write(void* stream, const void* qkv, const void* t, int ldt,
                                 const void* lora_b, int r, float lora_scale, const void* q_norm_w,
                                 const void* k_norm_w, const int32_t* positions, const int32_t* step,
                                 int buf_len, void* q_out, void* kcache, void* vcache, int B, int N,
                                 int Kh, int H, int C, float theta, float eps, int family) {
  if (!qkv || !positions || !step || !q_out || !kcache || !vcache || (t && !lora_b)) return TMX_ERR_ARG;
  if (B <= 0 || N <= 0 || Kh <= 0 || C <= 0) return TMX_ERR_SHAPE;
  RopeArgs a = {};
  a.qkv = (const uint16_t*)qkv;
  a.t = (const uint16_t*)t;
  a.ldt = ldt;
  a.lora_b = (const uint16_t*)lora_b;
  a.r = r;
  a.ls = lora_scale;
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

extern "C" int tmx_swiglu(void* stream, const void* gate_up, const void* t, int ldt, const void* lora_b,
                          int r, float lora_scale, void* act, int M, int F) {
  if (!gate_up || !act || (t && !lora_b)) return TMX_ERR_ARG;
  if (M <= 0 || F <= 0) return TMX_ERR_SHAPE;
  SwigluArgs a = {};
  a.gu = (const uint16_t*)gate_up;
  a.t = (const uint16_t*)t;
  a.ldt = ldt;
  a.lora_b = (const uint16_t*)lora_b;
  a.r = r;
  a.ls = lora_scale;
  a.act = (uint16_t*)act;
  a.F = F;
  return swiglu((hipStream_t)stream, a, M);
}
