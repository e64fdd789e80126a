// The decode step of the Sampler as one host function that enqueues every kernel
// of `n_steps` iterations on a stream; nothing here synchronises or allocates.
//
// Restates the body of the reference's lax.while_loop
// (tunix/generate/sampler.py:749-793 _sample_step + :520-599 _sample) around the
// model call (tunix/models/llama3/model.py:642-697, qwen3/model.py:1375-1442):
// the step counter, token buffer, positions, input mask, done flags and KV cache
// live in device memory exactly like _SamplingState (sampler.py:53-109), and the
// counter is advanced on the device, so the host never reads anything back
// between steps.
#include "tmx_kernels.h"

namespace tmx {

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct Workspace {
  uint16_t *x, *xn, *qkv, *q, *attn, *yo, *gu, *act, *t;
  float* attn_partial;
  void* head_partial;
  size_t total;
};

static Workspace carve(const tmx_model_desc* m, int B, int C, char* base) {
  Workspace w;
  size_t off = 0;
  auto take = [&](size_t bytes) { char* p = base ? base + off : nullptr; off += align256(bytes); return p; };
  const size_t D = m->embed_dim, NH = (size_t)m->num_heads * m->head_dim;
  const size_t QKV = NH + 2 * (size_t)m->num_kv_heads * m->head_dim, F = m->hidden_dim;
  w.x = (uint16_t*)take(B * D * 2);
  w.xn = (uint16_t*)take(B * D * 2);
  w.qkv = (uint16_t*)take(B * QKV * 2);
  w.q = (uint16_t*)take(B * NH * 2);
  w.attn = (uint16_t*)take(B * NH * 2);
  w.yo = (uint16_t*)take(B * D * 2);
  w.gu = (uint16_t*)take(B * 2 * F * 2);
  w.act = (uint16_t*)take(B * F * 2);
  w.t = (uint16_t*)take((size_t)B * TMX_MAX_RPAD * 2);
  w.attn_partial = (float*)take(attn_partial_bytes(B, m->num_heads, m->num_kv_heads, m->head_dim, C));
  w.head_partial = take(head_partial_bytes(B, m->vocab_size));
  w.total = off;
  return w;
}

static int check_linear(const tmx_qlinear_desc& l, int K, int N) {
  if (!l.qweight || !l.scales) return TMX_ERR_ARG;
  if (l.K != K || l.N != N) return TMX_ERR_SHAPE;
  if (l.lora_a_t && (!l.lora_b || l.rank <= 0 || l.r_pad > TMX_MAX_RPAD)) return TMX_ERR_ARG;
  return TMX_OK;
}

}  // namespace tmx

using namespace tmx;

extern "C" size_t tmx_decode_workspace_bytes(const tmx_model_desc* m, int batch, int cache_size) {
  if (!m || batch <= 0) return 0;
  return carve(m, batch, cache_size, nullptr).total;
}

extern "C" int tmx_decode_steps(const tmx_model_desc* m, const tmx_decode_state* s, void* stream,
                                int n_steps, int sample) {
  if (!m || !s || !m->layers || !m->embed || !m->final_norm_w || !m->head) return TMX_ERR_ARG;
  if (!s->token_buffer || !s->positions || !s->input_mask || !s->done || !s->step || !s->kv_cache ||
      !s->workspace)
    return TMX_ERR_ARG;
  if (m->num_experts > 0) return TMX_ERR_UNSUPPORTED;
  const int B = s->batch, C = s->cache_size, L = s->buf_len;
  if (B <= 0 || B > 128 || C <= 0 || L <= 0 || L > C) return TMX_ERR_SHAPE;
  if (sample && s->sampling_mode == TMX_SAMPLE_TOP_P && (s->top_p < 1.0f || s->top_k > 0))
    return TMX_ERR_UNSUPPORTED;
  const int D = m->embed_dim, N = m->num_heads, Kh = m->num_kv_heads, H = m->head_dim;
  const int F = m->hidden_dim, NH = N * H, QKV = (N + 2 * Kh) * H;
  if (carve(m, B, C, nullptr).total > s->workspace_bytes) return TMX_ERR_SHAPE;
  for (int i = 0; i < m->num_layers; ++i) {
    const tmx_layer_desc& l = m->layers[i];
    if (!l.norm1_w || !l.norm2_w) return TMX_ERR_ARG;
    int rc;
    if ((rc = check_linear(l.qkv, D, QKV)) || (rc = check_linear(l.o, NH, D)) ||
        (rc = check_linear(l.gate_up, D, 2 * F)) || (rc = check_linear(l.down, F, D)))
      return rc;
  }
  hipStream_t st = (hipStream_t)stream;
  const Workspace w = carve(m, B, C, (char*)s->workspace);
  const size_t kv_elems = (size_t)B * C * Kh * H;
  const float theta = m->family == TMX_FAMILY_LLAMA3 ? 1000000.0f : m->rope_theta;
  int rc;
#define TMX_TRY(expr) \
  if ((rc = (expr)) != TMX_OK) return rc;

  for (int it = 0; it < n_steps; ++it) {
    {  // embedding gather + first input norm
      RowNormArgs a = {};
      a.embed = (const uint16_t*)m->embed;
      a.token_buffer = s->token_buffer;
      a.step = s->step;
      a.buf_len = L;
      a.x_out = w.x;
      a.norm_w = (const uint16_t*)m->layers[0].norm1_w;
      a.xn_out = w.xn;
      a.D = D; a.eps = m->norm_eps; a.family = m->family;
      TMX_TRY(row_norm(st, a, B));
    }
    for (int i = 0; i < m->num_layers; ++i) {
      const tmx_layer_desc& l = m->layers[i];
      uint16_t* kc = (uint16_t*)s->kv_cache + (size_t)(2 * i) * kv_elems;
      uint16_t* vc = kc + kv_elems;
      TMX_TRY(qlinear_base(st, w.xn, D, l.qkv.qweight, l.qkv.scales, l.qkv.lora_a_t, w.qkv, QKV, w.t,
                           TMX_MAX_RPAD, B, D, QKV, l.qkv.G, l.qkv.r_pad));
      {
        RopeArgs a = {};
        a.qkv = w.qkv;
        a.t = l.qkv.lora_a_t ? w.t : nullptr;
        a.ldt = TMX_MAX_RPAD;
        a.lora_b = (const uint16_t*)l.qkv.lora_b;
        a.r = l.qkv.rank; a.ls = l.qkv.lora_scale;
        a.q_norm_w = (const uint16_t*)l.q_norm_w;
        a.k_norm_w = (const uint16_t*)l.k_norm_w;
        a.positions = s->positions; a.step = s->step; a.buf_len = L;
        a.q_out = w.q; a.kcache = kc; a.vcache = vc;
        a.N = N; a.Kh = Kh; a.H = H; a.C = C;
        a.theta = theta; a.eps = m->norm_eps; a.family = m->family;
        TMX_TRY(rope_kvwrite(st, a, B));
      }
      {
        AttnArgs a = {};
        a.q = w.q; a.kcache = kc; a.vcache = vc;
        a.input_mask = s->input_mask; a.step = s->step; a.buf_len = L;
        a.out = w.attn; a.partial = w.attn_partial;
        a.B = B; a.N = N; a.Kh = Kh; a.C = C;
        a.scale = 1.0f / sqrtf((float)H);
        TMX_TRY(gqa_decode(st, a, H));
      }
      TMX_TRY(qlinear_base(st, w.attn, NH, l.o.qweight, l.o.scales, l.o.lora_a_t, w.yo, D, w.t,
                           TMX_MAX_RPAD, B, NH, D, l.o.G, l.o.r_pad));
      {
        RowNormArgs a = {};
        a.y = w.yo;
        a.t = l.o.lora_a_t ? w.t : nullptr;
        a.ldt = TMX_MAX_RPAD;
        a.lora_b = (const uint16_t*)l.o.lora_b;
        a.r = l.o.rank; a.ls = l.o.lora_scale;
        a.residual = w.x; a.x_out = w.x;
        a.norm_w = (const uint16_t*)l.norm2_w; a.xn_out = w.xn;
        a.D = D; a.eps = m->norm_eps; a.family = m->family;
        TMX_TRY(row_norm(st, a, B));
      }
      TMX_TRY(qlinear_base(st, w.xn, D, l.gate_up.qweight, l.gate_up.scales, l.gate_up.lora_a_t, w.gu,
                           2 * F, w.t, TMX_MAX_RPAD, B, D, 2 * F, l.gate_up.G, l.gate_up.r_pad));
      {
        SwigluArgs a = {};
        a.gu = w.gu;
        a.t = l.gate_up.lora_a_t ? w.t : nullptr;
        a.ldt = TMX_MAX_RPAD;
        a.lora_b = (const uint16_t*)l.gate_up.lora_b;
        a.r = l.gate_up.rank; a.ls = l.gate_up.lora_scale;
        a.act = w.act; a.F = F;
        TMX_TRY(swiglu(st, a, B));
      }
      TMX_TRY(qlinear_base(st, w.act, F, l.down.qweight, l.down.scales, l.down.lora_a_t, w.yo, D, w.t,
                           TMX_MAX_RPAD, B, F, D, l.down.G, l.down.r_pad));
      {
        RowNormArgs a = {};
        a.y = w.yo;
        a.t = l.down.lora_a_t ? w.t : nullptr;
        a.ldt = TMX_MAX_RPAD;
        a.lora_b = (const uint16_t*)l.down.lora_b;
        a.r = l.down.rank; a.ls = l.down.lora_scale;
        a.residual = w.x; a.x_out = w.x;
        a.norm_w = (const uint16_t*)(i + 1 < m->num_layers ? m->layers[i + 1].norm1_w : m->final_norm_w);
        a.xn_out = w.xn;
        a.D = D; a.eps = m->norm_eps; a.family = m->family;
        TMX_TRY(row_norm(st, a, B));
      }
    }
    if (sample) {
      HeadArgs a = {};
      a.x = w.xn;
      a.w = (const uint16_t*)m->head;
      a.M = B; a.D = D; a.V = m->vocab_size;
      a.mode = s->sampling_mode;
      a.temperature = s->temperature;
      a.k0 = s->seed_hi; a.k1 = s->seed_lo;
      a.step = s->step;
      a.forbidden = s->forbidden; a.n_forbidden = s->n_forbidden;
      a.logits_out = s->logits_out;
      const size_t nwg = (m->vocab_size + 127) / 128;
      a.part_f = (float*)w.head_partial;
      a.part_i = (int32_t*)((float*)w.head_partial + (size_t)B * nwg * 4);
      a.token_buffer = s->token_buffer;
      a.logprobs = s->logprobs;
      a.done = s->done;
      a.eos = s->eos_ids; a.n_eos = s->n_eos;
      a.buf_len = L;
      TMX_TRY(head_sample(st, a));
    }
    TMX_TRY(advance_step(st, s->step));
  }
#undef TMX_TRY
  return TMX_OK;
}
