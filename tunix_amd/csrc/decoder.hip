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
#include <vector>

#include "tmx_kernels.h"

namespace tmx {

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct Workspace {
  uint16_t* delta;   // LoRA delta of a split projection, made by its LoRA blocks (up to 128 rows)
  void* dsync;       // their hand-over area
  uint32_t* status;  // first 256 bytes, the same place for every batch size: word 0 is set when a bounded wait inside a kernel runs out
  uint16_t *x, *xn, *q, *attn, *act, *y16;
  float *y_part, *t_part, *rope_tab;
  uint16_t* t16;  // bf16 LoRA projection of a many-rows pass
  void* gu_sync;  // hand-over area of the fused gate | up launch (LoRA projection computed once per launch)
  float* sb_tparts;        // small-batch step: parts of the down projection's t left by gate | up
  float* sb_attn_partial;  // small-batch step: split results of the attention kernel
  float* attn_partial;
  void* head_partial;
  // routed experts (MoE models)
  int32_t* expert_of;
  float* weight_of;
  uint16_t *pair_act, *pair_y;
  size_t total;
};

// gate | up + LoRA + SwiGLU in one launch pays up to 64 rows (the 8-wave kernel); at 65..128 rows the
// split-free k-way projection plus a SwiGLU launch is faster (8B shape, 128 rows: 1.76 against 2.18 ms per step)
static const int kFusedGateUpMaxRows = 64;

struct Splits { int qkv, o, gate_up, down; };

// One to four sequences, one token each, dense layers of either family whose shapes fit the small-batch
// kernels: five launches per layer (see smallbatch.hip).
static const int kSmallBatchMaxRows = 4;
static bool small_batch_ok(const tmx_model_desc* m, int B, int T) {
  if (B > kSmallBatchMaxRows || T != 1 || m->num_experts > 0) return false;
  const int D = m->embed_dim, N = m->num_heads, Kh = m->num_kv_heads, H = m->head_dim, F = m->hidden_dim;
  const int NH = N * H, QKV = (N + 2 * Kh) * H;
  if (!sb_attn_ok(N, Kh, H)) return false;
  for (int i = 0; i < m->num_layers; ++i) {
    const tmx_layer_desc& l = m->layers[i];
    if ((l.q_norm_w != nullptr) != (l.k_norm_w != nullptr)) return false;
    if (!sb_linear_ok(B, D, QKV, l.qkv.G, l.qkv.lora_a_t ? l.qkv.rank : 0, l.qkv.lora_a_t ? l.qkv.r_pad : 0, true)) return false;
    if (!sb_linear_ok(B, NH, D, l.o.G, l.o.lora_a_t ? l.o.rank : 0, l.o.lora_a_t ? l.o.r_pad : 0, false)) return false;
    if (F % 32 || !sb_linear_ok(B, D, 2 * F, l.gate_up.G, l.gate_up.lora_a_t ? l.gate_up.rank : 0,
                                l.gate_up.lora_a_t ? l.gate_up.r_pad : 0, true))
      return false;
    if (!sb_linear_ok(B, F, D, l.down.G, l.down.lora_a_t ? l.down.rank : 0, l.down.lora_a_t ? l.down.r_pad : 0, false))
      return false;
    if (l.qkv.lora_a_t && 3 * l.qkv.rank > 64) return false;
    if (l.gate_up.lora_a_t && (l.gate_up.r_pad != 32 || 2 * l.gate_up.rank > 32)) return false;
    if (l.down.lora_a_t && l.down.r_pad != 32) return false;
  }
  return true;
}

static Splits plan_splits(const tmx_model_desc* m, int B) {
  const int D = m->embed_dim, NH = m->num_heads * m->head_dim;
  const int QKV = NH + 2 * m->num_kv_heads * m->head_dim, F = m->hidden_dim;
  Splits s;
  s.qkv = qlinear_num_splits(D, QKV, B);
  s.o = qlinear_num_splits(NH, D, B);
  s.gate_up = m->num_experts > 0 ? 1 : qlinear_num_splits(D, 2 * F, B);
  // up to 64 rows the 8-wave gate | up kernel (projection + LoRA + SwiGLU in one launch) beats a
  // split projection plus a SwiGLU launch as soon as it has 64 workgroups to run
  const tmx_qlinear_desc& gu = m->layers[0].gate_up;
  if (m->num_experts == 0 && B <= 64 && D % 512 == 0 && D < 8192 && F % 64 == 0 && F / 64 >= 64 &&
      (!gu.lora_a_t || (2 * gu.rank <= 32 && gu.r_pad == 32)))
    s.gate_up = 1;
  s.down = m->num_experts > 0 ? 1 : qlinear_num_splits(F, D, B);
  return s;
}

static Workspace carve(const tmx_model_desc* m, int B, int C, char* base) {
  Workspace w;
  size_t off = 0;
  // a region of zero bytes has no address: its pointer is null, and users test the pointer
  auto take = [&](size_t bytes) { char* p = (base && bytes) ? base + off : nullptr; off += align256(bytes); return p; };
  const size_t D = m->embed_dim, NH = (size_t)m->num_heads * m->head_dim;
  const size_t QKV = NH + 2 * (size_t)m->num_kv_heads * m->head_dim, F = m->hidden_dim;
  const Splits sp = plan_splits(m, B);
  size_t ypart = sp.qkv * QKV;
  if (sp.o * D > ypart) ypart = sp.o * D;
  if (sp.down * D > ypart) ypart = sp.down * D;
  if (sp.gate_up > 1 && sp.gate_up * 2 * F > ypart) ypart = sp.gate_up * 2 * F;
  w.status = (uint32_t*)take(256);
  w.x = (uint16_t*)take(B * D * 2);
  w.xn = (uint16_t*)take(B * D * 2);
  w.q = (uint16_t*)take(B * NH * 2);
  w.attn = (uint16_t*)take(B * NH * 2);
  w.act = (uint16_t*)take(B * F * 2);
  w.y16 = (uint16_t*)take(B * 2 * F * 2);
  w.y_part = (float*)take((size_t)B * ypart * 4);
  w.t_part = (float*)take((size_t)TMX_MAX_LORA_SPLITS * B * TMX_MAX_RPAD * 4);
  w.t16 = (uint16_t*)take(B > 128 ? (size_t)B * TMX_MAX_RPAD * 2 : 0);
  {
    w.delta = (uint16_t*)take(B <= 128 ? (size_t)B * D * 2 : 0);
    w.dsync = take(B <= 128 ? qlinear_delta_sync_bytes(B, TMX_MAX_RPAD) : 0);
  }
  w.gu_sync = take(B <= kFusedGateUpMaxRows && m->num_experts == 0 && D % 256 == 0 ? qlinear_gate_up_sync_bytes(B, (int)D) : 0);
  const bool small = B <= kSmallBatchMaxRows && m->num_experts == 0;
  w.sb_tparts = (float*)take(small ? (F / 32 + 1) * (size_t)B * 32 * 4 : 0);
  w.sb_attn_partial = (float*)take(small ? sb_attn_partial_bytes(B, m->num_heads, m->num_kv_heads, m->head_dim, C) : 0);
  w.rope_tab = (float*)take((size_t)B * m->head_dim * 4);
  {
    // split results of decode attention; up to 128 rows also room for the shared walk over prompt slots
    size_t ab = attn_partial_bytes(B, m->num_heads, m->num_kv_heads, m->head_dim, C);
    if (B <= 128) {
      const size_t sb = attn_shared_partial_bytes(B, m->num_heads, m->num_kv_heads, m->head_dim, C);
      if (sb > ab) ab = sb;
    }
    w.attn_partial = (float*)take(ab);
  }
  w.head_partial = take(head_partial_bytes(B, m->vocab_size));
  const size_t P = m->num_experts > 0 ? (size_t)B * m->experts_per_tok : 0;
  w.expert_of = (int32_t*)take(P * 4);
  w.weight_of = (float*)take(P * 4);
  w.pair_act = (uint16_t*)take(P * F * 2);
  w.pair_y = (uint16_t*)take(P * D * 2);
  w.total = off;
  return w;
}

// Optional per-kernel-class timing with HIP events (used by the benchmark only).
struct Prof {
  std::vector<hipEvent_t> ev[TMX_NUM_KERNEL_CLASSES];
  void before(int k, hipStream_t st) { push(k, st); }
  void after(int k, hipStream_t st) { push(k, st); }
  void push(int k, hipStream_t st) {
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, st);
    ev[k].push_back(e);
  }
};

static int check_linear(const tmx_qlinear_desc& l, int K, int N) {
  if (!l.qweight || !l.scales) return TMX_ERR_ARG;
  if (l.K != K || l.N != N) return TMX_ERR_SHAPE;
  if (l.lora_a_t && (!l.lora_b || l.rank <= 0 || l.r_pad > TMX_MAX_RPAD || l.rank > 64)) return TMX_ERR_ARG;
  return TMX_OK;
}

}  // namespace tmx

using namespace tmx;

extern "C" size_t tmx_decode_workspace_bytes(const tmx_model_desc* m, int batch, int cache_size) {
  if (!m || batch <= 0) return 0;
  return carve(m, batch, cache_size, nullptr).total;
}

static int decode_steps_impl(const tmx_model_desc* m, const tmx_decode_state* s, void* stream,
                             int n_steps, int sample, Prof* prof) {
  if (!m || !s || !m->layers || !m->embed || !m->final_norm_w || !m->head) return TMX_ERR_ARG;
  if (!s->token_buffer || !s->positions || !s->input_mask || !s->done || !s->step || !s->kv_cache ||
      !s->workspace)
    return TMX_ERR_ARG;
  const bool moe = m->num_experts > 0;
  // rows of a pass: one per sequence, or tokens_per_pass consecutive tokens of every sequence
  // (cache fill and scoring only: sampling needs the previous token)
  const int NSEQ = s->batch, T = s->tokens_per_pass > 1 ? s->tokens_per_pass : 1;
  if (NSEQ <= 0 || NSEQ > TMX_MAX_FILL_ROWS || T > 128) return TMX_ERR_SHAPE;
  if (T > 1 && sample && s->sampling_mode != TMX_SAMPLE_SCORE) return TMX_ERR_ARG;
  const int B = NSEQ * T, C = s->cache_size, L = s->buf_len;
  // a pass takes up to TMX_MAX_FILL_ROWS rows; above 128 rows the projections multiply in 256-row
  // blocks (every K % 128 == 0), the head takes its rows 64 at a time or in 256 x 256 blocks; MoE models
  // are bounded by the routed pairs per pass (checked below)
  if (B > TMX_MAX_FILL_ROWS || C <= 0 || L <= 0 || L > C) return TMX_ERR_SHAPE;
  if (moe && (m->experts_per_tok <= 0 || m->experts_per_tok > m->num_experts ||
              (size_t)B * m->experts_per_tok > TMX_MAX_MOE_PAIRS))
    return TMX_ERR_SHAPE;
  const bool nucleus = sample && s->sampling_mode == TMX_SAMPLE_TOP_P && (s->top_p < 1.0f || s->top_k > 0);
  if (nucleus && !s->nucleus_workspace) return TMX_ERR_ARG;
  const int D = m->embed_dim, N = m->num_heads, Kh = m->num_kv_heads, H = m->head_dim;
  const int F = m->hidden_dim, NH = N * H, QKV = (N + 2 * Kh) * H;
  if (carve(m, B, C, nullptr).total > s->workspace_bytes) return TMX_ERR_SHAPE;
  for (int i = 0; i < m->num_layers; ++i) {
    const tmx_layer_desc& l = m->layers[i];
    if (!l.norm1_w || !l.norm2_w) return TMX_ERR_ARG;
    int rc;
    if ((rc = check_linear(l.qkv, D, QKV)) || (rc = check_linear(l.o, NH, D))) return rc;
    if (moe) {
      if (!l.router_w || l.gate_up.lora_a_t || l.down.lora_a_t) return TMX_ERR_ARG;
    }
    // dense: one matrix; MoE: num_experts stacked matrices of the same per-expert shape
    if ((rc = check_linear(l.gate_up, D, 2 * F)) || (rc = check_linear(l.down, F, D))) return rc;
  }
  hipStream_t st = (hipStream_t)stream;
  const Workspace w = carve(m, B, C, (char*)s->workspace);
  const size_t kv_elems = (size_t)NSEQ * C * Kh * H;
  const float theta = m->family == TMX_FAMILY_LLAMA3 ? 1000000.0f : m->rope_theta;
  int rc;
#define TMX_TRY(kind, expr)            \
  {                                    \
    if (prof) prof->before(kind, st);  \
    rc = (expr);                       \
    if (prof) prof->after(kind, st);   \
    if (rc != TMX_OK) return rc;       \
  }

  const Splits sp = plan_splits(m, B);
  const bool small = small_batch_ok(m, B, T);
  auto lora_of = [&](const tmx_qlinear_desc& l, int) {
    LoraIn li = {};
    if (l.lora_a_t) {
      li.t_part = w.t_part;
      li.ldt = TMX_MAX_RPAD;
      li.nsplit = qlinear_num_lora_splits(l.K, l.N);
      li.b = (const uint16_t*)l.lora_b;
      li.r = l.rank;
      li.ls = l.lora_scale;
    }
    return li;
  };
  // Up to 128 rows, o and down projections of the direct-to-LDS kernel whose K-slices are long enough to hide
  // it: the LoRA blocks of the launch also make delta = bf16(bf16(t . B) * ls), so the row kernel behind adds one
  // bf16 row instead of multiplying by B (every row re-read all of B there).
  auto delta_of = [&](const tmx_qlinear_desc& l, int nsplit, int e0, int e1, LoraDelta& ld) {
    if (!l.lora_a_t || !w.delta || !w.dsync || e0 % 32 || e1 % 32) return false;
    if (!qlinear_delta_ok(B, l.K, l.N, l.r_pad, l.rank, nsplit)) return false;
    ld = LoraDelta();
    ld.delta = w.delta;
    ld.lora_b = (const uint16_t*)l.lora_b; ld.r = l.rank; ld.ls = l.lora_scale;
    ld.seg_end[0] = e0; ld.seg_end[1] = e1; ld.seg_end[2] = l.N;
    ld.sync_ws = w.dsync; ld.status = w.status;
    return true;
  };
  if (w.dsync && n_steps > 0) {  // the hand-over words start at zero (the kernel leaves them so)
    rc = zero_words(st, (uint32_t*)w.dsync, 64);
    if (rc != TMX_OK) return rc;
  }
  // Many rows (B > 128): projection + LoRA in one pass into w.y16 where the shape allows it (unsplit,
  // rank % 8 == 0); returns TMX_ERR_UNSUPPORTED (nothing launched) when the caller must take the planes path.
  auto wide_linear = [&](const void* x, int ldx, const tmx_qlinear_desc& l, int e0, int e1) {
    if (B <= 128) return (int)TMX_ERR_UNSUPPORTED;
    const int seg_end[3] = {e0, e1, l.N};
    return qlinear_wide_lora(st, x, ldx, l.qweight, l.scales, l.lora_a_t, l.lora_b, l.rank, l.lora_scale, seg_end,
                             w.y16, w.t_part, w.t16, B, l.K, l.N, l.G, l.r_pad);
  };
  // the hand-over words of the fused gate | up launch start at zero (the kernel leaves them so)
  if (!moe && B <= kFusedGateUpMaxRows && w.gu_sync && n_steps > 0) {
    rc = zero_words(st, (uint32_t*)w.gu_sync, 64);
    if (rc != TMX_OK) return rc;
  }
  // samples of one prompt in consecutive rows: decode attention reads the prompt slots once per group
  const bool share_walk = T == 1 && !small && w.attn_partial && attn_share_ok(B, N, Kh, H, C, s->share_group, s->share_len);
  for (int it = 0; it < n_steps; ++it) {
    {  // embedding gather + first input norm + this step's RoPE table
      RowNormArgs a = {};
      a.embed = (const uint16_t*)m->embed;
      a.vocab = m->vocab_size;
      a.token_buffer = s->token_buffer;
      a.step = s->step;
      a.buf_len = L;
      a.tpp = T;
      a.positions = s->positions;
      a.rope_tab = w.rope_tab;
      a.half = H / 2;
      a.theta = theta;
      a.x_out = w.x;
      a.norm_w = (const uint16_t*)m->layers[0].norm1_w;
      a.xn_out = w.xn;
      a.D = D; a.eps = m->norm_eps; a.family = m->family;
      TMX_TRY(TMX_K_ROWNORM, row_norm(st, a, B));
    }
    if (small) {
      // the residual stream lives in w.x (the embedding row kernel wrote it); norms run inside the projections
      for (int i = 0; i < m->num_layers; ++i) {
        const tmx_layer_desc& l = m->layers[i];
        uint16_t* kc = (uint16_t*)s->kv_cache + (size_t)(2 * i) * kv_elems;
        uint16_t* vc = kc + kv_elems;
        auto base_args = [&](const tmx_qlinear_desc& d, bool own_t) {
          SbLinearArgs a = {};
          a.M = B;
          a.eps = m->norm_eps; a.family = m->family;
          a.qw = (const uint4*)d.qweight; a.scales = (const uint16_t*)d.scales;
          a.K = d.K; a.N = d.N; a.G = d.G;
          a.seg_end[0] = a.seg_end[1] = a.seg_end[2] = d.N;
          if (d.lora_a_t) {
            if (own_t) { a.a_t = (const uint16_t*)d.lora_a_t; a.Rpad = d.r_pad; }
            a.lora_b = (const uint16_t*)d.lora_b; a.lora_r = d.rank; a.lora_ls = d.lora_scale;
          }
          a.ldy = d.N;
          return a;
        };
        {
          SbLinearArgs a = base_args(l.qkv, true);
          a.x = w.x; a.ldx = D; a.norm_w = (const uint16_t*)l.norm1_w;
          a.seg_end[0] = NH; a.seg_end[1] = NH + Kh * H;
          a.y = w.y16;
          TMX_TRY(TMX_K_QKV, sb_linear(st, a, 1, 0));
        }
        const int ans = sb_attn_splits(B, Kh, C);
        {
          SbAttnArgs a = {};
          a.qkv = w.y16; a.rope_tab = w.rope_tab; a.kcache = kc; a.vcache = vc;
          a.input_mask = s->input_mask; a.step = s->step; a.buf_len = L;
          a.partial = w.sb_attn_partial;
          a.B = B; a.N = N; a.Kh = Kh; a.C = C; a.nsplit = ans;
          a.scale = 1.0f / sqrtf((float)H);
          a.q_norm_w = (const uint16_t*)l.q_norm_w; a.k_norm_w = (const uint16_t*)l.k_norm_w;
          a.eps = m->norm_eps; a.family = m->family;
          TMX_TRY(TMX_K_ATTN, sb_attn(st, a, H));
        }
        {
          SbLinearArgs a = base_args(l.o, true);
          a.attn_part = w.sb_attn_partial; a.attn_kh = Kh; a.attn_g = N / Kh; a.attn_h = H; a.attn_ns = ans;
          a.residual = w.x; a.y = w.x;
          TMX_TRY(TMX_K_O, sb_linear(st, a, 2, 1));
        }
        {
          SbLinearArgs a = base_args(l.gate_up, true);
          a.x = w.x; a.ldx = D; a.norm_w = (const uint16_t*)l.norm2_w;
          a.seg_end[0] = F;
          a.y = w.act; a.ldy = F; a.pair_off = F / 32;
          if (l.down.lora_a_t) { a.a_next = (const uint16_t*)l.down.lora_a_t; a.t_parts_out = w.sb_tparts; }
          TMX_TRY(TMX_K_GATE_UP, sb_linear(st, a, 1, 2));
        }
        {
          SbLinearArgs a = base_args(l.down, false);
          a.x = w.act; a.ldx = F;
          if (l.down.lora_a_t) { a.t_parts = w.sb_tparts; a.t_nparts = F / 32; }
          a.residual = w.x; a.y = w.x;
          TMX_TRY(TMX_K_DOWN, sb_linear(st, a, 0, 1));
        }
        if (prof) TMX_TRY(TMX_K_EMPTY, empty_launch(st));
      }
      {  // final norm in front of the head
        RowNormArgs a = {};
        a.y_bf16 = w.x;
        a.norm_w = (const uint16_t*)m->final_norm_w; a.xn_out = w.xn;
        a.D = D; a.eps = m->norm_eps; a.family = m->family;
        if (sample) TMX_TRY(TMX_K_ROWNORM, row_norm(st, a, B));
      }
    }
    for (int i = 0; !small && i < m->num_layers; ++i) {
      const tmx_layer_desc& l = m->layers[i];
      // gate | up with LoRA + SwiGLU in its epilogue: K % 256 == 0 below 8192, unsplit, 2 r <= 32
      const bool fused_gu = !moe && B <= kFusedGateUpMaxRows && sp.gate_up == 1 && D % 256 == 0 && D < 8192 && F % 64 == 0 &&
                            (!l.gate_up.lora_a_t || (2 * l.gate_up.rank <= 32 && l.gate_up.r_pad == 32));
      uint16_t* kc = (uint16_t*)s->kv_cache + (size_t)(2 * i) * kv_elems;
      uint16_t* vc = kc + kv_elems;
      bool fused;  // this projection ran with LoRA in its epilogue: the consumer reads bf16, no LoRA left
      LoraDelta ld;
      bool with_delta = false;  // the projection's LoRA blocks made the delta: the consumer adds it
      {
        if (prof) prof->before(TMX_K_QKV, st);
        rc = wide_linear(w.xn, D, l.qkv, NH, NH + Kh * H);
        fused = rc != TMX_ERR_UNSUPPORTED;
        if (!fused)
          rc = qlinear_base(st, w.xn, D, l.qkv.qweight, l.qkv.scales, l.qkv.lora_a_t, nullptr, w.y_part, w.t_part,
                            TMX_MAX_RPAD, B, D, QKV, l.qkv.G, l.qkv.r_pad, sp.qkv);
        if (prof) prof->after(TMX_K_QKV, st);
        if (rc != TMX_OK) return rc;
      }
      {
        RopeArgs a = {};
        if (fused) {
          a.qkv_bf16 = w.y16;
        } else {
          a.qkv_part = w.y_part;
          a.nsplit = sp.qkv;
          a.lora = lora_of(l.qkv, sp.qkv);
        }
        a.q_norm_w = (const uint16_t*)l.q_norm_w;
        a.k_norm_w = (const uint16_t*)l.k_norm_w;
        a.positions = s->positions; a.step = s->step; a.buf_len = L; a.tpp = T;
        a.rope_tab = w.rope_tab;
        a.q_out = w.q; a.kcache = kc; a.vcache = vc;
        a.N = N; a.Kh = Kh; a.H = H; a.C = C;
        a.theta = theta; a.eps = m->norm_eps; a.family = m->family;
        TMX_TRY(TMX_K_ROPE, rope_kvwrite(st, a, B));
      }
      {
        AttnArgs a = {};
        a.q = w.q; a.kcache = kc; a.vcache = vc;
        a.input_mask = s->input_mask; a.step = s->step; a.buf_len = L; a.tpp = T;
        a.out = w.attn; a.partial = w.attn_partial;
        a.B = B; a.N = N; a.Kh = Kh; a.C = C;
        a.scale = 1.0f / sqrtf((float)H);
        if (share_walk) { a.share_gs = s->share_group; a.share_len = s->share_len; }
        TMX_TRY(TMX_K_ATTN, gqa_decode(st, a, H));
      }
      {
        if (prof) prof->before(TMX_K_O, st);
        rc = wide_linear(w.attn, NH, l.o, D, D);
        fused = rc != TMX_ERR_UNSUPPORTED;
        if (!fused) {
          with_delta = delta_of(l.o, sp.o, D, D, ld);
          rc = qlinear_base(st, w.attn, NH, l.o.qweight, l.o.scales, l.o.lora_a_t, nullptr, w.y_part, w.t_part,
                            TMX_MAX_RPAD, B, NH, D, l.o.G, l.o.r_pad, sp.o, with_delta ? &ld : nullptr);
        }
        if (prof) prof->after(TMX_K_O, st);
        if (rc != TMX_OK) return rc;
      }
      {
        RowNormArgs a = {};
        if (fused) {
          a.y_bf16 = w.y16;
        } else {
          a.y_part = w.y_part;
          a.nsplit = sp.o;
          if (with_delta) a.delta = w.delta;
          else a.lora = lora_of(l.o, sp.o);
        }
        a.residual = w.x; a.x_out = w.x;
        a.norm_w = (const uint16_t*)l.norm2_w; a.xn_out = w.xn;
        a.D = D; a.eps = m->norm_eps; a.family = m->family;
        if (moe) {
          // the row's workgroup routes its token from the normed row it has just made: scores, softmax, top-k
          // (19 us per layer as a launch of its own on the 30B-A3B shape at 32 sequences)
          a.router.w = (const uint16_t*)l.router_w;
          a.router.D = D; a.router.E = m->num_experts; a.router.top_k = m->experts_per_tok;
          a.router.expert_of = w.expert_of; a.router.weight_of = w.weight_of;
        }
        TMX_TRY(TMX_K_ROWNORM, row_norm(st, a, B));
      }
      if (moe) {
        const int P = B * m->experts_per_tok;
        MoeArgs e = {};
        e.expert_of = w.expert_of; e.P = P; e.top_k = m->experts_per_tok;
        e.x = w.xn; e.ldx = D;
        e.qw = (const uint4*)l.gate_up.qweight; e.scales = (const uint16_t*)l.gate_up.scales;
        e.K = D; e.N = 2 * F; e.G = l.gate_up.G;
        e.qw_stride = (size_t)e.K * e.N / 32; e.sc_stride = (size_t)(e.K / e.G) * e.N;
        e.out = w.pair_act; e.ldo = F;
        TMX_TRY(TMX_K_GATE_UP, moe_experts(st, e, m->num_experts, false));
        e.x = w.pair_act; e.ldx = F;
        e.qw = (const uint4*)l.down.qweight; e.scales = (const uint16_t*)l.down.scales;
        e.K = F; e.N = D; e.G = l.down.G;
        e.qw_stride = (size_t)e.K * e.N / 32; e.sc_stride = (size_t)(e.K / e.G) * e.N;
        e.out = w.pair_y; e.ldo = D;
        TMX_TRY(TMX_K_DOWN, moe_experts(st, e, m->num_experts, true));
        RowNormArgs a = {};
        a.moe_y = w.pair_y; a.moe_w = w.weight_of; a.top_k = m->experts_per_tok;
        a.residual = w.x; a.x_out = w.x;
        a.norm_w = (const uint16_t*)(i + 1 < m->num_layers ? m->layers[i + 1].norm1_w : m->final_norm_w);
        a.xn_out = w.xn;
        a.D = D; a.eps = m->norm_eps; a.family = m->family;
        TMX_TRY(TMX_K_ROWNORM, row_norm(st, a, B));
      } else {
        if (fused_gu) {
          TMX_TRY(TMX_K_GATE_UP, qlinear_gate_up_swiglu(
              st, w.xn, D, l.gate_up.qweight, l.gate_up.scales, l.gate_up.lora_a_t, l.gate_up.lora_b,
              l.gate_up.rank, l.gate_up.lora_scale, w.act, B, D, F, l.gate_up.G, w.gu_sync, w.status));
        } else {
        const bool gu16 = sp.gate_up == 1;
        {
          if (prof) prof->before(TMX_K_GATE_UP, st);
          rc = wide_linear(w.xn, D, l.gate_up, F, 2 * F);
          fused = rc != TMX_ERR_UNSUPPORTED;
          if (!fused)
            rc = qlinear_base(st, w.xn, D, l.gate_up.qweight, l.gate_up.scales, l.gate_up.lora_a_t,
                              gu16 ? w.y16 : nullptr, w.y_part, w.t_part, TMX_MAX_RPAD, B, D, 2 * F, l.gate_up.G,
                              l.gate_up.r_pad, sp.gate_up);
          if (prof) prof->after(TMX_K_GATE_UP, st);
          if (rc != TMX_OK) return rc;
        }
        {
          SwigluArgs a = {};
          a.gu_bf16 = (gu16 || fused) ? w.y16 : nullptr;
          a.gu_part = w.y_part;
          a.nsplit = sp.gate_up;
          if (!fused) a.lora = lora_of(l.gate_up, sp.gate_up);
          a.act = w.act; a.F = F;
          TMX_TRY(TMX_K_SWIGLU, swiglu(st, a, B));
        }
        }
        {
          if (prof) prof->before(TMX_K_DOWN, st);
          rc = wide_linear(w.act, F, l.down, D, D);
          fused = rc != TMX_ERR_UNSUPPORTED;
          if (!fused) {
            with_delta = delta_of(l.down, sp.down, D, D, ld);
            rc = qlinear_base(st, w.act, F, l.down.qweight, l.down.scales, l.down.lora_a_t, nullptr, w.y_part,
                              w.t_part, TMX_MAX_RPAD, B, F, D, l.down.G, l.down.r_pad, sp.down, with_delta ? &ld : nullptr);
          }
          if (prof) prof->after(TMX_K_DOWN, st);
          if (rc != TMX_OK) return rc;
        }
        {
          RowNormArgs a = {};
          if (fused) {
            a.y_bf16 = w.y16;
          } else {
            a.y_part = w.y_part;
            a.nsplit = sp.down;
            if (with_delta) a.delta = w.delta;
            else a.lora = lora_of(l.down, sp.down);
          }
          a.residual = w.x; a.x_out = w.x;
          a.norm_w = (const uint16_t*)(i + 1 < m->num_layers ? m->layers[i + 1].norm1_w : m->final_norm_w);
          a.xn_out = w.xn;
          a.D = D; a.eps = m->norm_eps; a.family = m->family;
          TMX_TRY(TMX_K_ROWNORM, row_norm(st, a, B));
        }
      }
      if (prof) TMX_TRY(TMX_K_EMPTY, empty_launch(st));
    }
    if (sample && !nucleus && B > 64 && !s->logits_out && s->n_forbidden == 0 && D % 128 == 0) {
      // more than 64 rows: the head in 256 x 256 blocks, one pass over the head matrix (the 64-row kernel
      // would take one pass per 64 rows)
      HeadArgs a = {};
      a.x = w.xn;
      a.w = (const uint16_t*)m->head;
      a.M = B; a.D = D; a.V = m->vocab_size;
      a.mode = s->sampling_mode;
      a.temperature = s->temperature;
      a.k0 = s->seed_hi; a.k1 = s->seed_lo;
      a.step = s->step;
      a.part_f = (float*)w.head_partial;
      a.part_i = (int32_t*)((float*)w.head_partial + (size_t)B * ((m->vocab_size + 255) / 256) * 4);
      a.token_buffer = s->token_buffer;
      a.logprobs = s->logprobs;
      a.done = s->done;
      a.eos = s->eos_ids; a.n_eos = s->n_eos;
      a.buf_len = L;
      a.tpp = T;
      TMX_TRY(TMX_K_HEAD, head_wide(st, a));
    } else if (sample) {
      HeadArgs a = {};
      a.x = w.xn;
      a.w = (const uint16_t*)m->head;
      a.w_tiles = (const uint16_t*)m->head_tiles;
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
      a.tpp = T;
      if (nucleus) {
        TMX_TRY(TMX_K_HEAD, head_sample_nucleus(st, a, s->top_p, s->top_k, s->nucleus_workspace,
                                                s->nucleus_workspace_bytes));
      } else {
        TMX_TRY(TMX_K_HEAD, head_sample(st, a));
      }
    }
    TMX_TRY(TMX_K_ADVANCE, advance_step(st, s->step, T));
  }
#undef TMX_TRY
  return TMX_OK;
}

extern "C" int tmx_decode_steps(const tmx_model_desc* m, const tmx_decode_state* s, void* stream,
                                int n_steps, int sample) {
  return decode_steps_impl(m, s, stream, n_steps, sample, nullptr);
}

extern "C" int tmx_decode_status(const tmx_model_desc* m, const tmx_decode_state* s, void* stream) {
  if (!m || !s || !s->workspace || !m->layers) return TMX_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  if (s->workspace_bytes < 256) return TMX_ERR_ARG;
  uint32_t flag = 0;
  uint32_t* word = (uint32_t*)s->workspace;  // Workspace::status
  if (hipMemcpyAsync(&flag, word, 4, hipMemcpyDeviceToHost, st) != hipSuccess) return TMX_ERR_LAUNCH;
  if (hipStreamSynchronize(st) != hipSuccess) return TMX_ERR_LAUNCH;
  if (flag == 0) return TMX_OK;
  if (hipMemsetAsync(word, 0, 4, st) != hipSuccess) return TMX_ERR_LAUNCH;
  if (hipStreamSynchronize(st) != hipSuccess) return TMX_ERR_LAUNCH;
  return TMX_ERR_DEVICE_WAIT;
}

// One decode step recorded into a HIP graph and replayed: the step index lives on the device,
// so every replay is the same list of launches.  The first step runs eagerly (it also performs
// the one-time kernel attribute set-up), the capture happens on a private stream that is ordered
// after `stream` by events, and the replays are launched back on `stream`.
extern "C" int tmx_decode_steps_graph(const tmx_model_desc* m, const tmx_decode_state* s, void* stream,
                                      int n_steps, int sample) {
  if (n_steps < 4 || !m || !s) return decode_steps_impl(m, s, stream, n_steps, sample, nullptr);
  int rc = decode_steps_impl(m, s, stream, 1, sample, nullptr);
  if (rc != TMX_OK) return rc;
  hipStream_t user = (hipStream_t)stream;
  hipStream_t cap = nullptr;
  hipEvent_t ev = nullptr;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  rc = TMX_ERR_LAUNCH;
  bool captured = false;
  do {
    if (hipStreamCreateWithFlags(&cap, hipStreamNonBlocking) != hipSuccess) break;
    if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) break;
    if (hipStreamBeginCapture(cap, hipStreamCaptureModeThreadLocal) != hipSuccess) break;
    const int crc = decode_steps_impl(m, s, cap, 1, sample, nullptr);
    const hipError_t e = hipStreamEndCapture(cap, &graph);
    if (crc != TMX_OK) { rc = crc; break; }
    if (e != hipSuccess || !graph) break;
    if (hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) != hipSuccess) break;
    captured = true;
    rc = TMX_OK;
    for (int i = 1; i < n_steps; ++i)
      if (hipGraphLaunch(exec, user) != hipSuccess) { rc = TMX_ERR_LAUNCH; break; }
    // the graph objects may only go once the replays have run
    if (hipEventRecord(ev, user) == hipSuccess) (void)hipEventSynchronize(ev);
    else (void)hipStreamSynchronize(user);
  } while (false);
  if (exec) (void)hipGraphExecDestroy(exec);
  if (graph) (void)hipGraphDestroy(graph);
  if (ev) (void)hipEventDestroy(ev);
  if (cap) (void)hipStreamDestroy(cap);
  if (!captured && rc == TMX_ERR_LAUNCH) {
    (void)hipGetLastError();
    return decode_steps_impl(m, s, stream, n_steps - 1, sample, nullptr);  // capture unavailable
  }
  return rc;
}

extern "C" int tmx_decode_steps_profiled(const tmx_model_desc* m, const tmx_decode_state* s, void* stream,
                                         int n_steps, int sample, float* class_ms_host,
                                         int* class_launches_host) {
  if (!class_ms_host || !class_launches_host) return TMX_ERR_ARG;
  Prof prof;
  int rc = decode_steps_impl(m, s, stream, n_steps, sample, &prof);
  (void)hipStreamSynchronize((hipStream_t)stream);
  for (int k = 0; k < TMX_NUM_KERNEL_CLASSES; ++k) {
    float total = 0.f;
    for (size_t i = 0; i + 1 < prof.ev[k].size(); i += 2) {
      float ms = 0.f;
      if (hipEventElapsedTime(&ms, prof.ev[k][i], prof.ev[k][i + 1]) == hipSuccess) total += ms;
    }
    class_ms_host[k] = total;
    class_launches_host[k] = (int)(prof.ev[k].size() / 2);
    for (hipEvent_t e : prof.ev[k]) (void)hipEventDestroy(e);
  }
  return rc;
}
