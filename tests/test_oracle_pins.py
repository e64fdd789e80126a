"""Pins of the oracle that do not come from reference-held vectors: closed forms, invariants,
brute force in float64, and the `transformers` modelling code as a library routine for the
dense decoder forward (random weights built from a config object, fp32, CPU)."""
import numpy as np
import pytest

from oracle import int4
from oracle import layers as L
from oracle import model as OM
from oracle import masks as OMK
from oracle import sampling as OS
from oracle.bf16 import BF16, F32, bf16_round, bf16_bits, bf16_from_bits

import common as C


def test_bf16_round_matches_torch():
  import torch
  rng = np.random.default_rng(0)
  x = np.concatenate([rng.standard_normal(100000).astype(np.float32) * 10 ** rng.uniform(-30, 30, 100000),
                      np.array([0.0, -0.0, np.inf, -np.inf, 1.0039062, 1.00390625, 1.01171875, 3.3895314e38],
                               np.float32)]).astype(np.float32)
  want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
  np.testing.assert_array_equal(bf16_round(x), want)
  assert np.isnan(bf16_round(np.array([np.nan], np.float32)))[0]
  # ties to even on the 8th mantissa bit
  assert bf16_bits(bf16_round(bf16_from_bits(np.array([0x3F80], np.uint16)) + np.float32(2 ** -8)))[0] == 0x3F80
  assert bf16_bits(bf16_round(bf16_from_bits(np.array([0x3F81], np.uint16)) + np.float32(2 ** -8)))[0] == 0x3F82


def test_int4_pack_unpack_identity_and_layout():
  rng = np.random.default_rng(1)
  q = rng.integers(-8, 8, (192, 96)).astype(np.int8)
  packed = int4.pack_tiles(q)
  assert packed.size == q.size // 2
  np.testing.assert_array_equal(int4.unpack_tiles(packed, 192, 96), q)
  # explicit spot checks of the documented layout (independent index arithmetic)
  words = packed.view(np.uint32)
  for (k, n) in ((0, 0), (1, 0), (8, 5), (17, 31), (63, 32), (64, 33), (191, 95), (130, 64)):
    kb, nb, kk, nl = k // 64, n // 32, k % 64, n % 32
    t, h, j = kk // 16, (kk % 16) // 8, kk % 8
    i = (j // 2) + 4 * (j % 2)
    w = words[((nb * (192 // 64) + kb) * 64 + 32 * h + nl) * 4 + t]
    assert ((int(w) >> (4 * i)) & 15) - 8 == q[k, n], (k, n)


def test_int4_dequant_exhaustive_and_exact():
  # all 16 nibbles x every finite positive bf16 scale in a wide exponent range
  scales = bf16_from_bits(np.arange(0x3000, 0x4400, dtype=np.uint16))  # ~4.7e-10 .. 512
  q = np.repeat(np.arange(-8, 8, dtype=np.int8)[:, None], scales.size, axis=1)  # [16, S]
  q64 = np.tile(q, (4, 1))  # K = 64 rows, one group
  deq = int4.dequantize(q64, scales[None, :], 64)
  exact = q64.astype(np.float64) * scales.astype(np.float64)[None, :]
  # single RNE rounding of the exact product == a native bf16 multiply
  import torch
  want = (torch.from_numpy(q64.astype(np.float32)).to(torch.bfloat16) *
          torch.from_numpy(scales).to(torch.bfloat16)[None, :]).float().numpy()
  np.testing.assert_array_equal(deq, want)
  assert np.all(np.abs(deq - exact) <= np.abs(exact) * 2.0 ** -8 + 1e-45)


def test_int4_quantize_invariants():
  rng = np.random.default_rng(2)
  w = bf16_round(rng.standard_normal((256, 40)).astype(np.float32) * 0.02)
  w[64:128, 3] = 0  # a zero group
  q, s = int4.quantize(w, 64)
  assert q.min() >= -8 and q.max() <= 7 and s.shape == (4, 40)
  assert np.all(np.isfinite(s)) and np.all(s > 0)
  assert np.all(q[64:128, 3] == 0)
  deq = q.astype(np.float32) * np.repeat(s, 64, axis=0)
  err = np.abs(deq - w)
  clipped = (np.rint(w / np.repeat(s, 64, axis=0)) > 7)
  assert np.all(err[~clipped] <= np.repeat(s, 64, axis=0)[~clipped] / 2 + 1e-9)
  # sign symmetry (up to the asymmetric clip at +7)
  q2, s2 = int4.quantize(-w, 64)
  np.testing.assert_array_equal(s2, s)
  ok = (np.abs(q) < 8) & (np.abs(q2) < 8)
  np.testing.assert_array_equal(q2[ok], -q[ok])
  # the scale depends on the group's absmax only
  w3 = w.copy()
  w3[:64, 0] = np.where(np.abs(w3[:64, 0]) == np.abs(w3[:64, 0]).max(), w3[:64, 0], 0)
  assert int4.quantize(w3, 64)[1][0, 0] == s[0, 0]


def test_scale_pack_roundtrip():
  rng = np.random.default_rng(3)
  s = bf16_round(rng.uniform(1e-3, 1e-2, (6, 64)).astype(np.float32))
  np.testing.assert_array_equal(int4.unpack_scales(int4.pack_scales(s), 6, 64), s)


def test_product_quantizer_and_packer_match_oracle():
  import torch
  from tunix_amd import quant
  rng = np.random.default_rng(4)
  w = bf16_round(rng.standard_normal((256, 96)).astype(np.float32) * 0.02)
  for g in (64, 128):
    q, s = quant.quantize_int4(torch.from_numpy(w).to(torch.bfloat16), g)
    qo, so = int4.quantize(w, g)
    np.testing.assert_array_equal(q.numpy(), qo)
    np.testing.assert_array_equal(s.float().numpy(), so)
    np.testing.assert_array_equal(quant.pack_q4t(q).numpy().view(np.uint8).reshape(-1), int4.pack_tiles(qo))
    np.testing.assert_array_equal(quant.pack_scales(s).view(torch.int16).numpy().view(np.uint16),
                                  int4.pack_scales(so))


def test_lora_merged_weight_identity():
  # x W + (x A) B s == x (W + A B s)   (tunix/models/safetensors_saver.py:107-114,
  # tunix/tests/lora_params_test_base.py:349-397 use atol 1e-2)
  rng = np.random.default_rng(5)
  w = rng.standard_normal((128, 64)).astype(np.float32) * 0.05
  a = rng.standard_normal((128, 4)).astype(np.float32) * 0.05
  b = rng.standard_normal((4, 64)).astype(np.float32) * 0.05
  x = rng.standard_normal((3, 128)).astype(np.float32)
  lin = L.Linear(w=w, a=a, b=b, lora_scale=4.0)
  np.testing.assert_allclose(lin(x, F32), x @ lin.merged(), atol=1e-5)
  np.testing.assert_allclose(lin(x, F32, 'fused'), x @ lin.merged(), atol=1e-5)
  zero_b = L.Linear(w=w, a=a, b=np.zeros_like(b), lora_scale=4.0)
  np.testing.assert_array_equal(zero_b(x, F32), L.Linear(w=w)(x, F32))
  # quantised + bf16 rounding stays within the reference's own tolerance
  q, s = int4.quantize(bf16_round(w), 64)
  ql = L.Linear(q=q, scale=s, group=64, a=bf16_round(a), b=bf16_round(b), lora_scale=4.0)
  xb = bf16_round(x)
  np.testing.assert_allclose(ql(xb, BF16), xb @ ql.merged(), atol=5e-2)
  np.testing.assert_allclose(ql(xb, BF16, 'fused'), ql(xb, BF16), atol=3e-2)


def test_rmsnorm_closed_forms():
  rng = np.random.default_rng(6)
  x = rng.standard_normal((2, 3, 64)).astype(np.float32)
  w = rng.uniform(0.5, 1.5, 64).astype(np.float32)
  want = (w.astype(np.float64) * x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-5))
  np.testing.assert_allclose(L.rmsnorm_llama3(x, w, 1e-5, F32), want, rtol=2e-6, atol=2e-6)
  np.testing.assert_allclose(L.rmsnorm_qwen3(x, w, 1e-5, F32), want, rtol=2e-6, atol=2e-6)
  # unit weights: output rows have mean square 1 (eps = 0)
  np.testing.assert_allclose((L.rmsnorm_qwen3(x, np.ones(64, np.float32), 0.0, F32) ** 2).mean(-1), 1.0, rtol=1e-5)
  # bf16 policy: within half an ulp of the f32 result, and the two variants round differently
  xb, wb = bf16_round(x), bf16_round(w)
  a, b = L.rmsnorm_llama3(xb, wb, 1e-5, BF16), L.rmsnorm_qwen3(xb, wb, 1e-5, BF16)
  ref = L.rmsnorm_qwen3(xb, wb, 1e-5, F32)
  assert np.abs(b - ref).max() <= np.abs(ref).max() * 2.0 ** -8
  assert np.abs(a - ref).max() <= np.abs(ref).max() * 2.0 ** -7
  assert (a != b).any()


def test_rope_is_a_rotation_by_pos_over_timescale():
  rng = np.random.default_rng(7)
  h = 16
  x = rng.standard_normal((2, 5, 3, h))
  pos = np.array([[0, 1, 2, 3, 4], [7, 8, 9, 10, 11]])
  for theta, fn in ((1_000_000, lambda v: L.rope_llama3(v, pos, 1_000_000, F32)),
                    (10_000, lambda v: L.rope_qwen3(v, pos, 10_000, F32))):
    out = fn(x.astype(np.float32))
    z = x[..., : h // 2] + 1j * x[..., h // 2:]
    ang = pos[..., None, None] / theta ** (2 * np.arange(h // 2) / h)
    want = z * np.exp(1j * ang)
    np.testing.assert_allclose(out[..., : h // 2], want.real, atol=2e-5)
    np.testing.assert_allclose(out[..., h // 2:], want.imag, atol=2e-5)
    np.testing.assert_allclose(np.linalg.norm(out, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-5)
  # relative-position property: <rope(q, m), rope(k, n)> depends on m - n only
  q, k = rng.standard_normal((1, 1, 1, h)).astype(np.float32), rng.standard_normal((1, 1, 1, h)).astype(np.float32)
  dots = []
  for m, n in ((5, 2), (13, 10), (103, 100)):
    qm = L.rope_llama3(q, np.array([[m]]), 10_000, F32)
    kn = L.rope_llama3(k, np.array([[n]]), 10_000, F32)
    dots.append(float((qm * kn).sum()))
  assert max(dots) - min(dots) < 1e-4


def test_gqa_attention_brute_force_and_grouping():
  rng = np.random.default_rng(8)
  b, t, n, kh, h, s = 2, 1, 8, 2, 16, 12
  q = rng.standard_normal((b, t, n, h)).astype(np.float32)
  k = rng.standard_normal((b, s, kh, h)).astype(np.float32)
  v = rng.standard_normal((b, s, kh, h)).astype(np.float32)
  mask = rng.random((b, t, s)) < 0.7
  mask[..., 0] = True
  out = L.gqa_attention(q, k, v, mask, F32, 'fused')
  for bi in range(b):
    for head in range(n):
      kv = head // (n // kh)  # query heads are grouped consecutively per kv head
      sc = (k[bi, :, kv].astype(np.float64) @ q[bi, 0, head].astype(np.float64)) * h ** -0.5
      sc = np.where(mask[bi, 0], sc, -np.inf)
      p = np.exp(sc - sc.max())
      p /= p.sum()
      np.testing.assert_allclose(out[bi, 0, head], p @ v[bi, :, kv].astype(np.float64), atol=1e-5)
  # K_MASK semantics: a fully masked row is a uniform average over the WHOLE cache
  none = np.zeros((b, t, s), bool)
  np.testing.assert_allclose(L.gqa_attention(q, k, v, none, F32, 'fused')[0, 0, 0], v[0, :, 0].mean(0), atol=1e-5)
  # reference rounding differs from f32-internal by bf16 noise only
  qb, kb, vb = bf16_round(q), bf16_round(k), bf16_round(v)
  d = np.abs(L.gqa_attention(qb, kb, vb, mask, BF16) - L.gqa_attention(qb, kb, vb, mask, BF16, 'fused'))
  assert d.max() < 3e-2


def test_moe_routing_and_dense_equivalence():
  rng = np.random.default_rng(9)
  d, f, e, k = 32, 16, 8, 2
  x = rng.standard_normal((5, d)).astype(np.float32)
  rw = rng.standard_normal((d, e)).astype(np.float32)
  experts = [tuple(L.Linear(w=rng.standard_normal(s).astype(np.float32) * 0.1) for s in ((d, f), (d, f), (f, d)))
             for _ in range(e)]
  w, idx = L.moe_route(x, rw, k, F32)
  np.testing.assert_allclose(w.sum(-1), 1.0, rtol=1e-6)
  p = OS.softmax(x @ rw)
  for r in range(5):
    assert set(idx[r]) == set(np.argsort(-p[r])[:k])
  out, _ = L.moe_layer(x, rw, experts, k, F32)
  # dense restatement of tunix/models/qwen3/model.py:911-939: every expert evaluated, one-hot weights
  dense = np.zeros_like(x)
  for ei, (g, u, dn) in enumerate(experts):
    y = L.swiglu_mlp(x, g, u, dn, F32)
    dense += y * np.where(idx == ei, w, 0).sum(-1, keepdims=True)
  np.testing.assert_allclose(out, dense, atol=1e-5)


def test_log_softmax_and_top_p_rule():
  rng = np.random.default_rng(10)
  z = rng.standard_normal((3, 50)).astype(np.float32) * 3
  z64 = z.astype(np.float64)
  want = z64 - np.log(np.exp(z64 - z64.max(-1, keepdims=True)).sum(-1, keepdims=True)) - z64.max(-1, keepdims=True)
  np.testing.assert_allclose(OS.log_softmax(z), want, atol=2e-6)
  tok, lp = OS.sample_best(z)
  np.testing.assert_array_equal(tok, z.argmax(-1))
  np.testing.assert_allclose(lp, want[np.arange(3), tok], atol=2e-6)
  # ties: first index
  zt = np.zeros((1, 7), np.float32)
  assert OS.sample_best(zt)[0][0] == 0
  # nucleus: smallest prefix of the sorted distribution whose mass BEFORE the element is <= top_p
  for top_p in (0.1, 0.5, 0.9):
    members = OS.nucleus_members(z[0], top_p)
    order = np.argsort(-z64[0], kind='stable')
    probs = np.exp(want[0])[order]
    brute = {int(order[i]) for i in range(50) if probs[:i].sum() <= top_p + 1e-9}
    assert members == brute or len(members ^ brute) <= 1  # f32 cumsum vs f64 on the boundary element
  key = (np.uint32(0), np.uint32(3))
  for top_p in (0.3, 0.8):
    toks, lps = OS.sample_top_p(np.tile(z[:1], (200, 1)), key, 0.7, top_p)
    assert set(toks.tolist()) <= OS.nucleus_members(z[0] / np.float32(0.7), top_p)
    # logprob is of the temperature-scaled, NOT renormalised distribution
    np.testing.assert_allclose(lps, OS.log_softmax(z[:1] / np.float32(0.7))[0][toks], atol=1e-6)


def _cache_decode_equals_full_forward(cfg, lora_rank):
  st = C.make_state(cfg, 11, lora_rank, norm_jitter=0.1)
  dec = OM.Decoder(cfg, C.oracle_weights(cfg, st, 64, 8.0, lora_rank, quantized=False), F32)
  rng = np.random.default_rng(12)
  b, t, cs = 2, 6, 8
  toks = rng.integers(1, cfg.vocab_size, (b, t))
  in_mask = np.ones((b, t), bool)
  in_mask[1, :2] = False  # left padding
  pos = OMK.build_positions_from_mask(in_mask)
  full, _ = dec(toks, pos, None, OMK.make_causal_attn_mask(in_mask, t))
  cache = OM.init_cache(cfg, b, cs)
  full_mask = np.ones((b, cs), bool)
  full_mask[:, :t] = in_mask
  for step in range(t):
    m = OMK.compute_attention_masks(step, cs, ~full_mask)
    lg, cache = dec(toks[:, step:step + 1], pos[:, step:step + 1], cache, m)
    valid = in_mask[:, step]
    np.testing.assert_allclose(lg[valid, 0], full[valid, step], atol=2e-4)
    assert int(cache['layer_0']['end_index'][0]) == step + 1
  # prefill through the cache == the no-cache forward too
  cache2 = OM.init_cache(cfg, b, cs)
  pre, cache2 = dec(toks, pos, cache2, OMK.make_causal_attn_mask(in_mask, cs))
  np.testing.assert_allclose(pre[in_mask], full[in_mask], atol=2e-4)
  assert np.all(cache2['layer_0']['k'][:, :t][in_mask] != 0) and np.all(cache2['layer_0']['k'][:, t:] == 0)


def test_cache_decode_equals_full_forward_llama3():
  _cache_decode_equals_full_forward(OM.Config('llama3', 2, 64, 32, 64, 4, 8, 2, norm_eps=1e-5), 4)


def test_cache_decode_equals_full_forward_qwen3():
  _cache_decode_equals_full_forward(OM.Config('qwen3', 2, 64, 32, 64, 4, 8, 2, rope_theta=10_000, norm_eps=1e-6), 0)


def _hf_state_to_tunix(cfg, sd, qk_norm):
  """HF [out, in] -> tunix layouts (tunix/models/llama3/params.py:23-80,
  tunix/models/qwen3/params.py:47-121): transpose, then reshape to [D, N, H] / [N, H, D]."""
  d, n, kh, h = cfg.embed_dim, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim
  g = lambda k: sd[k].detach().numpy().astype(np.float32)
  st = {'embedder.input_embedding': g('model.embed_tokens.weight'), 'final_norm.w': g('model.norm.weight')}
  if not cfg.tied:
    st['lm_head.w'] = g('lm_head.weight').T.copy()
  for i in range(cfg.num_layers):
    p, hp = f'layers.{i}', f'model.layers.{i}'
    st[f'{p}.input_layernorm.w'] = g(f'{hp}.input_layernorm.weight')
    st[f'{p}.post_attention_layernorm.w'] = g(f'{hp}.post_attention_layernorm.weight')
    st[f'{p}.attn.q_proj.w'] = g(f'{hp}.self_attn.q_proj.weight').T.reshape(d, n, h)
    st[f'{p}.attn.k_proj.w'] = g(f'{hp}.self_attn.k_proj.weight').T.reshape(d, kh, h)
    st[f'{p}.attn.v_proj.w'] = g(f'{hp}.self_attn.v_proj.weight').T.reshape(d, kh, h)
    st[f'{p}.attn.o_proj.w'] = g(f'{hp}.self_attn.o_proj.weight').T.reshape(n, h, d)
    if qk_norm:
      st[f'{p}.attn.q_norm.w'] = g(f'{hp}.self_attn.q_norm.weight')
      st[f'{p}.attn.k_norm.w'] = g(f'{hp}.self_attn.k_norm.weight')
    for nm in ('gate_proj', 'up_proj', 'down_proj'):
      st[f'{p}.mlp.{nm}.kernel'] = g(f'{hp}.mlp.{nm}.weight').T.copy()
  return st


@pytest.mark.parametrize('family', ['llama3', 'qwen3'])
def test_dense_forward_matches_transformers(family):
  """The reference accepts HF as truth at 1e-3 (tests/model_alignment/qwen_align_test.py:110-201)."""
  import torch
  transformers = pytest.importorskip('transformers')
  torch.manual_seed(0)
  common = dict(vocab_size=128, hidden_size=64, intermediate_size=96, num_hidden_layers=2,
                num_attention_heads=4, num_key_value_heads=2, head_dim=16, max_position_embeddings=64,
                attention_bias=False, tie_word_embeddings=False)
  if family == 'llama3':
    # theta = 1e6: what the reference's Llama3 attention actually uses (llama3/model.py:356-365)
    hf_cfg = transformers.LlamaConfig(rms_norm_eps=1e-5, rope_theta=1_000_000.0, mlp_bias=False, **common)
    hf = transformers.LlamaForCausalLM(hf_cfg)
    cfg = OM.Config('llama3', 2, 128, 64, 96, 4, 16, 2, rope_theta=500_000, norm_eps=1e-5)
  else:
    hf_cfg = transformers.Qwen3Config(rms_norm_eps=1e-6, rope_theta=10_000.0, **common)
    hf = transformers.Qwen3ForCausalLM(hf_cfg)
    cfg = OM.Config('qwen3', 2, 128, 64, 96, 4, 16, 2, rope_theta=10_000, norm_eps=1e-6)
  hf = hf.float().eval()
  with torch.no_grad():
    for name, prm in hf.named_parameters():
      if 'norm' in name:
        prm.add_(0.1 * torch.randn_like(prm))
  st = _hf_state_to_tunix(cfg, hf.state_dict(), family == 'qwen3')
  dec = OM.Decoder(cfg, C.oracle_weights(cfg, st, 64, 0.0, 0, quantized=False), F32)
  toks = torch.randint(0, 128, (2, 9))
  with torch.no_grad():
    want = hf(toks).logits.numpy()
  pos = np.tile(np.arange(9), (2, 1))
  mask = OMK.make_causal_attn_mask(np.ones((2, 9), bool), 9)
  got, _ = dec(toks.numpy(), pos, None, mask)
  np.testing.assert_allclose(got, want, atol=1e-3)
  # and through the KV cache, token by token
  cache = OM.init_cache(cfg, 2, 12)
  for step in range(9):
    m = OMK.compute_attention_masks(step, 12, np.zeros((2, 12), bool))
    lg, cache = dec(toks.numpy()[:, step:step + 1], pos[:, step:step + 1], cache, m)
    np.testing.assert_allclose(lg[:, 0], want[:, step], atol=1e-3)


def test_moe_forward_matches_transformers():
  """The routed-expert layer (tunix/models/qwen3/model.py:894-939: f32 softmax over all experts,
  top-k, weights renormalised over the top-k, sum of weighted expert SwiGLU outputs) against
  transformers' Qwen3MoeForCausalLM with norm_topk_prob=True, random weights, fp32."""
  import torch
  transformers = pytest.importorskip('transformers')
  torch.manual_seed(1)
  e, topk, f = 8, 2, 32
  hf_cfg = transformers.Qwen3MoeConfig(
      vocab_size=128, hidden_size=64, intermediate_size=96, moe_intermediate_size=f, num_hidden_layers=2,
      num_attention_heads=4, num_key_value_heads=2, head_dim=16, max_position_embeddings=64, attention_bias=False,
      tie_word_embeddings=False, num_experts=e, num_experts_per_tok=topk, norm_topk_prob=True, decoder_sparse_step=1,
      mlp_only_layers=[], rms_norm_eps=1e-6, rope_theta=10_000.0)
  hf = transformers.Qwen3MoeForCausalLM(hf_cfg).float().eval()
  with torch.no_grad():
    for name, prm in hf.named_parameters():
      if 'norm' in name:
        prm.add_(0.1 * torch.randn_like(prm))
      if name.endswith('mlp.gate.weight'):
        prm.mul_(20.0)  # spread-out routing scores: top-k choices far from ties
      if 'experts' in name:
        prm.mul_(5.0)   # expert outputs large enough that a wrong routing weight or expert shows at 1e-3
  sd = hf.state_dict()
  cfg = OM.Config('qwen3', 2, 128, 64, f, 4, 16, 2, rope_theta=10_000, norm_eps=1e-6, num_experts=e, experts_per_tok=topk)
  g = lambda k: sd[k].detach().numpy().astype(np.float32)
  d, n, kh, h = cfg.embed_dim, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim
  st = {'embedder.input_embedding': g('model.embed_tokens.weight'), 'final_norm.w': g('model.norm.weight'),
        'lm_head.w': g('lm_head.weight').T.copy()}
  for i in range(cfg.num_layers):
    p, hp = f'layers.{i}', f'model.layers.{i}'
    st[f'{p}.input_layernorm.w'] = g(f'{hp}.input_layernorm.weight')
    st[f'{p}.post_attention_layernorm.w'] = g(f'{hp}.post_attention_layernorm.weight')
    st[f'{p}.attn.q_proj.w'] = g(f'{hp}.self_attn.q_proj.weight').T.reshape(d, n, h)
    st[f'{p}.attn.k_proj.w'] = g(f'{hp}.self_attn.k_proj.weight').T.reshape(d, kh, h)
    st[f'{p}.attn.v_proj.w'] = g(f'{hp}.self_attn.v_proj.weight').T.reshape(d, kh, h)
    st[f'{p}.attn.o_proj.w'] = g(f'{hp}.self_attn.o_proj.weight').T.reshape(n, h, d)
    st[f'{p}.attn.q_norm.w'] = g(f'{hp}.self_attn.q_norm.weight')
    st[f'{p}.attn.k_norm.w'] = g(f'{hp}.self_attn.k_norm.weight')
    st[f'{p}.mlp.router.kernel'] = g(f'{hp}.mlp.gate.weight').T.copy()                # [D, E]
    gu = g(f'{hp}.mlp.experts.gate_up_proj')                                           # [E, 2F, D]: gate rows, then up rows
    st[f'{p}.mlp.gate_proj'] = np.ascontiguousarray(gu[:, :f, :].transpose(0, 2, 1))  # [E, D, F]
    st[f'{p}.mlp.up_proj'] = np.ascontiguousarray(gu[:, f:, :].transpose(0, 2, 1))
    st[f'{p}.mlp.down_proj'] = np.ascontiguousarray(g(f'{hp}.mlp.experts.down_proj').transpose(0, 2, 1))  # [E, F, D]
  dec = OM.Decoder(cfg, C.oracle_weights(cfg, st, 64, 0.0, 0, quantized=False), F32)
  toks = torch.randint(0, 128, (2, 9))
  with torch.no_grad():
    out = hf(toks, output_router_logits=True)
  want = out.logits.numpy()
  pos = np.tile(np.arange(9), (2, 1))
  got, _ = dec(toks.numpy(), pos, None, OMK.make_causal_attn_mask(np.ones((2, 9), bool), 9))
  np.testing.assert_allclose(got, want, atol=1e-3)
  # the routing itself: the same experts per token as the library's top-k of its router logits
  for i, rl in enumerate(out.router_logits):
    hf_idx = np.sort(torch.topk(torch.softmax(rl.float(), -1), topk, dim=-1).indices.numpy(), axis=-1)
    np.testing.assert_array_equal(np.sort(np.asarray(dec.routed[i]).reshape(-1, topk), axis=-1), hf_idx)
  # a wrong renormalisation would show: without it the logits move by far more than the tolerance
  hf.config.norm_topk_prob = False
  for layer in hf.model.layers:
    layer.mlp.gate.norm_topk_prob = False
  with torch.no_grad():
    other = hf(toks).logits.numpy()
  assert np.abs(other - want).max() > 1e-2


def test_oracle_sampler_loop_invariants():
  cfg = OM.Config('llama3', 1, 64, 64, 64, 2, 32, 2)
  st = C.make_state(cfg, 13, 0)
  dec = OM.Decoder(cfg, C.oracle_weights(cfg, st, 64, 0.0, 0))
  from oracle import sampler as OSAM
  prompts = [np.array([5, 6, 7]), np.array([9, 10, 11, 12, 13])]
  out = OSAM.generate(dec, cfg, prompts, 6, 16, eos_ids=(-1,), max_prompt_length=8)
  assert all(len(t) == 6 for t in out['tokens']) and all(len(l) == 6 for l in out['logprobs'])
  # padded == unpadded outputs (tests/generate/sampler_test.py:95-147)
  solo = OSAM.generate(dec, cfg, prompts[:1], 6, 16, eos_ids=(-1,), max_prompt_length=3)
  margins = np.array(out['state'].margins)[:, 0]
  n = 6 if (margins > 1e-3).all() else int(np.argmax(margins <= 1e-3))
  np.testing.assert_array_equal(solo['tokens'][0][:n], out['tokens'][0][:n])
  # one generation step: the decode loop runs zero iterations (sampler_test.py:407-461)
  one = OSAM.generate(dec, cfg, prompts, 1, 16, eos_ids=(-1,))
  assert all(len(t) == 1 for t in one['tokens'])
  # eos truncation excludes the eos token
  eos = int(out['tokens'][0][2])
  cut = OSAM.generate(dec, cfg, prompts, 6, 16, eos_ids=(eos,), max_prompt_length=8)
  assert len(cut['tokens'][0]) <= 2 and eos not in cut['tokens'][0]
  # forbidden ids never appear (sampler_test.py:627-660)
  banned = [int(t) for t in out['tokens'][0][:2]]
  fb = OSAM.generate(dec, cfg, prompts, 6, 16, eos_ids=(-1,), forbidden=banned, temperature=1.0, top_p=1.0, seed=3)
  assert not (set(np.concatenate(fb['tokens']).tolist()) & set(banned))
  with pytest.raises(ValueError, match='must be less than the cache size'):
    OSAM.generate(dec, cfg, prompts, 20, 16, max_prompt_length=8)


def test_scoring_pass_reproduces_the_logprobs_of_generation():
  """oracle.scoring (full-sequence forward, no cache) against the sampler loop (prefill + cached
  decode): scoring the tokens a greedy rollout produced returns the log-probs it reported, and
  a hand-built 2-row case checks the gather / slicing convention of compute_per_token_logps
  (logit at position i scores token i + 1; completion slice only)."""
  from oracle import sampler as OSAM
  from oracle import scoring
  cfg = OM.Config('llama3', 2, 64, 64, 128, 2, 32, 2, rope_theta=10000, norm_eps=1e-5, tied=True)
  dec = OM.Decoder(cfg, OM.random_weights(cfg, 3, 64, 4, 8.0, ('q', 'v')))
  rng = np.random.default_rng(1)
  prompts = [rng.integers(3, 64, n) for n in (5, 3)]
  ref = OSAM.generate(dec, cfg, prompts, 6, 16, eos_ids=(-1,))
  comp = np.stack(ref['tokens'])
  got = scoring.per_token_logps(dec, ref['padded_prompt_tokens'], comp, 0)
  np.testing.assert_allclose(got, np.stack(ref['logprobs']), atol=2e-3)
  # slicing convention, by hand: one forward over the concatenation
  ids = np.concatenate([ref['padded_prompt_tokens'], comp], axis=1)
  valid = ids != 0
  logits, _ = dec(ids, OMK.build_positions_from_mask(valid), None, OMK.make_causal_attn_mask(valid, ids.shape[1]))
  lp = OS.log_softmax(logits)
  p = ref['padded_prompt_tokens'].shape[1]
  for b in range(2):
    for t in range(comp.shape[1]):
      # logit - logsumexp against the shifted log-softmax: equal up to f32 rounding
      assert abs(got[b, t] - lp[b, p + t - 1, comp[b, t]]) <= 2e-6


def test_selective_log_softmax_clips_like_the_reference():
  """tunix/rl/common.py:217-221: NaN -> -1e9, clip to [-1e9, 1e9], then logits[id] - logsumexp.
  Closed form: with one +1e9 entry the normaliser is 1e9, so that entry scores 0, a NaN or -inf
  entry -2e9 and a zero entry -1e9; without special values it is the plain log-softmax."""
  from oracle import scoring
  z = np.array([[np.nan, np.inf, 0.0, -np.inf, 3e9]], np.float32)
  ids = np.arange(5)[None, :]
  got = scoring.selective_log_softmax(np.repeat(z[:, None, :], 5, 1), ids)[0]
  # two entries sit at +1e9 (inf and 3e9): logsumexp = f32(1e9 + log 2) = 1e9 exactly
  np.testing.assert_array_equal(got, np.array([-2e9, 0.0, -1e9, -2e9, 0.0], np.float32))
  assert np.isfinite(got).all()
  rng = np.random.default_rng(0)
  x = rng.standard_normal((3, 4, 50)).astype(np.float32) * 5
  tok = rng.integers(0, 50, (3, 4))
  want = np.take_along_axis(OS.log_softmax(x), tok[..., None], -1)[..., 0]
  np.testing.assert_allclose(scoring.selective_log_softmax(x, tok), want, atol=4e-6)
  # logsumexp form, not the shifted one: 600 entries at the clip score 1e9 - f32(1e9 + log 600) = 0
  flat = scoring.selective_log_softmax(np.full((1, 600), 2e9, np.float32), np.array([5]))
  assert flat[0] == 0.0
