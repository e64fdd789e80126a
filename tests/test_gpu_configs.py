"""The other benchmark configurations at their real shapes, through the C ABI and the Sampler:
Llama-3.2-1B single sequence (d 2048, head_dim 64, tied 128 256-row head), Qwen3-8B at 128
sequences (group 128, rank 32, vocabulary 151 936, top-p 0.95) and the Qwen3-30B-A3B expert shape
(128 experts, top-8, expert MLP 768, d 2048, 32 sequences).

The CPU oracle cannot run these sizes in seconds, so the kernels are checked through inputs
with a closed-form answer (one-hot activations: a projection becomes a row lookup of the
bit-exactly dequantised matrix, the head a column lookup) and the whole path through two layers
of the real shape (reproducible, well formed, scoring pass == rollout log-probs).
"""
import numpy as np
import pytest
import torch

from oracle import prng
from oracle import sampling as OS
from tunix_amd import _lib
from tunix_amd import quant
from tunix_amd.configs import CacheConfig
from tunix_amd.model import ModelConfig, QLoRAModel
from tunix_amd.sampler import Sampler

import common as C
import gpu_util as G

pytestmark = pytest.mark.gpu


def S():
  return _lib.stream()


def _rb(t):
  return t.to(torch.bfloat16).float()


def _one_hot_rows(M, K, g, edge):
  ks = torch.randint(0, K, (M,), generator=g, device=G.DEV)
  amp = torch.ones(M, device=G.DEV)
  ks[0] = K - 1
  if M > 5:
    ks[1], ks[2] = 0, edge
    amp[3], amp[4], amp[5] = 2.0, -0.5, 0.0
  x = torch.zeros(M, K, dtype=torch.bfloat16, device=G.DEV)
  x[torch.arange(M), ks] = amp.to(torch.bfloat16)
  return x, ks, amp


def _dense_of(pl, K, N, group):
  dense = torch.empty(K, N, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_int4_dequant', S(), G.p(pl.qweight), G.p(pl.scales), G.p(dense), K, N, group)
  return dense


# (rows, K, N, group, rank): q|k|v, o, down of the 1B shape at one row; q|k|v, o, gate|up, down of Qwen3-8B at 128 rows
@pytest.mark.parametrize('M,K,N,group,r', [
    (1, 2048, 3072, 64, 16), (1, 2048, 2048, 64, 16), (1, 8192, 2048, 64, 16), (1, 2048, 16384, 64, 16),
    (128, 4096, 6144, 128, 32), (128, 4096, 4096, 128, 32), (128, 4096, 24576, 128, 32), (128, 12288, 4096, 128, 32),
    (32, 2048, 5120, 64, 8), (32, 4096, 2048, 64, 8),  # attention projections of the 30B-A3B shape (32 x 128 q, 4 kv heads)
])
def test_projection_of_one_hot_rows_at_config_shapes(M, K, N, group, r):
  g = torch.Generator(device=G.DEV).manual_seed(K + N + M)
  rnd = lambda *s: (torch.randn(*s, generator=g, device=G.DEV) * 0.02).to(torch.bfloat16)
  w, a, b = rnd(K, N), rnd(K, r), rnd(r, N)
  pl = quant.PackedLinear.from_dense([w], group, G.DEV, [(a, b)], 2.0)
  lib = _lib.lib()
  dense = _dense_of(pl, K, N, group)
  x, ks, amp = _one_hot_rows(M, K, g, 63)
  ws = torch.empty(lib.tmx_qlora_linear_workspace_bytes(M, K, N), dtype=torch.uint8, device=G.DEV)
  y = torch.empty(M, N, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_qlora_linear', S(), G.p(x), G.p(pl.qweight), G.p(pl.scales), None, None, None, G.p(y), G.p(ws),
         M, K, N, group, 0, 0, 0.0)
  G.sync()
  want = _rb(dense[ks].float() * amp[:, None])
  assert torch.equal(y.float(), want)
  G.call('tmx_qlora_linear', S(), G.p(x), G.p(pl.qweight), G.p(pl.scales), G.p(pl.lora_a_t), G.p(pl.lora_b),
         None, G.p(y), G.p(ws), M, K, N, group, r, pl.r_pad, 2.0)
  G.sync()
  t = _rb(a[ks].float() * amp[:, None])
  delta = _rb(_rb(t @ b.float()) * 2.0)
  G.assert_bf16_close(G.host(y), _rb(want + delta).cpu().numpy(), ulps=1.0, extra=G.ulp_bf16(delta.cpu().numpy()),
                      min_exact=0.99, what=f'one-hot {M}x{K}x{N}')


@pytest.mark.parametrize('M,K,F,group,r', [(1, 2048, 8192, 64, 16)])
def test_fused_gate_up_at_the_1b_shape(M, K, F, group, r):
  g = torch.Generator(device=G.DEV).manual_seed(77)
  rnd = lambda *s: (torch.randn(*s, generator=g, device=G.DEV) * 0.05).to(torch.bfloat16)
  ws = [rnd(K, F), rnd(K, F)]
  pl = quant.PackedLinear.from_dense(ws, group, G.DEV, None, 0.0)
  dense = _dense_of(pl, K, 2 * F, group)
  x, ks, _ = _one_hot_rows(M, K, g, 511)
  x *= 8
  act = torch.empty(M, F, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_qlora_gate_up_swiglu', S(), G.p(x), G.p(pl.qweight), G.p(pl.scales), None, None, G.p(act), M, K, F,
         group, 0, 0.0)
  G.sync()
  y = _rb(dense[ks].float() * 8.0)
  gte, up = y[:, :F], y[:, F:]
  sg = _rb(1.0 / (1.0 + torch.exp(-gte)))
  want = _rb(_rb(gte * sg) * up)
  G.assert_bf16_close(G.host(act), want.cpu().numpy(), ulps=1.0, min_exact=0.99, what='fused gate_up 1B')


@pytest.mark.parametrize('M,D,V', [(1, 2048, 128256), (128, 4096, 151936), (32, 2048, 151936)])
def test_head_at_config_vocabularies_is_a_column_lookup(M, D, V):
  g = torch.Generator(device=G.DEV).manual_seed(V + M)
  w = (torch.randn(V, D, generator=g, device=G.DEV) * 0.05).to(torch.bfloat16)
  ds = torch.randint(0, D, (M,), generator=g, device=G.DEV)
  x = torch.zeros(M, D, dtype=torch.bfloat16, device=G.DEV)
  x[torch.arange(M), ds] = 1.0
  lib = _lib.lib()
  ws = torch.empty(lib.tmx_head_sample_workspace_bytes(M, V), dtype=torch.uint8, device=G.DEV)
  tok = torch.full((M, 4), -1, dtype=torch.int32, device=G.DEV)
  lp = torch.zeros(M, 4, dtype=torch.float32, device=G.DEV)
  done = torch.zeros(M, dtype=torch.uint8, device=G.DEV)
  step = torch.tensor([1], dtype=torch.int32, device=G.DEV)
  eos = torch.tensor([-1], dtype=torch.int32, device=G.DEV)
  G.call('tmx_head_sample', S(), G.p(x), G.p(w), M, D, V, 0, 1.0, 0, 0, G.p(step), None, 0, G.p(eos), 1,
         G.p(tok), G.p(lp), G.p(done), 4, None, G.p(ws))
  G.sync()
  logits = w[:, ds].float().t().contiguous()
  mx = logits.max(dim=-1, keepdim=True).values
  first = (logits == mx).float().argmax(dim=-1)
  assert torch.equal(tok[:, 2].long(), first)
  want_lp = torch.log_softmax(logits.double(), dim=-1)[torch.arange(M), first].float()
  assert (lp[:, 2] - want_lp).abs().max().item() < 2e-4


def test_nucleus_at_128_rows_of_the_qwen3_vocabulary():
  """top-p 0.95 at 128 x 151 936 (temperature 1): one-hot hidden states make the logits an exact column of the
  head, so the oracle's sample_top_p runs on the very same values; rows whose cut or winner is not within
  rounding distance of a tie must agree token for token."""
  M, D, V, top_p, step = 128, 4096, 151936, 0.95, 3
  g = torch.Generator(device=G.DEV).manual_seed(21)
  # sharp rows (a nucleus of tens to thousands of candidates out of 151 936)
  w = (torch.randn(V, D, generator=g, device=G.DEV) * 2.5).to(torch.bfloat16)
  ds = torch.randint(0, D, (M,), generator=g, device=G.DEV)
  x = torch.zeros(M, D, dtype=torch.bfloat16, device=G.DEV)
  x[torch.arange(M), ds] = 1.0
  lib = _lib.lib()
  ws = torch.empty(lib.tmx_head_sample_workspace_bytes(M, V), dtype=torch.uint8, device=G.DEV)
  nb = lib.tmx_nucleus_workspace_bytes(M, V)
  assert nb > 0
  nws = torch.empty(nb, dtype=torch.uint8, device=G.DEV)
  tok = torch.full((M, 8), -5, dtype=torch.int32, device=G.DEV)
  lp = torch.zeros(M, 8, dtype=torch.float32, device=G.DEV)
  done = torch.zeros(M, dtype=torch.uint8, device=G.DEV)
  st = torch.tensor([step], dtype=torch.int32, device=G.DEV)
  eos = torch.tensor([-1], dtype=torch.int32, device=G.DEV)
  seed_key = prng.prng_key(9)
  G.call('tmx_head_sample_nucleus', S(), G.p(x), G.p(w), M, D, V, 1.0, top_p, 0, int(seed_key[0]), int(seed_key[1]),
         G.p(st), None, 0, G.p(eos), 1, G.p(tok), G.p(lp), G.p(done), 8, G.p(ws), G.p(nws), nb)
  G.sync()
  z = w[:, ds].float().t().contiguous().cpu().numpy()
  key = prng.fold_in(seed_key, step)
  want_tok, want_lp = OS.sample_top_p(z, key, 1.0, top_p, None)
  # Rows clear of rounding.  The running sum crosses top_p in steps of 1e-6 and is accumulated in another order
  # on the GPU, so the candidates within 1e-4 of the cut may fall on either side of it: a row is clear when its
  # winner is a candidate safely inside the nucleus and leads every other safe or borderline candidate by 1e-4.
  order = np.argsort(-z, axis=-1, kind='stable')
  zs = np.take_along_axis(z, order, axis=-1)
  ps = OS.softmax(zs)
  cs = np.cumsum(ps, axis=-1, dtype=np.float32)
  before = cs - ps
  safe = before <= np.float32(top_p) - np.float32(1e-4)
  maybe = before <= np.float32(top_p) + np.float32(1e-4)
  noisy = zs + prng.gumbel(key, zs.shape)
  srt = np.sort(np.where(maybe, noisy, -np.inf), axis=-1)
  win = np.argmax(np.where(maybe, noisy, -np.inf), axis=-1)
  clear = safe[np.arange(M), win] & (((srt[:, -1] - srt[:, -2]) > 1e-4) | ~np.isfinite(srt[:, -2]))
  assert clear.mean() > 0.6 and safe.sum(-1).max() > 50
  got = tok.cpu().numpy()[:, step + 1]
  np.testing.assert_array_equal(got[clear], want_tok[clear])
  full_lp = OS.log_softmax(z)
  np.testing.assert_allclose(lp.cpu().numpy()[:, step + 1], full_lp[np.arange(M), got], atol=5e-5)
  assert np.all(tok.cpu().numpy()[:, :step + 1] == -5)


def test_routed_experts_at_the_30b_a3b_shape():
  """tmx_moe_experts at 128 experts, top-8, d 2048, expert MLP 768, 32 rows: with one-hot hidden states the
  gate | up product of pair (token, expert) is a row of that expert's dequantised matrices, and with one-hot
  activations the down product is a row of its down matrix."""
  B, D, F, E, k, group = 32, 2048, 768, 128, 8, 64
  g = torch.Generator(device=G.DEV).manual_seed(30)
  rnd = lambda *s: (torch.randn(*s, generator=g, device=G.DEV) * 0.05).to(torch.bfloat16)
  gu = rnd(D, E * 2 * F)   # per expert: F gate columns then F up columns
  dn = rnd(F, E * D)
  pgu = quant.PackedLinear.from_dense([gu], group, G.DEV)
  pdn = quant.PackedLinear.from_dense([dn], group, G.DEV)
  dgu, ddn = _dense_of(pgu, D, E * 2 * F, group), _dense_of(pdn, F, E * D, group)
  rng = np.random.default_rng(3)
  idx = np.stack([rng.permutation(E)[:k] for _ in range(B)]).astype(np.int32)
  idx[:, 0] = 5  # one expert takes every row (32 rows of one expert), the others a few each
  P = B * k
  idx_t = torch.from_numpy(idx.reshape(-1)).to(G.DEV)
  x, ks, _ = _one_hot_rows(B, D, g, 255)
  x *= 8
  act = torch.full((P, F), 7.0, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_moe_experts', S(), G.p(x), D, G.p(pgu.qweight), G.p(pgu.scales), G.p(idx_t), P, k, E, D, 2 * F, group,
         0, G.p(act), F)
  G.sync()
  e_of = idx_t.long()
  tok_of = torch.arange(P, device=G.DEV) // k
  cols = e_of[:, None] * 2 * F + torch.arange(2 * F, device=G.DEV)[None, :]
  rows = _rb(dgu[ks[tok_of]].gather(1, cols).float() * x[tok_of, ks[tok_of]].float()[:, None])  # [P, 2F]
  gte, up = rows[:, :F], rows[:, F:]
  want = _rb(_rb(gte * _rb(1.0 / (1.0 + torch.exp(-gte)))) * up)
  G.assert_bf16_close(G.host(act), want.cpu().numpy(), ulps=1.0, min_exact=0.99, what='expert gate|up 30B-A3B')
  # down: one-hot activation rows per pair
  a1 = torch.zeros(P, F, dtype=torch.bfloat16, device=G.DEV)
  fs = torch.randint(0, F, (P,), generator=g, device=G.DEV)
  a1[torch.arange(P), fs] = 1.0
  y = torch.full((P, D), 7.0, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_moe_experts', S(), G.p(a1), F, G.p(pdn.qweight), G.p(pdn.scales), G.p(idx_t), P, k, E, F, D, group,
         1, G.p(y), D)
  G.sync()
  dcols = e_of[:, None] * D + torch.arange(D, device=G.DEV)[None, :]
  assert torch.equal(y.float(), ddn[fs].gather(1, dcols).float())


def _two_layer(cfg_full, **kw):
  cfg = ModelConfig(**{**cfg_full.__dict__, 'num_layers': 2})
  return cfg, QLoRAModel.random_init(cfg, seed=2, **kw)


def _well_formed(out, batch, steps, vocab):
  toks = np.stack(out.tokens)
  assert toks.shape == (batch, steps) and toks.min() >= 0 and toks.max() < vocab
  lps = np.stack([np.asarray(l) for l in out.logprobs])
  assert np.isfinite(lps).all() and (lps <= 0).all()
  return toks, lps


def test_llama32_1b_shape_single_sequence_rollout():
  """Two layers of the 1B shape, one sequence, temperature 1.0 with log-probs: reproducible, well formed, and the
  scoring pass over the sampled tokens returns the rollout's own log-probs (same kernels, one row)."""
  cfg, model = _two_layer(ModelConfig.llama3p2_1b(), group=64, lora_rank=16, lora_alpha=32.0)
  s = Sampler(model, C.ToyTokenizer(), CacheConfig(96, 2, cfg.num_kv_heads, cfg.head_dim))
  rng = np.random.default_rng(0)
  prompts = [rng.integers(3, cfg.vocab_size, 40)]
  kw = dict(prompt_token_ids=prompts, max_generation_steps=24, eos_tokens=[-1], temperature=1.0, top_p=1.0,
            return_logprobs=True)
  a, b, c = s(seed=5, **kw), s(seed=5, **kw), s(seed=6, **kw)
  toks, lps = _well_formed(a, 1, 24, cfg.vocab_size)
  assert (a.tokens[0] == b.tokens[0]).all() and (a.tokens[0] != c.tokens[0]).any()
  assert np.array_equal(np.asarray(a.logprobs[0]), np.asarray(b.logprobs[0]))
  scored = s.per_token_logps(a.padded_prompt_tokens, toks, pad_id=0, temperature=1.0)
  # scoring walks several tokens per pass through the block attention kernel, the rollout one token per step:
  # a hidden state may round the other way, which moves a bf16 logit of magnitude 2..4 by one ulp (2^-6)
  np.testing.assert_allclose(scored, lps, atol=2.0 ** -6 + 1e-2)


def test_qwen3_8b_shape_128_sequences_top_p_rollout():
  """Two layers of the Qwen3-8B shape (group 128, rank 32, QK-norm, vocabulary 151 936), 128 sequences, top-p 0.95."""
  cfg, model = _two_layer(ModelConfig.qwen3_8b(), group=128, lora_rank=32, lora_alpha=64.0)
  s = Sampler(model, C.ToyTokenizer(), CacheConfig(64, 2, cfg.num_kv_heads, cfg.head_dim))
  rng = np.random.default_rng(1)
  prompts = [rng.integers(3, cfg.vocab_size, 24) for _ in range(128)]
  kw = dict(prompt_token_ids=prompts, max_generation_steps=8, eos_tokens=[-1], temperature=1.0, top_p=0.95,
            return_logprobs=True)
  a, b = s(seed=3, **kw), s(seed=3, **kw)
  toks, lps = _well_formed(a, 128, 8, cfg.vocab_size)
  assert all((x == y).all() for x, y in zip(a.tokens, b.tokens))
  # greedy through the same model agrees with the largest log-prob the scoring pass finds for its own tokens
  gr = s(prompt_token_ids=prompts[:4], max_generation_steps=4, eos_tokens=[-1], return_logprobs=True)
  sc = s.per_token_logps(gr.padded_prompt_tokens, np.stack(gr.tokens), pad_id=0)
  # (one bf16 ulp of the winning logit, which lies in 4..8 here: 2^-5, see the 1B test)
  np.testing.assert_allclose(sc, np.stack([np.asarray(l) for l in gr.logprobs]), atol=2.0 ** -5 + 1e-2)


def test_qwen3_30b_a3b_shape_moe_rollout():
  """Two layers of the MoE shape (128 experts, top-8, expert MLP 768, d 2048, 32 / 4 heads, LoRA rank 8 on
  attention only), 32 sequences, temperature 0.9."""
  cfg, model = _two_layer(ModelConfig.qwen3_30b_a3b(), group=64, lora_rank=8, lora_alpha=16.0,
                          lora_targets=('q_proj', 'k_proj', 'v_proj', 'o_proj'))
  s = Sampler(model, C.ToyTokenizer(), CacheConfig(64, 2, cfg.num_kv_heads, cfg.head_dim))
  rng = np.random.default_rng(2)
  prompts = [rng.integers(3, cfg.vocab_size, 20) for _ in range(32)]
  kw = dict(prompt_token_ids=prompts, max_generation_steps=8, eos_tokens=[-1], temperature=0.9, top_p=1.0,
            return_logprobs=True)
  a, b = s(seed=3, **kw), s(seed=3, **kw)
  _well_formed(a, 32, 8, cfg.vocab_size)
  assert all((x == y).all() for x, y in zip(a.tokens, b.tokens))
