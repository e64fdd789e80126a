"""Size-independent properties at the benchmark's full shapes (Llama-3.1-8B rollout, 64 rows).

The CPU oracle cannot run these sizes in seconds, so each test picks inputs whose exact answer is
known in closed form: one-hot activations turn a projection into a row lookup of the bit-exactly
dequantised matrix, a zero query turns attention into a mean over the valid positions, one-hot
hidden states turn the vocabulary head into a column lookup.  All calls go through the C ABI.
"""
import numpy as np
import pytest
import torch

from tunix_amd import _lib
from tunix_amd import quant

import gpu_util as G

pytestmark = pytest.mark.gpu


def S():
  return _lib.stream()


def _bf16_round(t):
  return t.to(torch.bfloat16).float()


@pytest.mark.parametrize('K,N,group', [(4096, 6144, 64), (4096, 4096, 64), (4096, 28672, 64), (14336, 4096, 64),
                                       (4096, 24576, 128)])
def test_projection_of_one_hot_rows_is_a_row_lookup(K, N, group):
  M, r = 64, 16
  g = torch.Generator(device=G.DEV).manual_seed(K + N)
  rnd = lambda *s: (torch.randn(*s, generator=g, device=G.DEV) * 0.02).to(torch.bfloat16)
  w, a, b = rnd(K, N), rnd(K, r), rnd(r, N)
  pl = quant.PackedLinear.from_dense([w], group, G.DEV, [(a, b)], 2.0)
  lib = _lib.lib()
  dense = torch.empty(K, N, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_int4_dequant', S(), G.p(pl.qweight), G.p(pl.scales), G.p(dense), K, N, group)
  ks = torch.randint(0, K, (M,), generator=g, device=G.DEV)
  ks[0], ks[1], ks[2] = 0, K - 1, 63            # first / last row, tile edge
  amp = torch.ones(M, device=G.DEV)
  amp[3], amp[4], amp[5] = 2.0, -0.5, 0.0       # scaling, sign, an all-zero activation row
  x = torch.zeros(M, K, dtype=torch.bfloat16, device=G.DEV)
  x[torch.arange(M), ks] = amp.to(torch.bfloat16)
  ws = torch.empty(lib.tmx_qlora_linear_workspace_bytes(M, K, N), dtype=torch.uint8, device=G.DEV)
  y = torch.empty(M, N, dtype=torch.bfloat16, device=G.DEV)
  # base projection alone: exact
  G.call('tmx_qlora_linear', S(), G.p(x), G.p(pl.qweight), G.p(pl.scales), None, None, None, G.p(y), G.p(ws),
         M, K, N, group, 0, 0, 0.0)
  G.sync()
  want = _bf16_round(dense[ks].float() * amp[:, None])
  assert torch.equal(y.float(), want)
  # with LoRA: y = bf16(base + bf16(bf16(bf16(x A) B) * ls)); the r-term sum may round differently
  G.call('tmx_qlora_linear', S(), G.p(x), G.p(pl.qweight), G.p(pl.scales), G.p(pl.lora_a_t), G.p(pl.lora_b),
         None, G.p(y), G.p(ws), M, K, N, group, r, pl.r_pad, 2.0)
  G.sync()
  t = _bf16_round(a[ks].float() * amp[:, None])
  delta = _bf16_round(_bf16_round(t @ b.float()) * 2.0)
  want_l = _bf16_round(want + delta)
  G.assert_bf16_close(G.host(y), want_l.cpu().numpy(), ulps=1.0, extra=G.ulp_bf16(delta.cpu().numpy()),
                      min_exact=0.99, what=f'one-hot {K}x{N}')


@pytest.mark.parametrize('M,r,handover', [(64, 16, False), (64, 0, False), (17, 16, False),
                                          (64, 16, True), (33, 16, True), (17, 16, True)])
def test_fused_gate_up_of_one_hot_rows_is_swiglu_of_a_row_lookup(M, r, handover):
  """gate | up + LoRA + SwiGLU in one launch at the 8B shape (K = 4096, F = 14336): with one-hot
  activation rows the two projections are rows of the bit-exactly dequantised matrix, so the
  activation is known in closed form."""
  K, F, group = 4096, 14336, 64
  g = torch.Generator(device=G.DEV).manual_seed(31 + M + r)
  rnd = lambda *s: (torch.randn(*s, generator=g, device=G.DEV) * 0.05).to(torch.bfloat16)
  ws = [rnd(K, F), rnd(K, F)]
  loras = [(rnd(K, r), rnd(r, F)) for _ in range(2)] if r else None
  pl = quant.PackedLinear.from_dense(ws, group, G.DEV, loras, 2.0)
  dense = torch.empty(K, 2 * F, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_int4_dequant', S(), G.p(pl.qweight), G.p(pl.scales), G.p(dense), K, 2 * F, group)
  ks = torch.randint(0, K, (M,), generator=g, device=G.DEV)
  ks[0], ks[1], ks[2] = 0, K - 1, 511          # first / last row, step edge
  amp = torch.full((M,), 8.0, device=G.DEV)     # |g| around 1: the sigmoid is exercised
  amp[3], amp[4], amp[5] = -16.0, 0.5, 0.0
  x = torch.zeros(M, K, dtype=torch.bfloat16, device=G.DEV)
  x[torch.arange(M), ks] = amp.to(torch.bfloat16)
  act = torch.empty(M, F, dtype=torch.bfloat16, device=G.DEV)
  if handover:
    # the form the decode step runs: x . A once per launch by 16 (8 up to 32 rows) extra workgroups
    nb = _lib.lib().tmx_qlora_gate_up_swiglu_handover_bytes(M, K, F, r)
    assert nb > 0
    wsb = torch.empty(nb, dtype=torch.uint8, device=G.DEV)
    G.call('tmx_qlora_gate_up_swiglu_handover', S(), G.p(x), G.p(pl.qweight), G.p(pl.scales), G.p(pl.lora_a_t),
           G.p(pl.lora_b), G.p(act), G.p(wsb), M, K, F, group, r, 2.0)
    G.call('tmx_handover_status', S(), G.p(wsb))
  else:
    G.call('tmx_qlora_gate_up_swiglu', S(), G.p(x), G.p(pl.qweight), G.p(pl.scales), G.p(pl.lora_a_t), G.p(pl.lora_b),
           G.p(act), M, K, F, group, r, 2.0)
  G.sync()
  y = _bf16_round(dense[ks].float() * amp[:, None])            # [M, 2F], exact
  slack = torch.zeros_like(y)                                  # how far a last-bit flip of the LoRA sum can move y
  if r:
    for i, (a, b) in enumerate(loras):
      t = _bf16_round(a[ks].float() * amp[:, None])
      delta = _bf16_round(_bf16_round(t @ b.float()) * 2.0)
      base = y[:, i * F:(i + 1) * F].clone()
      y[:, i * F:(i + 1) * F] = _bf16_round(base + delta)
      ulp = lambda v: torch.exp2(torch.floor(torch.log2(v.abs().clamp(min=2.0 ** -120))) - 7)
      slack[:, i * F:(i + 1) * F] = torch.maximum(torch.maximum(ulp(base), ulp(delta)), ulp(y[:, i * F:(i + 1) * F]))
  gte, up = y[:, :F], y[:, F:]
  sg = _bf16_round(1.0 / (1.0 + torch.exp(-gte)))
  want = _bf16_round(_bf16_round(gte * sg) * up)
  if r == 0:
    # no rounding freedom except the sigmoid's last bit (expf vs torch.exp)
    G.assert_bf16_close(G.host(act), want.cpu().numpy(), ulps=1.0, min_exact=0.99, what='fused gate_up one-hot')
  else:
    # the r-term LoRA sum may round differently (f32 summation order): a last-bit flip of the delta
    # moves g or u by `slack`, and the product by |d act / d g| <= 1.1 |u|, |d act / d u| = |silu(g)|
    silu = (gte * sg).abs()
    extra = 1.5 * (1.1 * slack[:, :F] * up.abs() + slack[:, F:] * silu).cpu().numpy()
    G.assert_bf16_close(G.host(act), want.cpu().numpy(), ulps=2.0, extra=extra, min_exact=0.97,
                        what='fused gate_up + LoRA one-hot')


def test_attention_with_zero_query_is_the_mean_of_valid_values():
  B, N, Kh, H, C = 64, 32, 8, 128, 768
  g = torch.Generator(device=G.DEV).manual_seed(5)
  k = torch.randn(B, C, Kh, H, generator=g, device=G.DEV).to(torch.bfloat16)
  v = torch.randn(B, C, Kh, H, generator=g, device=G.DEV).to(torch.bfloat16)
  q = torch.zeros(B, N * H, dtype=torch.bfloat16, device=G.DEV)
  mask = torch.ones(B, C, dtype=torch.uint8, device=G.DEV)
  mask[1, :100] = 0                 # left padding
  mask[2, 5:700:7] = 0              # holes
  lib = _lib.lib()
  ws = torch.empty(max(lib.tmx_gqa_decode_workspace_bytes(B, N, Kh, H, C), 16), dtype=torch.uint8, device=G.DEV)
  out = torch.empty(B, N * H, dtype=torch.bfloat16, device=G.DEV)
  for step in (C - 1, 300, 0):
    st = torch.tensor([step], dtype=torch.int32, device=G.DEV)
    G.call('tmx_gqa_decode_attention', S(), G.p(q), G.p(k), G.p(v), G.p(mask), G.p(st), C, G.p(out), G.p(ws),
           B, N, Kh, H, C)
    G.sync()
    valid = mask[:, :step + 1].float()                                   # [B, S]
    cnt = valid.sum(1).clamp(min=1)
    mean = (v[:, :step + 1].float() * valid[:, :, None, None]).sum(1) / cnt[:, None, None]  # [B, Kh, H]
    want = mean[:, :, None, :].expand(B, Kh, N // Kh, H).reshape(B, N * H)
    got = out.float()
    rows = valid.sum(1) > 0
    err = (got - want).abs()[rows]
    assert err.max().item() <= 2.0 ** -8 * max(1.0, want.abs().max().item()), (step, err.max().item())


def test_head_of_one_hot_hidden_states_is_a_column_lookup():
  M, D, V = 64, 4096, 128256
  g = torch.Generator(device=G.DEV).manual_seed(9)
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
  logits = w[:, ds].float().t().contiguous()                  # [M, V]: column d of the head, exactly
  want_tok = torch.argmax(logits, dim=-1)                     # first index on ties (CPU and GPU alike)
  mx = logits.max(dim=-1, keepdim=True).values
  first = (logits == mx).float().argmax(dim=-1)
  assert torch.equal(tok[:, 2].long(), first)
  want_lp = torch.log_softmax(logits.double(), dim=-1)[torch.arange(M), first].float()
  assert (lp[:, 2] - want_lp).abs().max().item() < 2e-4
  assert (tok[:, 0] == -1).all() and (tok[:, 3] == -1).all()


def test_rollout_at_benchmark_shape_is_reproducible_and_well_formed():
  """Two layers of the 8B shape with the real vocabulary, 64 rows: the same seed gives the same
  tokens, rows that share a prompt draw different continuations, logprobs are proper."""
  from tunix_amd.configs import CacheConfig
  from tunix_amd.model import ModelConfig, QLoRAModel
  from tunix_amd.sampler import Sampler
  import common as C
  cfg = ModelConfig('llama3', 2, 128256, 4096, 14336, 32, 128, 8, 500_000, 1e-5, False)
  model = QLoRAModel.random_init(cfg, seed=1, group=64, lora_rank=16, lora_alpha=32.0)
  s = Sampler(model, C.ToyTokenizer(), CacheConfig(96, 2, 8, 128))
  rng = np.random.default_rng(0)
  base = rng.integers(3, cfg.vocab_size, (8, 64))
  prompts = [p for p in np.repeat(base, 8, axis=0)]
  kw = dict(prompt_token_ids=prompts, max_generation_steps=24, eos_tokens=[-1], temperature=0.9, top_p=1.0,
            return_logprobs=True)
  a = s(seed=11, **kw)
  b = s(seed=11, **kw)
  c = s(seed=12, **kw)
  assert all((x == y).all() for x, y in zip(a.tokens, b.tokens))
  assert any((x != y).any() for x, y in zip(a.tokens, c.tokens))
  toks = np.stack(a.tokens)
  assert toks.shape == (64, 24) and toks.min() >= 0 and toks.max() < cfg.vocab_size
  assert len({tuple(t) for t in toks[:8]}) > 1   # samples of one prompt differ
  lps = np.stack([np.asarray(l) for l in a.logprobs])
  assert np.isfinite(lps).all() and (lps <= 0).all()
