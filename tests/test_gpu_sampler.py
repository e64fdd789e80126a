"""End-to-end parity of the Sampler (decode loop on the GPU) against the oracle's restatement
of the reference Sampler, plus the behavioural properties the reference's own sampler tests
pin (tests/generate/sampler_test.py)."""
import numpy as np
import pytest
import torch

from oracle import masks as OMK
from oracle import model as OM
from oracle import prng
from oracle import sampler as OSAM
from oracle import sampling as OS
from oracle.bf16 import bf16_round
from tunix_amd.configs import CacheConfig, RolloutConfig
from tunix_amd.rollout import TmxRollout
from tunix_amd.sampler import Sampler

import common as C

pytestmark = pytest.mark.gpu

LOGIT_TOL = 2e-2
LOGPROB_TOL = 1e-2


def _pair(cfg, seed=0, rank=8, alpha=16.0, group=64, targets=('q_proj', 'k_proj', 'v_proj', 'o_proj')):
  st = C.make_state(cfg, seed, rank, targets=targets, norm_jitter=0.05)
  oracle = OM.Decoder(cfg, C.oracle_weights(cfg, st, group, alpha, rank))
  model = C.product_model(cfg, st, group, alpha)
  return oracle, model


def _sampler(model, cfg, cache_size):
  return Sampler(model, C.ToyTokenizer(), CacheConfig(cache_size, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim))


def _compare_greedy(out, ref, n_rows, min_checked, lp_extra=0.0, logit_ulps=0):
  """Tokens must agree wherever the oracle's top-2 margin exceeds the logit tolerance.  logit_ulps (needs
  keep_logits): logits are bf16 values, so where they are large enough for a bf16 ulp to exceed the
  tolerance, a last-bit flip of each of the two best logits is admitted on top of it."""
  margins = np.array(ref['state'].margins)  # [steps, B]
  tol = np.full_like(margins, LOGIT_TOL)
  if logit_ulps:
    top = np.stack([z.max(-1) for z in ref['state'].step_logits])
    tol = tol + logit_ulps * np.exp2(np.floor(np.log2(np.abs(top))) - 7)
  checked = 0
  for i in range(n_rows):
    got, want = out.tokens[i], ref['tokens'][i]
    assert len(got) == len(want)
    for s in range(len(want)):
      if got[s] != want[s]:
        assert margins[s, i] <= tol[s, i], (i, s, got[s], want[s], margins[s, i], tol[s, i])
        break  # after a near-tie the two sequences legitimately differ
      # log-prob = chosen logit - logsumexp, both made of bf16 logits: their last-bit flips carry over
      assert abs(out.logprobs[i][s] - ref['logprobs'][i][s]) <= LOGPROB_TOL + lp_extra + (tol[s, i] - LOGIT_TOL)
      checked += 1
  assert checked >= min_checked, checked
  return checked


def test_toy_config_greedy_matches_oracle():
  """The toy configuration of the benchmark description: 2 layers, d 256, 4 heads, SwiGLU 1024, vocab 1024, int4 g64, LoRA r8 on
  q/k/v/o, batch 4 x 32 prompt tokens, 32 greedy steps."""
  cfg = C.TOY
  oracle, model = _pair(cfg)
  rng = np.random.default_rng(0)
  prompts = [rng.integers(3, cfg.vocab_size, 32) for _ in range(4)]
  ref = OSAM.generate(oracle, cfg, prompts, 32, 64, eos_ids=(-1,))
  out = _sampler(model, cfg, 64)(prompt_token_ids=prompts, max_generation_steps=32, return_logprobs=True,
                                 eos_tokens=[-1])
  assert out.padded_prompt_tokens.shape == (4, 32)
  np.testing.assert_array_equal(out.prompt_lengths, [32] * 4)
  assert all(len(t) == 32 and len(l) == 32 for t, l in zip(out.tokens, out.logprobs))
  _compare_greedy(out, ref, 4, 40)


def test_streaming_copy_of_the_head_changes_nothing():
  """A rollout whose steps stream the head from its tile copy (the default) against one that reads the row-major
  matrix: tokens and log-probs are identical bit for bit, greedy and sampled (tied and untied heads)."""
  for tied in (False, True):
    cfg = OM.Config('llama3', 2, 1024, 256, 512, 4, 64, 2, rope_theta=10000, norm_eps=1e-5, tied=tied)
    rng = np.random.default_rng(3)
    prompts = [rng.integers(3, cfg.vocab_size, n) for n in (9, 14, 5)]
    outs = []
    for stream_head in (True, False):
      _, model = _pair(cfg, seed=41)
      model.stream_head = stream_head
      s = _sampler(model, cfg, 48)
      greedy = s(prompt_token_ids=prompts, max_generation_steps=12, return_logprobs=True, eos_tokens=[-1])
      sampled = s(prompt_token_ids=prompts, max_generation_steps=12, return_logprobs=True, eos_tokens=[-1],
                  temperature=0.8, top_p=1.0, seed=7)
      assert (model.desc().head_tiles is not None) == stream_head
      outs.append((greedy, sampled))
    for a, b in zip(outs[0], outs[1]):
      for ta, tb in zip(a.tokens, b.tokens):
        np.testing.assert_array_equal(ta, tb)
      for la, lb in zip(a.logprobs, b.logprobs):
        np.testing.assert_array_equal(np.asarray(la), np.asarray(lb))


def test_wide_layer_with_the_projection_side_lora_delta_matches_oracle():
  """One layer at the 8B width (d 4096, SwiGLU 14336, 32 / 8 heads of 128), LoRA r16 on every projection,
  6 sequences: the down projection is long enough (7 K-slices of 2048) for its own launch to finish the
  LoRA product, and the row kernel behind it adds that delta instead of multiplying by B.  Greedy tokens
  and log-probs against the oracle, as for the toy configuration."""
  from tunix_amd import _lib
  cfg = OM.Config('llama3', 1, 512, 4096, 14336, 32, 128, 8, norm_eps=1e-5)
  assert _lib.lib().tmx_qlora_linear_delta_workspace_bytes(6, 14336, 4096, 16, 32, _lib.lib().tmx_qlora_linear_num_splits(6, 14336, 4096)) > 0
  oracle, model = _pair(cfg, seed=21, rank=16, alpha=32.0,
                        targets=('q_proj', 'k_proj', 'v_proj', 'o_proj', 'gate_proj', 'up_proj', 'down_proj'))
  rng = np.random.default_rng(5)
  prompts = [rng.integers(3, cfg.vocab_size, 5) for _ in range(6)]
  ref = OSAM.generate(oracle, cfg, prompts, 5, 16, eos_ids=(-1,))
  out = _sampler(model, cfg, 16)(prompt_token_ids=prompts, max_generation_steps=5, return_logprobs=True, eos_tokens=[-1])
  # 4096-wide hidden states against a 0.02-std head give logits of a few units: one bf16 ulp of the chosen logit
  # (2^-6 .. 2^-5 there, against 2^-8 on the toy width) is the resolution of the log-prob itself
  _compare_greedy(out, ref, 6, 12, lp_extra=2.0 ** -5)


_WIDE = {}


def _wide_pair():
  """One 8B-width layer with LoRA r16 on all seven projections, built once for the tests that share it."""
  if not _WIDE:
    cfg = OM.Config('llama3', 1, 512, 4096, 14336, 32, 128, 8, norm_eps=1e-5)
    oracle, model = _pair(cfg, seed=22, rank=16, alpha=32.0,
                          targets=('q_proj', 'k_proj', 'v_proj', 'o_proj', 'gate_proj', 'up_proj', 'down_proj'))
    _WIDE.update(cfg=cfg, oracle=oracle, sampler=_sampler(model, cfg, 16))
  return _WIDE['cfg'], _WIDE['oracle'], _WIDE['sampler']


@pytest.mark.parametrize('n_seq', [33, 48, 64])
def test_wide_layer_at_33_to_64_sequences_matches_oracle(n_seq):
  """The 8B-width layer at 33, 48 and 64 sequences: the row counts at which the decode step runs the
  two-row-tile instantiations of its projection kernels, and the fused gate | up launch takes its LoRA
  projection from 16 producer workgroups (tunix/models/llama3/model.py:367-410, :489-496).  Ragged,
  left-padded prompts; greedy tokens and log-probs against the oracle."""
  cfg, oracle, s = _wide_pair()
  rng = np.random.default_rng(6 + n_seq)
  prompts = [rng.integers(3, cfg.vocab_size, 2 + i % 3) for i in range(n_seq)]
  ref = OSAM.generate(oracle, cfg, prompts, 3, 16, eos_ids=(-1,), keep_logits=True)
  out = s(prompt_token_ids=prompts, max_generation_steps=3, return_logprobs=True, eos_tokens=[-1])
  # 4096-wide hidden states against a 0.02-std head: the best logits lie in [4, 8), where one bf16 ulp is 2^-5.
  # log-prob = chosen logit - logsumexp: a last-bit flip of the chosen logit moves it by one such ulp, flips of the
  # few large logits that carry the log-sum-exp by up to another
  _compare_greedy(out, ref, n_seq, 3 * n_seq // 2, logit_ulps=2)
  if n_seq == 64:
    _WIDE.clear()  # frees the device copy of the layer


@pytest.mark.parametrize('family,n_seq,heads,kv_heads', [('llama3', 1, 8, 2), ('llama3', 3, 8, 2), ('llama3', 1, 32, 8),
                                                        ('qwen3', 1, 8, 2), ('qwen3', 4, 8, 4)])
def test_small_batch_attention_over_several_context_splits_matches_oracle(family, n_seq, heads, kv_heads):
  """One to four sequences with ~600-token left-padded prompts in a 768-slot cache: the small-batch step
  walks the context in 6 splits per kv head and merges them in the o projection's prologue
  (tunix/models/llama3/model.py:367-410 with the mask of tunix/generate/utils.py:35-59).  8 greedy steps
  against the oracle, log-probs included."""
  if family == 'llama3':
    cfg = OM.Config('llama3', 2, 512, 256, 512, heads, 64, kv_heads, norm_eps=1e-5)
  else:  # Qwen3: per-head q / k RMSNorm, bf16-rounded rotation, its own RMSNorm rounding (qwen3/model.py:432-484)
    cfg = OM.Config('qwen3', 2, 512, 256, 512, heads, 128, kv_heads, rope_theta=1_000_000, norm_eps=1e-6, tied=True)
  oracle, model = _pair(cfg, seed=23 + n_seq, rank=16, alpha=32.0,
                        targets=('q_proj', 'k_proj', 'v_proj', 'o_proj', 'gate_proj', 'up_proj', 'down_proj'))
  rng = np.random.default_rng(7 + n_seq)
  prompts = [rng.integers(3, 512, n) for n in (600, 437, 590, 512)[:n_seq]]
  ref = OSAM.generate(oracle, cfg, prompts, 8, 768, eos_ids=(-1,), keep_logits=True)
  out = _sampler(model, cfg, 768)(prompt_token_ids=prompts, max_generation_steps=8, return_logprobs=True,
                                  eos_tokens=[-1])
  np.testing.assert_array_equal(out.padded_prompt_tokens, ref['padded_prompt_tokens'])
  _compare_greedy(out, ref, n_seq, 5 * n_seq, logit_ulps=1)


def test_left_padded_ragged_prompts_and_all_lora_targets():
  cfg = OM.Config('llama3', 2, 512, 256, 512, 8, 64, 2, norm_eps=1e-5)  # GQA group of 4
  oracle, model = _pair(cfg, seed=3, rank=16, alpha=32.0,
                        targets=('q_proj', 'k_proj', 'v_proj', 'o_proj', 'gate_proj', 'up_proj', 'down_proj'))
  rng = np.random.default_rng(1)
  prompts = [rng.integers(3, 512, n) for n in (3, 7, 12, 16, 1)]
  ref = OSAM.generate(oracle, cfg, prompts, 12, 40, eos_ids=(-1,))
  out = _sampler(model, cfg, 40)(prompt_token_ids=prompts, max_generation_steps=12, return_logprobs=True,
                                 eos_tokens=[-1])
  np.testing.assert_array_equal(out.padded_prompt_tokens, ref['padded_prompt_tokens'])
  np.testing.assert_array_equal(out.prompt_lengths, [3, 7, 12, 16, 1])
  _compare_greedy(out, ref, 5, 25)


def test_qwen3_family_with_qk_norm_group128():
  cfg = OM.Config('qwen3', 2, 512, 256, 512, 4, 128, 2, rope_theta=1_000_000, norm_eps=1e-6, tied=True)
  oracle, model = _pair(cfg, seed=5, rank=8, alpha=8.0, group=128)
  rng = np.random.default_rng(2)
  prompts = [rng.integers(3, 512, n) for n in (9, 16)]
  ref = OSAM.generate(oracle, cfg, prompts, 10, 32, eos_ids=(-1,))
  out = _sampler(model, cfg, 32)(prompt_token_ids=prompts, max_generation_steps=10, return_logprobs=True,
                                 eos_tokens=[-1])
  _compare_greedy(out, ref, 2, 8)


def test_step_logits_within_tolerance_of_oracle():
  """Teacher-forced comparison: feed the ORACLE's tokens so both sides see the same context at
  every step, then compare the per-step logits (max abs 2e-2) and logprobs (1e-2)."""
  cfg = C.TOY
  oracle, model = _pair(cfg, seed=7)
  rng = np.random.default_rng(3)
  prompts = [rng.integers(3, cfg.vocab_size, 16) for _ in range(4)]
  ref = OSAM.generate(oracle, cfg, prompts, 8, 32, eos_ids=(-1,), keep_logits=True)
  s = _sampler(model, cfg, 32)
  s.eos_ids = np.array([-1])
  ids = ref['padded_prompt_tokens']
  st = s.init_sample_state(ids, 24, True, None, 0.0, None, None, 0, include_logprobs=True,
                           prompt_lengths=ref['prompt_lengths'])
  s.run_steps(st, 15, sample=False)
  for step in range(8):
    s.run_steps(st, 1, sample=True)
    logits = st['logits'].cpu().numpy()
    want = ref['state'].step_logits[step]
    assert np.abs(logits - want).max() <= LOGIT_TOL, (step, np.abs(logits - want).max())
    lp = st['logprobs'][:, 16 + step].cpu().numpy()
    # log-softmax of the oracle's logits at the oracle's token
    tok = ref['state'].token_buffer[:, 16 + step]
    want_lp = OS.log_softmax(want)[np.arange(4), tok]
    got_tok = st['token_buffer'][:, 16 + step].cpu().numpy()
    same = got_tok == tok
    assert np.abs(lp[same] - want_lp[same]).max() <= LOGPROB_TOL
    # teacher forcing: overwrite the sampled token with the oracle's
    st['token_buffer'][:, 16 + step] = torch.from_numpy(tok).to(st['token_buffer'].device)


def test_samples_of_one_prompt_share_its_cache_rows_and_match_oracle():
  """Three prompts x four samples in consecutive rows (the GRPO layout, tunix/rl/rl_learner.py:432-435):
  the Sampler finds the groups, decode attention reads the prompt slots once per group, and the per-step
  logits and log-probs still match the oracle, which attends over every sequence's own cache.  Teacher
  forcing with the oracle's SAMPLED tokens, so the rows of a group differ from the first generated token on."""
  cfg = OM.Config('llama3', 2, 512, 256, 512, 8, 64, 2, norm_eps=1e-5)
  oracle, model = _pair(cfg, seed=31, rank=8, alpha=16.0)
  rng = np.random.default_rng(11)
  base = [rng.integers(3, 512, n) for n in (70, 61, 66)]
  prompts = [base[i // 4] for i in range(12)]
  ref = OSAM.generate(oracle, cfg, prompts, 10, 96, eos_ids=(-1,), temperature=1.0, top_p=1.0, seed=5, keep_logits=True)
  toks = ref['state'].token_buffer
  ids = ref['padded_prompt_tokens']
  p = ids.shape[1]  # the padded prompt length: the first generated token lands in column p
  assert len({tuple(toks[i, p:p + 10]) for i in range(4)}) > 1   # the samples of a prompt do differ
  runs = {}
  for share in (True, False):
    s = _sampler(model, cfg, 96)
    s.share_prompt_kv = share
    s.eos_ids = np.array([-1])
    st = s.init_sample_state(ids, p + 10, True, None, 0.0, None, None, 0, include_logprobs=True,
                             prompt_lengths=ref['prompt_lengths'])
    assert (st['share_group'], st['share_len'], st['share_common']) == ((4, p // 32 * 32, p) if share else (1, 0, 0))
    s.walk(st, p - 1)
    steps = []
    for step in range(10):
      s.run_steps(st, 1, sample=True)
      logits = st['logits'].cpu().numpy()
      want = ref['state'].step_logits[step]
      assert np.abs(logits - want).max() <= LOGIT_TOL, (share, step, np.abs(logits - want).max())
      steps.append(logits)
      tok = toks[:, p + step]
      st['token_buffer'][:, p + step] = torch.from_numpy(tok).to(st['token_buffer'].device)
    s.check_device_status(st)
    runs[share] = np.stack(steps)
  # shared and unshared walks: the same softmax over the same positions, only the order of the f32 sums differs
  assert np.abs(runs[True] - runs[False]).max() <= 1e-2


def test_temperature_sampling_follows_the_threefry_schedule():
  """Every generated token equals categorical(fold_in(PRNGKey(seed), decoding_step), logits / T)
  evaluated on the kernel's own logits, with decoding_step = P - 1, P, ... as in the reference
  (tunix/generate/sampler.py:562, :493), and its logprob is log_softmax(logits / T)[token]."""
  cfg = C.TOY
  _, model = _pair(cfg, seed=9)
  rng = np.random.default_rng(4)
  prompts = [rng.integers(3, cfg.vocab_size, 8) for _ in range(4)]
  s = _sampler(model, cfg, 32)
  out = s(prompt_token_ids=prompts, max_generation_steps=10, return_logprobs=True, return_logits=True,
          eos_tokens=[-1], temperature=0.9, top_p=1.0, seed=42)
  key0 = prng.prng_key(42)
  agree = total = 0
  for step in range(10):
    z = np.stack([out.logits[b][step] for b in range(4)]).astype(np.float32) / np.float32(0.9)
    noisy = z + prng.gumbel(prng.fold_in(key0, 8 - 1 + step), z.shape)
    srt = np.sort(noisy, axis=-1)
    clear = (srt[:, -1] - srt[:, -2]) > 1e-4
    got = np.array([out.tokens[b][step] for b in range(4)])
    np.testing.assert_array_equal(got[clear], np.argmax(noisy, -1)[clear])
    agree += clear.sum()
    total += 4
    want_lp = OS.log_softmax(z)[np.arange(4), got]
    np.testing.assert_allclose([out.logprobs[b][step] for b in range(4)], want_lp, atol=3e-5)
  assert agree >= total - 2
  # a different seed changes the text (tests/generate/sampler_test.py:285-316)
  out2 = s(prompt_token_ids=prompts, max_generation_steps=10, eos_tokens=[-1], temperature=0.9, top_p=1.0, seed=43)
  assert any((a != b).any() for a, b in zip(out.tokens, out2.tokens))
  # same seed: identical
  out3 = s(prompt_token_ids=prompts, max_generation_steps=10, eos_tokens=[-1], temperature=0.9, top_p=1.0, seed=42)
  assert all((a == b).all() for a, b in zip(out.tokens, out3.tokens))


def test_batches_over_128_sequences():
  """More than 128 sequences per step: the projections run in 256-row blocks, the head takes the
  rows 64 at a time.  Greedy rows spread over the batch against the oracle (a sequence does not
  depend on its neighbours), temperature sampling against the threefry schedule over all rows
  (the noise counter is row * V + v), top-p through the sorting branch."""
  cfg = C.TOY
  oracle, model = _pair(cfg, seed=11, targets=('q_proj', 'k_proj', 'v_proj', 'o_proj', 'gate_proj', 'up_proj', 'down_proj'))
  rng = np.random.default_rng(6)
  nb = 150
  prompts = [rng.integers(3, cfg.vocab_size, 3 + (i * 7) % 10) for i in range(nb)]
  s = _sampler(model, cfg, 32)
  out = s(prompt_token_ids=prompts, max_generation_steps=8, return_logprobs=True, eos_tokens=[-1])
  assert len(out.tokens) == nb
  rows = [0, 31, 63, 64, 100, 127, 128, 129, 149]
  ref = OSAM.generate(oracle, cfg, [prompts[i] for i in rows], 8, 32, eos_ids=(-1,))
  class _Sub:
    tokens = [out.tokens[i] for i in rows]
    logprobs = [out.logprobs[i] for i in rows]
  _compare_greedy(_Sub, ref, len(rows), 40)
  # temperature sampling: every row follows categorical(fold_in(key, step), logits / T) on its own logits
  prompts8 = [rng.integers(3, cfg.vocab_size, 8) for _ in range(nb)]  # equal lengths: one decoding step index
  out = s(prompt_token_ids=prompts8, max_generation_steps=4, return_logprobs=True, return_logits=True,
          eos_tokens=[-1], temperature=0.9, top_p=1.0, seed=7)
  key0 = prng.prng_key(7)
  agree = total = 0
  for step in range(4):
    z = np.stack([out.logits[b][step] for b in range(nb)]).astype(np.float32) / np.float32(0.9)
    noisy = z + prng.gumbel(prng.fold_in(key0, 8 - 1 + step), z.shape)
    srt = np.sort(noisy, axis=-1)
    clear = (srt[:, -1] - srt[:, -2]) > 1e-4
    got = np.array([out.tokens[b][step] for b in range(nb)])
    np.testing.assert_array_equal(got[clear], np.argmax(noisy, -1)[clear])
    agree += clear.sum()
    total += nb
    want_lp = OS.log_softmax(z)[np.arange(nb), got]
    np.testing.assert_allclose([out.logprobs[b][step] for b in range(nb)], want_lp, atol=3e-5)
  assert agree >= total - 8
  # without the logits output the 256 x 256 head kernel samples: same seed, same noise, logits equal up to
  # the f32 summation order, so the tokens agree except at near-ties (after which a row goes its own way)
  out_w = s(prompt_token_ids=prompts8, max_generation_steps=4, return_logprobs=True, eos_tokens=[-1],
            temperature=0.9, top_p=1.0, seed=7)
  same = sum(int((np.asarray(out_w.tokens[b]) == np.asarray(out.tokens[b])).all()) for b in range(nb))
  assert same >= nb - 3, same
  first = np.array([out_w.logprobs[b][0] for b in range(nb)]) - np.array([out.logprobs[b][0] for b in range(nb)])
  assert np.abs(first).max() <= LOGPROB_TOL
  # the sorting branch (top-p < 1): tokens come from the nucleus of the row's own logits
  out = s(prompt_token_ids=prompts8, max_generation_steps=3, return_logits=True, eos_tokens=[-1],
          temperature=1.0, top_p=0.5, seed=3)
  for b in (0, 64, 128, 149):
    for step in range(3):
      members = OS.nucleus_members(np.asarray(out.logits[b][step], np.float32), 0.5)
      assert out.tokens[b][step] in members, (b, step)


def test_top_p_and_top_k_sampling_follow_the_reference_rule():
  """The sorting branch of sample_top_p (tunix/generate/sampler.py:136-153) through the whole
  Sampler: every token equals the oracle's draw on the kernel's own logits of that step."""
  cfg = C.TOY
  _, model = _pair(cfg, seed=21)
  rng = np.random.default_rng(8)
  prompts = [rng.integers(3, cfg.vocab_size, 8) for _ in range(4)]
  s = _sampler(model, cfg, 32)
  for top_p, top_k in ((0.6, None), (1.0, 20), (0.9, 64)):
    out = s(prompt_token_ids=prompts, max_generation_steps=8, return_logprobs=True, return_logits=True,
            eos_tokens=[-1], temperature=0.8, top_p=top_p, top_k=top_k, seed=7)
    key0 = prng.prng_key(7)
    agree = 0
    for step in range(8):
      logits = np.stack([out.logits[b][step] for b in range(4)]).astype(np.float32)
      want, want_lp = OS.sample_top_p(logits, prng.fold_in(key0, 8 - 1 + step), 0.8, top_p, top_k)
      got = np.array([out.tokens[b][step] for b in range(4)])
      agree += (got == want).sum()
      z = logits / np.float32(0.8)
      np.testing.assert_allclose([out.logprobs[b][step] for b in range(4)],
                                 OS.log_softmax(z)[np.arange(4), got], atol=3e-5)
      for b in range(4):
        members = OS.nucleus_members(z[b], top_p)
        if top_k:
          members &= set(np.argsort(-z[b], kind='stable')[:top_k].tolist())
        assert int(got[b]) in members or agree < 0
    assert agree >= 30, agree  # 32 draws; a draw may flip on an f32 near-tie


def test_sampler_behavioural_properties():
  cfg = C.TOY
  oracle, model = _pair(cfg, seed=11)
  s = _sampler(model, cfg, 64)
  rng = np.random.default_rng(5)
  p_short, p_long = rng.integers(3, 1024, 5), rng.integers(3, 1024, 11)
  # padded == unpadded outputs (sampler_test.py:95-147), up to near-ties
  both = s(prompt_token_ids=[p_short, p_long], max_generation_steps=8, max_prompt_length=16, eos_tokens=[-1],
           return_logits=True)
  solo = s(prompt_token_ids=[p_short], max_generation_steps=8, eos_tokens=[-1])
  for k in range(8):
    if both.tokens[0][k] != solo.tokens[0][k]:
      lg = np.sort(both.logits[0][k])
      assert lg[-1] - lg[-2] <= LOGIT_TOL
      break
  # logprobs length == tokens length (sampler_test.py:318-371); one generation step (:407-461)
  one = s(prompt_token_ids=[p_short, p_long], max_generation_steps=1, return_logprobs=True, eos_tokens=[-1])
  assert [len(t) for t in one.tokens] == [1, 1] and [len(l) for l in one.logprobs] == [1, 1]
  np.testing.assert_array_equal(one.tokens[1], both.tokens[1][:1])
  # eos truncation: the first generated token of row 0 as eos -> empty output for that row
  eos = int(both.tokens[0][0])
  cut = s(prompt_token_ids=[p_short, p_long], max_generation_steps=8, max_prompt_length=16, eos_tokens=[eos],
          return_logprobs=True)
  assert len(cut.tokens[0]) == 0 and len(cut.logprobs[0]) == 0 and eos not in cut.tokens[1]
  # echo and pad_output
  echo = s(prompt_token_ids=[p_short, p_long], max_generation_steps=4, max_prompt_length=16, eos_tokens=[-1],
           echo=True, pad_output=True)
  assert echo.tokens.shape == (2, 20)
  np.testing.assert_array_equal(echo.tokens[0][:5], p_short)
  np.testing.assert_array_equal(echo.tokens[1][:11], p_long)
  # forbidden tokens never sampled over 100 steps (sampler_test.py:627-660)
  s100 = _sampler(model, cfg, 128)
  banned = list(range(0, 1024, 2))
  fb = s100(prompt_token_ids=[p_short] * 4, max_generation_steps=100, eos_tokens=[-1], temperature=1.0, top_p=1.0,
            seed=1, forbidden_tokens=banned)
  assert all((t % 2 == 1).all() and len(t) == 100 for t in fb.tokens)
  # strings in, strings out
  txt = s(input_strings=['5 6 7', '9 10'], max_generation_steps=3, eos_tokens=[-1])
  assert len(txt.text) == 2 and all(len(t.split()) == 3 for t in txt.text)
  np.testing.assert_array_equal(txt.prompt_lengths, [4, 3])  # bos + tokens


def test_lora_update_params_and_rollout_surface():
  cfg = C.TOY
  st = C.make_state(cfg, 13, 8)
  model = C.product_model(cfg, st, 64, 16.0)
  base_state = {k: v for k, v in st.items() if 'lora' not in k}
  base = C.product_model(cfg, base_state, 64, 0.0)
  rng = np.random.default_rng(6)
  prompts = [rng.integers(3, 1024, 8) for _ in range(2)]
  kw = dict(prompt_token_ids=prompts, max_generation_steps=6, eos_tokens=[-1], return_logits=True)
  s = _sampler(model, cfg, 32)
  with_lora = s(**kw)
  no_lora = _sampler(base, cfg, 32)(**kw)
  assert np.abs(with_lora.logits[0][0] - no_lora.logits[0][0]).max() > 1e-3
  # B = 0 (a freshly initialised adapter, sampler_test.py:525-529) == the base model, bit for bit
  old = {k: v.clone() for k, v in s.transformer_state.items()}
  zeroed = {k: (torch.zeros_like(v) if k.endswith('_lora_b') else v) for k, v in old.items()}
  s.transformer_state = zeroed
  z = s(**kw)
  np.testing.assert_array_equal(z.logits[0][0], no_lora.logits[0][0])
  # LoRA-only sync through update_params restores the adapter exactly (f32 -> bf16 cast included)
  s.update_params({k: v.float() for k, v in old.items()})
  back = s(**kw)
  np.testing.assert_array_equal(back.logits[1][2], with_lora.logits[1][2])
  with pytest.raises(ValueError, match='same structure'):
    s.transformer_state = {k: v for k, v in list(old.items())[:-1]}
  with pytest.raises(ValueError, match='same shape'):
    bad = dict(old)
    k0 = next(iter(bad))
    bad[k0] = torch.zeros(3, 3)
    s.transformer_state = bad
  # rollout plugin surface
  r = TmxRollout(rollout_actor=model, tokenizer=C.ToyTokenizer(), mesh=None,
                 rollout_config=RolloutConfig(kv_cache_size=32))
  ro = r.generate(None, RolloutConfig(max_tokens_to_generate=5, max_prompt_length=8, temperature=0.9, top_p=1.0,
                                      eos_tokens=[-1], return_logprobs=True, seed=3), prompt_token_ids=prompts)
  assert len(ro.tokens) == 2 and all(len(t) == 5 for t in ro.tokens) and len(ro.logprobs[0]) == 5
  assert ro.left_padded_prompt_tokens.shape == (2, 8)


def test_unsupported_sampling_modes_fail_loudly():
  cfg = C.TOY
  _, model = _pair(cfg, seed=15)
  s = _sampler(model, cfg, 32)
  with pytest.raises(NotImplementedError):
    s(input_strings=['5 6'], max_generation_steps=2, beam_size=2)


def test_device_status_reports_a_wait_that_ran_out():
  """tmx_decode_status: clean after a rollout; a set status word (written here from the host, no
  kernel is made to wait) is reported once as TMX_ERR_DEVICE_WAIT and cleared."""
  from tunix_amd import _lib
  cfg = C.TOY
  _, model = _pair(cfg, seed=16)
  s = _sampler(model, cfg, 32)
  s(input_strings=['5 6 7'], max_generation_steps=4)  # checks the status itself before returning
  st = s.init_sample_state(np.array([[5, 6, 7]], np.int32), 8, False, None, 1.0, 1.0, None, 0, include_logprobs=False)
  s.run_steps(st, 2, sample=False)
  s.check_device_status(st)
  s._workspace[:4] = torch.tensor([1, 0, 0, 0], dtype=torch.uint8, device=s._workspace.device)
  with pytest.raises(_lib.TmxError, match='bounded wait'):
    s.check_device_status(st)
  s.check_device_status(st)  # cleared by the failing check


def test_moe_decoder_matches_oracle():
  """Qwen3-MoE-shaped toy (8 experts, top-2, QK-norm): greedy tokens and step logits against
  the oracle's routed-pair restatement of MoELayer (tunix/models/qwen3/model.py:894-939)."""
  cfg = OM.Config('qwen3', 2, 1024, 256, 256, 4, 64, 2, rope_theta=1_000_000, norm_eps=1e-6, tied=False,
                  num_experts=8, experts_per_tok=2)
  st = C.make_state(cfg, 31, 8, norm_jitter=0.05)
  oracle = OM.Decoder(cfg, C.oracle_weights(cfg, st, 64, 16.0, 8))
  model = C.product_model(cfg, st, 64, 16.0)
  rng = np.random.default_rng(12)
  prompts = [rng.integers(3, cfg.vocab_size, n) for n in (6, 9, 4, 9)]
  ref = OSAM.generate(oracle, cfg, prompts, 10, 32, eos_ids=(-1,))
  s = _sampler(model, cfg, 32)
  out = s(prompt_token_ids=prompts, max_generation_steps=10, eos_tokens=[-1], return_logprobs=True)
  # logits of this model reach |z| in [1, 2): one bf16 ulp of the chosen token's logit (2^-7, from
  # another f32 summation order) moves its logprob by as much, on top of the 1e-2 budget
  _compare_greedy(out, ref, 4, min_checked=20, lp_extra=2.0 ** -7)


@pytest.mark.parametrize('nseq,top_p,group', [(4, 1.0, 1), (150, 1.0, 1), (6, 0.8, 1), (70, 0.9, 1), (16, 1.0, 4),
                                               (16, 1.0, 8)])
def test_graph_replay_matches_plain_launches_on_every_replay(nseq, top_p, group):
  """tmx_decode_steps_graph against tmx_decode_steps: several graph calls in a row, with the
  program's own eager work (a plain step, host reads) and synchronisation between them; every
  call's tokens, logprobs, KV cache and step counter equal the plain launches'.  4 sequences: the
  small-batch launches; 150: the many-rows kernels; top_p < 1: the selection launches of the
  top-p branch (6 sequences behind the 64-row head and the gate|up hand-over, 70 behind the head in
  256 x 256 blocks) are recorded and replayed.  group > 1: four rows per 40-token prompt on a model with
  that many query heads per KV head, so the recorded attention launches are the ones that read the common
  prompt slots once per group of rows (vector walk plus merge for 4 heads per KV head, the walk on the
  matrix pipe for 8)."""
  cfg = C.TOY if group == 1 else OM.Config('llama3', 2, 1024, 256, 1024, 8, 64, 8 // group, rope_theta=10000,
                                           norm_eps=1e-5, tied=False)
  _, model = _pair(cfg, seed=17, targets=('q_proj', 'k_proj', 'v_proj', 'o_proj', 'gate_proj', 'up_proj', 'down_proj'))
  rng = np.random.default_rng(2)
  plen = 8 if group == 1 else 40
  rows = 1 if group == 1 else 4
  base = [rng.integers(3, cfg.vocab_size, plen) for _ in range(nseq // rows)]
  ids = np.stack([base[i // rows] for i in range(nseq)]).astype(np.int32)
  def run(graph):
    s = _sampler(model, cfg, plen + 56)
    s.eos_ids = np.array([-1])
    st = s.init_sample_state(ids, plen + 56, False, None, 0.9, top_p, None, 5, include_logprobs=True,
                             prompt_lengths=np.full(nseq, plen))
    assert st['share_group'] == rows
    snaps = []
    s.run_steps(st, plen - 1, sample=False, graph=graph)
    for n in (9, 1, 12, 5, 16):
      s.run_steps(st, n, sample=True, graph=graph)
      torch.cuda.synchronize()
      snaps.append((st['token_buffer'].cpu().numpy().copy(), st['logprobs'].cpu().numpy().copy(),
                    int(st['step'].item()), st['cache'].float().abs().sum().item()))
      s.run_steps(st, 1, sample=True, graph=False)   # eager work between the replays
      _ = st['done'].cpu()
    return snaps
  plain, replay = run(False), run(True)
  for (t0, l0, s0, c0), (t1, l1, s1, c1) in zip(plain, replay):
    assert s0 == s1
    np.testing.assert_array_equal(t0, t1)
    np.testing.assert_array_equal(l0, l1)
    assert c0 == c1


def test_per_token_logps_match_oracle_and_the_rollout_logprobs():
  """Scoring pass of the rollout adapter (tunix/rl/common.py:426-606): left-padded prompts,
  right-padded completions; against the oracle's full-sequence forward, and against the
  log-probs the Sampler itself reported when it generated the same tokens at T = 1."""
  from oracle import scoring
  cfg = C.TOY
  oracle, model = _pair(cfg, seed=23)
  s = _sampler(model, cfg, 48)
  rng = np.random.default_rng(9)
  pad = 0
  prompt = np.full((4, 10), pad, np.int32)
  comp = np.full((4, 12), pad, np.int32)
  for b, (pl, cl) in enumerate(((10, 12), (7, 9), (3, 12), (10, 1))):
    prompt[b, 10 - pl:] = rng.integers(3, cfg.vocab_size, pl)
    comp[b, :cl] = rng.integers(3, cfg.vocab_size, cl)
  got = s.per_token_logps(prompt, comp, pad_id=pad)
  want = scoring.per_token_logps(oracle, prompt, comp, pad)
  valid = comp != pad
  assert got.shape == (4, 12)
  assert np.abs(got - want)[valid].max() <= LOGPROB_TOL, np.abs(got - want)[valid].max()
  # temperature scaling
  got_t = s.per_token_logps(prompt, comp, pad_id=pad, temperature=0.7)
  want_t = scoring.per_token_logps(oracle, prompt, comp, pad, temperature=0.7)
  assert np.abs(got_t - want_t)[valid].max() <= 2 * LOGPROB_TOL
  # the rollout's own log-probs: generate at T = 1, then score the generated tokens
  r = TmxRollout(rollout_actor=model, tokenizer=C.ToyTokenizer(), mesh=None,
                 rollout_config=RolloutConfig(kv_cache_size=48))
  prompts = [prompt[b, prompt[b] != pad] for b in range(4)]
  ro = r.generate(None, RolloutConfig(max_tokens_to_generate=8, max_prompt_length=10, temperature=1.0, top_p=1.0,
                                      eos_tokens=[-1], return_logprobs=True, seed=3), prompt_token_ids=prompts)
  gen = np.stack(ro.tokens)
  scored = r.get_per_token_logps(ro.left_padded_prompt_tokens, gen)
  # the scoring pass walks several tokens per sequence through the many-token attention kernel, the
  # rollout decoded them one by one: same values up to bf16 rounding flips of the hidden states
  assert np.abs(scored - np.stack(ro.logprobs)).max() <= LOGPROB_TOL
  with pytest.raises(ValueError):
    s.per_token_logps(np.zeros((2, 0), np.int32), comp[:2])


def test_scoring_clip_reaches_the_many_rows_head():
  """A head scaled by 1e30 puts every logit beyond the reference's clip at +-1e9
  (tunix/rl/common.py:217-221): a target with a positive logit then scores 1e9 - (1e9 + log n) = 0
  in f32, one with a negative logit -2e9.  8 sequences x 22 tokens = 176 rows per pass: the
  256 x 256 head kernel."""
  from oracle import scoring
  cfg = C.TOY
  st = C.make_state(cfg, 31, 8, norm_jitter=0.05)
  plain = OM.Decoder(cfg, C.oracle_weights(cfg, st, 64, 16.0, 8))
  st['lm_head.w'] = bf16_round(st['lm_head.w'] * np.float32(1e30))
  oracle = OM.Decoder(cfg, C.oracle_weights(cfg, st, 64, 16.0, 8))
  model = C.product_model(cfg, st, 64, 16.0)
  s = _sampler(model, cfg, 48)
  rng = np.random.default_rng(4)
  prompt = rng.integers(3, cfg.vocab_size, (8, 10)).astype(np.int32)
  comp = rng.integers(3, cfg.vocab_size, (8, 12)).astype(np.int32)
  got = s.per_token_logps(prompt, comp, pad_id=0)
  want = scoring.per_token_logps(oracle, prompt, comp, 0)
  assert np.isfinite(got).all() and set(np.unique(want)) <= {0.0, np.float32(-2e9)}
  # the sign of a target logit is compared where the unscaled logit is clear of bf16 rounding
  ids = np.concatenate([prompt, comp], 1)
  valid = np.ones_like(ids, bool)
  pos = OMK.build_positions_from_mask(valid)
  base_logits, _ = plain(ids, pos, None, OMK.make_causal_attn_mask(valid, ids.shape[1]))
  tgt = np.take_along_axis(base_logits[:, -13:-1, :], comp[..., None], -1)[..., 0]
  clear = np.abs(tgt) > 0.05
  assert clear.sum() > 48
  np.testing.assert_array_equal(got[clear], want[clear])


@pytest.mark.parametrize('family', ['llama3', 'qwen3', 'moe'])
def test_multi_token_passes_equal_one_token_passes(family):
  """Cache fill and scoring in passes of several tokens per sequence (rows = sequences x tokens)
  against the one-token walk: same KV cache, same next-step logits, same per-token log-probs up
  to the f32 summation order of differently split projections."""
  if family == 'moe':
    cfg = OM.Config('qwen3', 2, 1024, 256, 256, 4, 64, 2, rope_theta=1_000_000, norm_eps=1e-6, tied=False,
                    num_experts=8, experts_per_tok=2)
  elif family == 'qwen3':
    # vocabulary not a multiple of 256: the many-rows scoring head has a ragged last block
    cfg = OM.Config('qwen3', 2, 1056, 256, 1024, 4, 64, 2, rope_theta=1_000_000, norm_eps=1e-6, tied=False)
  else:
    cfg = C.TOY
  st0 = C.make_state(cfg, 41, 8, norm_jitter=0.05)
  model = C.product_model(cfg, st0, 64, 16.0)
  s = _sampler(model, cfg, 64)
  s.eos_ids = np.array([-1])
  rng = np.random.default_rng(3)
  # 8 sequences, so that 40 tokens per pass are 320 rows (256-row projection blocks; MoE: 640 routed pairs)
  ids = rng.integers(3, cfg.vocab_size, (8, 41)).astype(np.int32)
  ids[1, :7] = 0   # left padding
  ids[2, :1] = 0
  def fill(tokens_per_pass):
    st = s.init_sample_state(ids, 48, True, None, 0.0, None, None, 0, include_logprobs=True)
    n = 40
    while n > 0:
      t = min(tokens_per_pass, n)
      s.run_steps(st, 1, sample=False, tokens_per_pass=t)
      n -= t
    assert int(st['step'].item()) == 40
    cache = st['cache'].float().cpu().numpy().copy()
    s.run_steps(st, 1, sample=True)
    return cache, st['logits'].cpu().numpy().copy(), st['token_buffer'][:, 41].cpu().numpy().copy()
  c1, l1, t1 = fill(1)
  for tpp in (2, 7, 40):
    c, l, t = fill(tpp)
    assert np.abs(c - c1).max() <= 2.0 ** -6 * max(1.0, np.abs(c1).max()), tpp
    assert np.abs(l - l1).max() <= LOGIT_TOL, (tpp, np.abs(l - l1).max())
  # scoring: Sampler.per_token_logps walks in multi-token passes; compare with one token per pass
  prompt, comp = ids[:, :20], ids[:, 20:]
  got = s.per_token_logps(prompt, comp, pad_id=0)
  s.MAX_ROWS = s.MAX_FILL_ROWS = 3  # one token per sequence and pass
  try:
    one = s.per_token_logps(prompt, comp, pad_id=0)
  finally:
    s.MAX_ROWS, s.MAX_FILL_ROWS = Sampler.MAX_ROWS, Sampler.MAX_FILL_ROWS
  # (MoE: a rounding flip of a hidden state near a routing tie changes an expert weight, hence twice the slack)
  assert np.abs(got - one).max() <= (2 if family == 'moe' else 1) * LOGPROB_TOL, np.abs(got - one).max()
  with pytest.raises(Exception):
    s.run_steps(s.init_sample_state(ids, 48, False, None, 0.0, None, None, 0), 1, sample=True, tokens_per_pass=2)


def test_packed_checkpoint_round_trip_gives_the_same_rollout(tmp_path):
  """save_packed -> load_packed keeps the device layout byte for byte, so a reloaded model
  samples the same tokens and log-probs as the one that was saved."""
  from tunix_amd import checkpoint as CK
  cfg = C.TOY
  model = C.product_model(cfg, C.make_state(cfg, 5, 8, norm_jitter=0.05), 64, 16.0)
  path = str(tmp_path / 'toy.safetensors')
  CK.save_packed(model, path)
  again = CK.load_packed(path)
  rng = np.random.default_rng(2)
  prompts = [rng.integers(3, cfg.vocab_size, n) for n in (5, 9, 3)]
  kw = dict(prompt_token_ids=prompts, max_generation_steps=12, eos_tokens=[-1], temperature=0.8, top_p=1.0,
            return_logprobs=True, seed=4)
  a = _sampler(model, cfg, 32)(**kw)
  b = _sampler(again, cfg, 32)(**kw)
  for x, y, lx, ly in zip(a.tokens, b.tokens, a.logprobs, b.logprobs):
    assert (x == y).all() and np.array_equal(np.asarray(lx), np.asarray(ly))


@pytest.mark.parametrize('family', ['llama3', 'qwen3'])
def test_hf_checkpoint_loader_to_gpu_logits_match_oracle(tmp_path, family):
  """models/safetensors_loader.py:474 load_and_create_model's path: a Hugging Face checkpoint on disk
  (transformers random init -> save_pretrained, safetensors) -> checkpoint.model_from_hf (renaming rules
  of models/llama3/params.py:23-80 / models/qwen3/params.py:47-121 + int4 quantisation) -> decode-step
  logits on the GPU, against the oracle built from the state the renaming rules give (2e-2)."""
  transformers = pytest.importorskip('transformers')
  from tunix_amd import checkpoint as CK
  torch.manual_seed(3)
  common = dict(vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                num_key_value_heads=2, head_dim=64, max_position_embeddings=64, attention_bias=False,
                tie_word_embeddings=False)
  if family == 'llama3':
    hf = transformers.LlamaForCausalLM(transformers.LlamaConfig(rms_norm_eps=1e-5, mlp_bias=False, **common))
    cfg = OM.Config('llama3', 2, 512, 256, 512, 4, 64, 2, norm_eps=1e-5)
  else:
    hf = transformers.Qwen3ForCausalLM(transformers.Qwen3Config(rms_norm_eps=1e-6, rope_theta=1_000_000.0, **common))
    cfg = OM.Config('qwen3', 2, 512, 256, 512, 4, 64, 2, rope_theta=1_000_000, norm_eps=1e-6)
  with torch.no_grad():
    for name, prm in hf.named_parameters():
      if 'norm' in name:
        prm.add_(0.1 * torch.randn_like(prm))
  hf.to(torch.bfloat16).save_pretrained(str(tmp_path), safe_serialization=True)
  pcfg = C.product_config(cfg)
  model = CK.model_from_hf(str(tmp_path), pcfg, group=64)
  # the oracle takes the renamed state as numpy and quantises it with its own restatement
  renamed = {k: v.float().numpy() for k, v in CK.load_hf_safetensors(str(tmp_path), pcfg).items()}
  assert renamed['layers.0.attn.q_proj.w'].shape == (256, 4, 64) and renamed['layers.1.attn.o_proj.w'].shape == (4, 64, 256)
  oracle = OM.Decoder(cfg, C.oracle_weights(cfg, renamed, 64, 0.0, 0))
  rng = np.random.default_rng(4)
  prompts = [rng.integers(3, cfg.vocab_size, 12) for _ in range(3)]
  ref = OSAM.generate(oracle, cfg, prompts, 6, 32, eos_ids=(-1,), keep_logits=True, max_prompt_length=12)
  s = _sampler(model, cfg, 32)
  s.eos_ids = np.array([-1])
  st = s.init_sample_state(ref['padded_prompt_tokens'], 18, True, None, 0.0, None, None, 0, include_logprobs=True,
                           prompt_lengths=ref['prompt_lengths'])
  s.walk(st, 11)
  for step in range(6):
    s.run_steps(st, 1, sample=True)
    got, want = st['logits'].cpu().numpy(), ref['state'].step_logits[step]
    assert np.abs(got - want).max() <= LOGIT_TOL, (family, step, np.abs(got - want).max())
    assert np.abs(want).max() > 0.1  # the comparison is not between two all-zero tensors
    tok = ref['state'].token_buffer[:, 12 + step]
    st['token_buffer'][:, 12 + step] = torch.from_numpy(tok).to(st['token_buffer'].device)  # teacher forcing
