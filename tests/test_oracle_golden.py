"""The oracle against every golden vector the reference's own tests hold for this path
(tests/generate/utils_test.py:91-179, tests/generate/sampler_test.py:1095-1132) and the
Random123 known-answer vectors for threefry2x32, all kept as data in
tests/golden/reference_vectors.json.  The product's host helpers
(tunix_amd.utils) are checked against the same vectors."""
import json
import os

import numpy as np
import pytest

from oracle import masks as OM
from oracle import prng
from tunix_amd import utils as PU

IMPLS = [pytest.param(OM, id='oracle'), pytest.param(PU, id='product')]
GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'reference_vectors.json')))


@pytest.mark.parametrize('m', IMPLS)
def test_compute_attention_mask_golden(m):
  g = GOLD['compute_attention_masks']
  input_mask = np.array(g['input_mask'], dtype=bool)
  for case in g['cases']:
    got = m.compute_attention_masks(case['time_step'], case['seq_len'], input_mask)
    assert got.shape == (2, 1, case['seq_len'])
    np.testing.assert_array_equal(got[:, 0], np.array(case['expected'], dtype=bool))


@pytest.mark.parametrize('m', IMPLS)
def test_make_causal_attn_mask_golden(m):
  g = GOLD['make_causal_attn_mask']
  got = m.make_causal_attn_mask(np.array(g['input_mask']), g['cache_size'])
  np.testing.assert_array_equal(got.astype(int), np.array(g['expected']))


@pytest.mark.parametrize('m', IMPLS)
def test_next_power_of_2_and_cdiv_golden(m):
  g = GOLD['next_power_of_2']
  assert [m.next_power_of_2(x) for x in g['inputs']] == g['expected']
  for a, b, want in GOLD['cdiv']['cases']:
    assert m.cdiv(a, b) == want


@pytest.mark.parametrize('m', IMPLS)
def test_index_finders_golden(m):
  g = GOLD['find_first_non_pad_idx']
  for ids, want in g['cases']:
    assert m.find_first_non_pad_idx(np.array(ids), g['pad_id']) == want
  g = GOLD['find_first_eos_idx']
  for ids, want in g['cases']:
    assert m.find_first_eos_idx(np.array(ids), g['eos_id']) == want
  g = GOLD['find_last_non_pad_idx']
  for ids, want in g['cases']:
    assert m.find_last_non_pad_idx(np.array(ids), g['pad_id']) == want


@pytest.mark.parametrize('m', IMPLS)
def test_left_pad_and_positions_golden(m):
  g = GOLD['left_pad_and_positions']
  ids, lens, p = m.left_pad_prompt_tokens(g['prompt_token_ids'], g['max_prompt_length'], g['pad_id'],
                                          max_allowed_length=14)
  np.testing.assert_array_equal(ids, np.array(g['padded_prompt_tokens'], np.int32))
  np.testing.assert_array_equal(lens, np.array(g['prompt_lengths'], np.int32))
  assert p == g['max_prompt_length']
  mask = np.arange(p)[None, :] >= (p - lens[:, None])
  np.testing.assert_array_equal(mask, np.array(g['input_mask'], dtype=bool))
  np.testing.assert_array_equal(m.build_positions_from_mask(mask), g['positions'])


@pytest.mark.parametrize('m', IMPLS)
def test_left_pad_bucketing(m):
  # generate/utils.py:2208-2216: pow-2 bucket capped at cache_size - max_generation_steps
  _, _, p = m.left_pad_prompt_tokens([[1] * 5], None, 0, max_allowed_length=100)
  assert p == 8
  _, _, p = m.left_pad_prompt_tokens([[1] * 5], None, 0, max_allowed_length=6)
  assert p == 6
  _, _, p = m.left_pad_prompt_tokens([[1] * 5], 3, 0, max_allowed_length=4)
  assert p == 8  # longest prompt does not fit the allowance: keep the bucket


def test_threefry2x32_known_answers():
  num = lambda v: int(v, 16) if isinstance(v, str) else int(v)
  for case in GOLD['threefry2x32']['cases']:
    k0, k1 = (np.uint32(num(v)) for v in case['key'])
    c0, c1 = (np.uint32(num(v)) for v in case['counter'])
    x0, x1 = prng.threefry2x32(k0, k1, c0, c1)
    assert (int(x0), int(x1)) == tuple(num(v) for v in case['expected'])


def test_threefry_matches_the_key_pair_of_jax_split():
  """jax.random.split(jax.random.PRNGKey(0)) prints [[4146024105, 967050713], [2718843009, 1272950319]]
  in JAX's own documentation (the pseudo-random numbers tutorial).  split hashes the counters
  0..3 under the key (0, 0) with the first half as word 0 and the second half as word 1, so
  the pair pins how JAX feeds keys and counters to threefry2x32, which fold_in shares."""
  k0, k1 = prng.prng_key(0)
  assert (int(k0), int(k1)) == (0, 0)
  y0, y1 = prng.threefry2x32(k0, k1, np.array([0, 1], np.uint32), np.array([2, 3], np.uint32))
  assert [int(v) for v in y0] == [4146024105, 967050713]
  assert [int(v) for v in y1] == [2718843009, 1272950319]


def test_random_bits_reproduce_the_documented_normal_of_key_42():
  """JAX's documentation prints jax.random.normal(jax.random.key(42)) = -0.028304616 (releases
  with jax_threefry_partitionable on by default, 0.5.0 and later: the reference needs
  jax >= 0.6.0, pyproject.toml:31) and -0.18471177 before that.  normal() is
  sqrt(2) * erfinv(u) with u uniform in (-1, 1) built from one 32-bit word the same way
  uniform_from_bits builds it, so the first value pins random_bits (64-bit element index as the
  counter words, x0 ^ x1 as the output) together with the mantissa trick; the second shows
  that the older scheme (counter words (0, 0), first output word) is the one NOT restated."""
  from scipy.special import erfinv

  def normal_of(word):
    f = ((np.uint32(word) >> np.uint32(9)) | np.uint32(0x3F800000)).view(np.float32) - np.float32(1.0)
    lo, hi = np.nextafter(np.float32(-1.0), np.float32(0.0)), np.float32(1.0)
    u = np.maximum(lo, f * (hi - lo) + lo)
    return float(np.sqrt(2.0) * erfinv(np.float64(u)))

  key = prng.prng_key(42)
  assert abs(normal_of(prng.random_bits(key, (1,))[0]) - (-0.028304616)) < 2e-8
  y0, _ = prng.threefry2x32(key[0], key[1], np.array([0], np.uint32), np.array([0], np.uint32))
  assert abs(normal_of(y0[0]) - (-0.18471177)) < 1e-7
  # jax.random.uniform(jax.random.key(0)) prints 0.947667 with the partitionable scheme and
  # 0.41845703 with the older one: the [0, 1) map itself, without the erfinv on top
  key0 = prng.prng_key(0)
  unit = lambda w: float(((np.uint32(w) >> np.uint32(9)) | np.uint32(0x3F800000)).view(np.float32) - np.float32(1.0))
  assert abs(unit(prng.random_bits(key0, (1,))[0]) - 0.947667) < 5e-7
  z0, _ = prng.threefry2x32(key0[0], key0[1], np.array([0], np.uint32), np.array([0], np.uint32))
  assert abs(unit(z0[0]) - 0.41845703) < 5e-8


def test_uniform_and_gumbel_ranges():
  bits = np.array([0, 1, 0xFFFFFFFF, 0x80000000], np.uint32)
  u = prng.uniform_from_bits(bits)
  assert u[0] == np.finfo(np.float32).tiny and u[2] < 1.0 and abs(u[3] - 0.5) < 1e-6
  g = prng.gumbel(prng.prng_key(0), (4, 1000))
  assert np.isfinite(g).all()
  # Gumbel(0, 1): mean = Euler-Mascheroni, var = pi^2 / 6
  assert abs(g.mean() - 0.5772) < 0.06 and abs(g.var() - np.pi ** 2 / 6) < 0.2


def test_categorical_distribution_chi2():
  z = np.log(np.array([0.5, 0.25, 0.125, 0.125], np.float32))[None, :].repeat(4000, 0)
  tok = prng.categorical(prng.prng_key(7), z)
  counts = np.bincount(tok, minlength=4)
  expected = 4000 * np.array([0.5, 0.25, 0.125, 0.125])
  chi2 = ((counts - expected) ** 2 / expected).sum()
  assert chi2 < 16.3  # 3 dof, p = 0.001
