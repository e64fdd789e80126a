"""CPU-side checks of the product: the C ABI library loads and exports every symbol the
header declares, argument checks return error codes without launching, and the Sampler's
input validation raises the reference's errors (tests/generate/sampler_test.py:1150-1170)."""
import ctypes
import os
import re

import numpy as np
import pytest

from tunix_amd import _lib
from tunix_amd.configs import CacheConfig, RolloutConfig
from tunix_amd.model import ModelConfig

import common as C

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
  text = open(os.path.join(ROOT, 'include', 'tmx.h')).read()
  text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
  return sorted(set(re.findall(r'\b(tmx_[a-z0-9_]+)\s*\(', text)))


def test_library_exports_every_declared_symbol():
  lib = _lib.lib()
  syms = _declared_symbols()
  assert len(syms) >= 15
  for s in syms:
    assert hasattr(lib, s), f'{s} declared in include/tmx.h but not exported'
  # and the Python binding knows all of them
  bound = set(_lib.SIGNATURES) | set(_lib.SIZE_FUNCS) | {'tmx_status_string'}
  assert set(syms) <= bound, sorted(set(syms) - bound)


def test_status_strings_and_version():
  lib = _lib.lib()
  assert lib.tmx_abi_version() == 3
  assert lib.tmx_status_string(0) == b'ok'
  for code in (-1, -2, -3, -4):
    assert len(lib.tmx_status_string(code)) > 5
  with pytest.raises(_lib.TmxError, match='shape'):
    _lib.check(-2, 'x')


def test_argument_checks_return_codes_without_a_gpu():
  lib = _lib.lib()
  assert lib.tmx_int4_dequant(None, None, None, None, 64, 32, 64) == -1
  assert lib.tmx_int4_dequant(None, 1, 1, 1, 65, 32, 64) == -2
  assert lib.tmx_qlora_linear(None, None, None, None, None, None, None, None, None, 1, 64, 32, 64, 0, 0, 0.0) == -1
  assert lib.tmx_qlora_linear_planes(None, 1, 1, 1, None, 1, None, 4, 100, 32, 64, 0, 1) == -2
  assert lib.tmx_qlora_linear_planes(None, 1, 1, 1, None, 1, None, 200, 192, 32, 64, 0, 1) == -2  # more than 128 rows: K % 128
  assert lib.tmx_decode_steps(None, None, None, 1, 1) == -1
  assert lib.tmx_head_sample_workspace_bytes(4, 1024) == 4 * 8 * 5 * 4
  assert lib.tmx_qlora_linear_num_splits(64, 4096, 4096) >= 1
  assert lib.tmx_gqa_decode_workspace_bytes(64, 32, 8, 128, 768) == 0  # enough workgroups without a split
  assert lib.tmx_gqa_decode_workspace_bytes(1, 32, 8, 64, 768) > 0


class _StubModel:
  """Only what the Sampler reads before touching the GPU."""

  def __init__(self):
    self.config = ModelConfig.toy()
    self.device = 'cpu'


def _sampler(cache_size=5):
  from tunix_amd.sampler import Sampler
  c = ModelConfig.toy()
  return Sampler(_StubModel(), C.ToyTokenizer(), CacheConfig(cache_size, c.num_layers, c.num_kv_heads, c.head_dim))


def test_sampler_rejects_invalid_inputs_like_the_reference():
  s = _sampler(5)
  with pytest.raises(ValueError, match='exactly one'):
    s(input_strings=['3 4'], prompt_token_ids=[[1]], max_generation_steps=1)
  with pytest.raises(ValueError, match='exactly one'):
    s(max_generation_steps=1)
  with pytest.raises(ValueError, match='one output per row'):
    s(prompt_token_ids=[[1]], max_generation_steps=1, beam_size=2)
  with pytest.raises(ValueError, match='exceeds cache_size'):
    s(prompt_token_ids=[[1, 2, 3, 4]], max_generation_steps=2)
  with pytest.raises(ValueError, match='must not be empty'):
    s(input_strings=[], max_generation_steps=1)
  with pytest.raises(ValueError, match='must not be empty'):
    s(prompt_token_ids=[], max_generation_steps=1)
  with pytest.raises(ValueError, match='1-D'):
    s(prompt_token_ids=[np.zeros((1, 2), dtype=np.int32)], max_generation_steps=1)
  with pytest.raises(ValueError, match='must be less than the cache size'):
    _sampler(8)(input_strings=['3 4 5 6 7'], max_generation_steps=4, max_prompt_length=8)


def test_sampler_row_limits_are_checked_on_the_host():
  """More than 128 rows per pass need K % 128 == 0 in every projection; 4096 rows at most; MoE models
  at most 8192 routed pairs per pass."""
  import dataclasses
  import torch
  s = _sampler(16)
  assert s._many_rows_ok() and s._fill_rows() == s.MAX_FILL_ROWS
  with pytest.raises(ValueError, match='at most 4096 rows'):
    s._c_state({'token_buffer': torch.zeros(5000, 16, dtype=torch.int32)})
  moe = _sampler(16)
  moe._transformer.config = dataclasses.replace(ModelConfig.toy(), num_experts=16, num_experts_per_tok=8)
  assert moe._max_rows() == 1024 and moe._fill_rows() == 1024
  with pytest.raises(ValueError, match='at most 1024 rows'):
    moe._c_state({'token_buffer': torch.zeros(1025, 16, dtype=torch.int32)})
  odd = _sampler(16)
  odd._transformer.config = dataclasses.replace(ModelConfig.toy(), hidden_dim=ModelConfig.toy().hidden_dim + 64)
  assert not odd._many_rows_ok() and odd._fill_rows() == 128
  with pytest.raises(ValueError, match='at most 128 rows'):
    odd._c_state({'token_buffer': torch.zeros(130, 16, dtype=torch.int32)})


def test_sampler_tokenize_and_surface():
  s = _sampler(16)
  np.testing.assert_array_equal(s.tokenize('5 6 7'), [1, 5, 6, 7])  # bos prepended
  np.testing.assert_array_equal(s.tokenize('1 5'), [1, 5])  # duplicate bos removed
  from tunix_amd.sampler import TokenizerAdapter
  with pytest.raises(ValueError, match='missing methods'):
    TokenizerAdapter(object())
  with pytest.raises(ValueError, match='cache_config does not match'):
    from tunix_amd.sampler import Sampler
    Sampler(_StubModel(), C.ToyTokenizer(), CacheConfig(16, 3, 4, 64))
  for name in ('transformer', 'transformer_state', 'update_params', 'tokenize', 'dtype', 'init_sample_state'):
    assert hasattr(type(s), name) or hasattr(s, name)


def test_rollout_surface_matches_the_plugin_contract():
  from tunix_amd.rollout import BaseRollout, TmxRollout
  for m in ('generate', 'get_per_token_logps', 'update_params', 'pad_id', 'eos_id', 'model'):
    assert m in BaseRollout.__abstractmethods__
  r = TmxRollout(rollout_actor=_StubModel(), tokenizer=C.ToyTokenizer(), mesh=None,
                 rollout_config=RolloutConfig(kv_cache_size=32))
  assert r.pad_id() == 0 and r.eos_id() == 2 and isinstance(r.model(), _StubModel)
  with pytest.raises(ValueError):
    TmxRollout(tokenizer=C.ToyTokenizer(), rollout_config=RolloutConfig())


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
  monkeypatch.setattr(_lib, '_lib', None)
  monkeypatch.setattr(_lib, 'LIB_PATH', str(tmp_path / 'nope.so'))
  with pytest.raises(_lib.TmxError, match='no CPU fallback'):
    _lib.lib()


def test_bench_refuses_more_than_one_gpu():
  import subprocess, sys
  r = subprocess.run([sys.executable, os.path.join(ROOT, 'bench.py'), '--gpus', '2'], capture_output=True, text=True)
  assert r.returncode != 0 and 'ONE GPU' in r.stderr
