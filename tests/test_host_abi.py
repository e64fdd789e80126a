"""CPU-side checks of the product: the C ABI library loads and exports every symbol the
header declares, argument checks return error codes without launching, and the Sampler's
input validation raises the reference's errors (tests/generate/sampler_test.py:1150-1170)."""
import ctypes
import os
import re
import sys

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


def test_header_is_plain_c_and_cxx():
  """include/tmx.h is the boundary a foreign-function binding reads: it must compile as C99 and as C++
  on its own (no torch, HIP or C++-only types in any signature)."""
  import shutil
  import subprocess
  hdr = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), 'include', 'tmx.h')
  for cc, lang, std in (('gcc', 'c', '-std=c99'), ('g++', 'c++', '-std=c++11')):
    if shutil.which(cc) is None:
      pytest.skip(f'{cc} is not installed')
    res = subprocess.run([cc, std, '-Wall', '-Wextra', '-Werror', '-pedantic', '-fsyntax-only', '-x', lang, hdr],
                         capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


def test_status_strings_and_version():
  lib = _lib.lib()
  assert lib.tmx_abi_version() == 7 == _lib.ABI_VERSION
  header = open(os.path.join(os.path.dirname(os.path.abspath(__file__)), '..', 'include', 'tmx.h')).read()
  assert '#define TMX_ABI_VERSION 7' in header
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


class _Var:
  """Stand-in for an nnx.LoRAParam leaf: the array sits in `.value`."""

  def __init__(self, value):
    self.value = value


class _PathKey:
  """Stand-in for a jax tree path entry (DictKey): the name sits in `.key`."""

  def __init__(self, key):
    self.key = key


def test_flatten_state_takes_what_the_weight_sync_hands_over():
  import torch
  from tunix_amd import utils
  a = np.arange(6, dtype=np.float32).reshape(2, 3)
  b = np.ones((3, 4), np.float32)
  want = {'layers.0.attn.q_proj.w_lora_a', 'layers.0.attn.q_proj.w_lora_b'}
  nested = {'layers': {0: {'attn': {'q_proj': {'w_lora_a': _Var(a), 'w_lora_b': _Var(b)}}}}}
  by_tuple = {('layers', 0, 'attn', 'q_proj', 'w_lora_a'): a, ('layers', 0, 'attn', 'q_proj', 'w_lora_b'): torch.from_numpy(b)}
  by_pathkeys = {tuple(_PathKey(k) for k in ('layers', 0, 'attn', 'q_proj', 'w_lora_a')): a,
                 tuple(_PathKey(k) for k in ('layers', 0, 'attn', 'q_proj', 'w_lora_b')): b}
  dotted = {'layers.0.attn.q_proj.w_lora_a': a, 'layers.0.attn.q_proj.w_lora_b': b}
  pure = {'layers': {'0': {'attn': {'q_proj': {'w_lora_a': {'value': a}, 'w_lora_b': {'value': b}}}}}}
  as_list = {'layers': [{'attn': {'q_proj': {'w_lora_a': a, 'w_lora_b': b}}}]}
  for tree in (nested, by_tuple, by_pathkeys, dotted, pure, as_list):
    flat = utils.flatten_state(tree)
    assert set(flat) == want
    np.testing.assert_array_equal(flat['layers.0.attn.q_proj.w_lora_a'].float().numpy(), a)
    assert tuple(flat['layers.0.attn.q_proj.w_lora_b'].shape) == (3, 4)


class _LoraStub:
  """Model stand-in for the weight-sync logic: LoRA state in, LoRA state out, with the product's checks."""

  def __init__(self):
    import torch
    self.config = ModelConfig.toy()
    self.device = 'cpu'
    self.state = {'layers.0.attn.q_proj.w_lora_a': torch.zeros(256, 8, dtype=torch.bfloat16),
                  'layers.0.attn.q_proj.w_lora_b': torch.zeros(8, 256, dtype=torch.bfloat16)}

  def lora_state(self):
    return dict(self.state)

  def update_lora(self, state):
    import torch
    from tunix_amd.model import QLoRAModel
    QLoRAModel.check_lora_state(self.state, state)
    self.state = {k: torch.as_tensor(v).to(torch.bfloat16).reshape(self.state[k].shape) for k, v in state.items()}


def test_update_params_accepts_nested_states_and_keeps_the_reference_errors():
  from tunix_amd.sampler import Sampler
  c = ModelConfig.toy()
  s = Sampler(_LoraStub(), C.ToyTokenizer(), CacheConfig(8, c.num_layers, c.num_kv_heads, c.head_dim))
  a = np.full((256, 8), 0.5, np.float32)
  # q_proj B arrives as the reference's [r, N, H] Einsum shape
  b = np.full((8, 4, 64), 0.25, np.float32)
  s.update_params({'layers': {0: {'attn': {'q_proj': {'w_lora_a': _Var(a), 'w_lora_b': _Var(b)}}}}})
  got = s.transformer_state
  assert got['layers.0.attn.q_proj.w_lora_a'].dtype.is_floating_point
  assert float(got['layers.0.attn.q_proj.w_lora_a'].float().mean()) == 0.5
  assert float(got['layers.0.attn.q_proj.w_lora_b'].float().mean()) == 0.25
  # partial update: only A
  s.update_params({('layers', 0, 'attn', 'q_proj', 'w_lora_a'): a * 2})
  assert float(s.transformer_state['layers.0.attn.q_proj.w_lora_a'].float().mean()) == 1.0
  with pytest.raises(ValueError, match='same structure'):
    s.update_params({'layers': {0: {'attn': {'z_proj': {'w_lora_a': a}}}}})
  with pytest.raises(ValueError, match='same shape'):
    s.update_params({'layers.0.attn.q_proj.w_lora_a': np.zeros((256, 4), np.float32)})
  with pytest.raises(ValueError, match='same structure'):
    s.transformer_state = {'layers.0.attn.q_proj.w_lora_a': a}  # the setter wants the whole LoRA state


def test_seed_words_follow_prngkey_without_x64():
  from oracle import prng
  from tunix_amd.sampler import _seed_key
  for seed in (0, 42, -1, 2 ** 32 + 5, 2 ** 40):
    assert _seed_key(seed) == (0, seed & 0xFFFFFFFF)
    assert tuple(int(w) for w in prng.prng_key(seed)) == (0, seed & 0xFFFFFFFF)
  assert _seed_key(None) == (0, 0)
  assert _seed_key(np.array([7, 9], np.uint32)) == (7, 9)
  typed = type('K', (), {'_base_array': np.array([1, 2], np.uint32)})()
  assert _seed_key(typed) == (1, 2)
  with pytest.raises(ValueError):
    _seed_key(np.arange(3))


def test_token_ids_outside_the_vocabulary_are_rejected_before_the_gpu():
  s = _sampler(cache_size=16)
  v = ModelConfig.toy().vocab_size
  for bad in ([[3, v]], [[-2, 4]]):
    with pytest.raises(ValueError, match='outside the vocabulary'):
      s(prompt_token_ids=bad, max_generation_steps=2)
  with pytest.raises(ValueError, match='outside the vocabulary'):
    s.per_token_logps(np.array([[3, 4]]), np.array([[5, v + 7]]))
  with pytest.raises(NotImplementedError, match='echo'):
    s(prompt_token_ids=[[3, 4]], max_generation_steps=2, echo=True, return_logits=True)


def test_model_from_state_tree_flattens_before_it_builds(monkeypatch):
  """QLoRAModel.from_state_tree hands from_state the dotted paths of a nested state (no GPU: from_state is stubbed)."""
  from tunix_amd.model import QLoRAModel
  seen = {}
  monkeypatch.setattr(QLoRAModel, 'from_state', classmethod(lambda cls, cfg, state, **kw: seen.update(state=state, kw=kw) or 'built'))
  w = np.zeros((4, 2, 3), np.float32)
  tree = {'layers': {0: {'attn': {'q_proj': {'w': _Var(w), 'w_lora_a': _Var(np.zeros((4, 2), np.float32))}}}},
          'embedder': {'input_embedding': _Var(np.zeros((8, 4), np.float32))}}
  assert QLoRAModel.from_state_tree(ModelConfig.toy(), tree, group=64, lora_alpha=8.0, device='cpu') == 'built'
  assert set(seen['state']) == {'layers.0.attn.q_proj.w', 'layers.0.attn.q_proj.w_lora_a', 'embedder.input_embedding'}
  assert tuple(seen['state']['layers.0.attn.q_proj.w'].shape) == (4, 2, 3) and seen['kw']['lora_alpha'] == 8.0


def test_rollout_takes_the_actor_forms_the_cluster_hands_over(monkeypatch):
  """TmxRollout(rollout_actor=...): a (reference config, state tree) pair is converted with the
  reference's field names (llama3/model.py:85-101, qwen3/model.py:160-185); an nnx module without
  flax importable and anything else raise TypeError (no GPU: the quantising constructor is stubbed)."""
  import dataclasses as dc
  from tunix_amd.model import QLoRAModel
  from tunix_amd.rollout import TmxRollout

  @dc.dataclass
  class RefLlama:  # the reference's Llama3 ModelConfig, fields only
    num_layers: int = 2
    vocab_size: int = 1024
    embed_dim: int = 256
    hidden_dim: int = 1024
    num_heads: int = 4
    head_dim: int = 64
    num_kv_heads: int = 4
    rope_theta: int = 10_000
    norm_eps: float = 1e-5
    weight_tying: bool = True

  @dc.dataclass
  class RefQwen(RefLlama):
    use_tied_embedding: bool = False
    num_experts: int = 8
    num_experts_per_tok: int = 2

  c = ModelConfig.from_reference(RefLlama())
  assert (c.family, c.num_layers, c.vocab_size, c.head_dim, c.weight_tying, c.num_experts) == ('llama3', 2, 1024, 64, True, None)
  q = ModelConfig.from_reference(RefQwen(weight_tying=False))
  assert (q.family, q.weight_tying, q.num_experts, q.num_experts_per_tok) == ('qwen3', False, 8, 2)
  seen = {}
  monkeypatch.setattr(QLoRAModel, 'from_state_tree',
                      classmethod(lambda cls, cfg, tree, **kw: seen.update(cfg=cfg, tree=tree, kw=kw) or 'policy'))
  tree = {'layers': {0: {}}}
  assert TmxRollout._as_policy((RefLlama(), tree), 128, 32.0, 7.5) == 'policy'
  assert seen['cfg'].family == 'llama3' and seen['tree'] is tree and seen['kw'] == {'group': 128, 'lora_alpha': 32.0, 'bound': 7.5}

  class Module:  # stands for an nnx module: has .config, its state needs flax
    config = RefLlama()
  with pytest.raises(TypeError, match='flax is not importable'):
    TmxRollout._as_policy(Module(), 64, None, 7.5)
  with pytest.raises(TypeError, match='expected a QLoRAModel'):
    TmxRollout._as_policy(object(), 64, None, 7.5)


def test_host_code_under_address_and_undefined_sanitizers():
  """The host side of the C ABI (argument checks, slice planning, workspace carving: everything that runs
  before the first launch) compiled with -fsanitize=address,undefined and driven over the shapes of the five
  benchmark configurations in a child process that preloads the sanitizer runtime.  The sanitizer build is
  made on first use and again when a source is newer than it (about two minutes; the device code is
  compiled as usual, sanitizers apply to host code only)."""
  import subprocess
  from tunix_amd import build as tb
  rt = tb.sanitizer_runtime()
  if rt is None:
    pytest.skip('clang AddressSanitizer runtime not found')
  newest = max(os.path.getmtime(os.path.join(tb.CSRC, f)) for f in os.listdir(tb.CSRC))
  newest = max(newest, os.path.getmtime(os.path.join(os.path.dirname(tb.CSRC), '..', 'include', 'tmx.h')))
  if not os.path.exists(tb.HOSTSAN_LIB_PATH) or os.path.getmtime(tb.HOSTSAN_LIB_PATH) < newest:
    tb.build(host_sanitizers=True)
  # the sanitizer runtime goes in front of whatever the environment already preloads (it must come first)
  preload = ':'.join(p for p in (rt, os.environ.get('LD_PRELOAD', '')) if p)
  env = dict(os.environ, TMX_LIB=tb.HOSTSAN_LIB_PATH, LD_PRELOAD=preload,
             ASAN_OPTIONS='detect_leaks=0:abort_on_error=1', UBSAN_OPTIONS='halt_on_error=1:print_stacktrace=1')
  child = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'host_sanitizer_child.py')
  res = subprocess.run([sys.executable, child], capture_output=True, text=True, env=env, timeout=300)
  assert res.returncode == 0, res.stdout + res.stderr
  assert 'host sanitizer run ok' in res.stdout
  assert 'AddressSanitizer' not in res.stderr and 'runtime error' not in res.stderr, res.stderr


def test_shared_prompt_groups_are_found_on_the_host():
  """Rows that hold samples of one prompt (tunix/rl/rl_learner.py:432-435: every prompt repeated
  num_generations times, consecutively) are grouped by the columns they have in common; a differing mask or
  token ends the common part, and a batch of distinct prompts shares nothing."""
  from tunix_amd.sampler import shared_prompt_groups as groups
  rng = np.random.default_rng(0)
  base = rng.integers(3, 100, (8, 256))
  ids = np.repeat(base, 8, axis=0)
  ones = lambda a: np.ones_like(a, bool)
  assert groups(ids, ones(ids)) == (8, 256, 256)
  tail = np.concatenate([ids, rng.integers(3, 100, (64, 200))], axis=1)   # private columns behind the prompt
  assert groups(tail, ones(tail)) == (8, 256, 256)
  assert groups(base, ones(base)) == (1, 0, 0)
  odd = np.repeat(rng.integers(3, 100, (2, 70)), 4, axis=0)
  assert groups(odd, ones(odd)) == (4, 64, 70)                             # 70 common columns, 64 = two blocks of 32
  odd[5, 40] = 1
  assert groups(odd, ones(odd)) == (4, 32, 40)
  m = ones(ids)
  m[3, 10] = False                                                          # one row masks a column: not the same prompt any more
  assert groups(ids, m)[1] < 32 or groups(ids, m)[0] != 8
  assert groups(ids[:, :16], ones(ids[:, :16])) == (1, 0, 0)               # too short to be worth a launch of its own
