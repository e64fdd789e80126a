"""Checkpoint loaders (host logic, CPU): Hugging Face safetensors -> the reference's parameter
paths (rules of tunix/models/llama3/params.py:23-80, tunix/models/qwen3/params.py:25-121), and
the packed on-disk format of the quantised model."""
import numpy as np
import pytest
import torch

from tunix_amd import checkpoint as CK
from tunix_amd.model import ModelConfig, QLoRAModel


def _tiny(family, tied=False, experts=None):
  return ModelConfig(family, 2, 128, 64, 128, 4, 16, 2, 10_000, 1e-6, tied, experts, 2 if experts else None)


@pytest.mark.parametrize('family', ['llama3', 'qwen3'])
def test_hf_safetensors_are_renamed_like_the_reference(family, tmp_path):
  transformers = pytest.importorskip('transformers')
  torch.manual_seed(0)
  common = dict(vocab_size=128, hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
                num_key_value_heads=2, head_dim=16, max_position_embeddings=64, attention_bias=False,
                tie_word_embeddings=False)
  if family == 'llama3':
    hf = transformers.LlamaForCausalLM(transformers.LlamaConfig(mlp_bias=False, **common))
  else:
    hf = transformers.Qwen3ForCausalLM(transformers.Qwen3Config(**common))
  hf.save_pretrained(tmp_path, safe_serialization=True)
  cfg = _tiny(family)
  st = CK.load_hf_safetensors(str(tmp_path), cfg)
  sd = hf.state_dict()
  d, n, kh, h = 64, 4, 2, 16
  for i in range(2):
    q = sd[f'model.layers.{i}.self_attn.q_proj.weight']          # torch [out, in]
    assert st[f'layers.{i}.attn.q_proj.w'].shape == (d, n, h)
    # element [in, head, dim] of the tunix tensor is row head * H + dim, column in of the torch one
    torch.testing.assert_close(st[f'layers.{i}.attn.q_proj.w'][5, 3, 7], q[3 * h + 7, 5])
    o = sd[f'model.layers.{i}.self_attn.o_proj.weight']
    assert st[f'layers.{i}.attn.o_proj.w'].shape == (n, h, d)
    torch.testing.assert_close(st[f'layers.{i}.attn.o_proj.w'][2, 9, 11], o[11, 2 * h + 9])
    assert st[f'layers.{i}.attn.k_proj.w'].shape == (d, kh, h)
    g = sd[f'model.layers.{i}.mlp.gate_proj.weight']
    torch.testing.assert_close(st[f'layers.{i}.mlp.gate_proj.kernel'], g.t())
    torch.testing.assert_close(st[f'layers.{i}.input_layernorm.w'], sd[f'model.layers.{i}.input_layernorm.weight'])
    if family == 'qwen3':
      torch.testing.assert_close(st[f'layers.{i}.attn.q_norm.w'], sd[f'model.layers.{i}.self_attn.q_norm.weight'])
  torch.testing.assert_close(st['lm_head.w'], sd['lm_head.weight'].t())
  torch.testing.assert_close(st['embedder.input_embedding'], sd['model.embed_tokens.weight'])
  # the renamed state is exactly what QLoRAModel.from_state consumes
  m = QLoRAModel.from_state(cfg, st, group=64, device='cpu')
  assert len(m.layers) == 2 and m.layers[0]['qkv'].n == (n + 2 * kh) * h
  with pytest.raises(FileNotFoundError):
    CK.load_hf_safetensors(str(tmp_path / 'nothing'), cfg)


def test_moe_expert_keys_are_stacked():
  cfg = _tiny('qwen3', experts=4)
  g = torch.Generator().manual_seed(1)
  t = lambda *s: torch.randn(*s, generator=g)
  sd = {'model.embed_tokens.weight': t(128, 64), 'model.norm.weight': t(64), 'lm_head.weight': t(128, 64)}
  for i in range(2):
    p = f'model.layers.{i}.'
    sd.update({p + 'self_attn.q_proj.weight': t(64, 64), p + 'self_attn.k_proj.weight': t(32, 64),
               p + 'self_attn.v_proj.weight': t(32, 64), p + 'self_attn.o_proj.weight': t(64, 64),
               p + 'self_attn.q_norm.weight': t(16), p + 'self_attn.k_norm.weight': t(16),
               p + 'input_layernorm.weight': t(64), p + 'post_attention_layernorm.weight': t(64),
               p + 'mlp.gate.weight': t(4, 64)})
    for e in range(4):
      sd.update({p + f'mlp.experts.{e}.gate_proj.weight': t(128, 64), p + f'mlp.experts.{e}.up_proj.weight': t(128, 64),
                 p + f'mlp.experts.{e}.down_proj.weight': t(64, 128)})
  st = CK.rename_hf_state(cfg, sd)
  assert st['layers.1.mlp.gate_proj'].shape == (4, 64, 128) and st['layers.1.mlp.down_proj'].shape == (4, 128, 64)
  torch.testing.assert_close(st['layers.1.mlp.up_proj'][3], sd['model.layers.1.mlp.experts.3.up_proj.weight'].t())
  torch.testing.assert_close(st['layers.0.mlp.router.kernel'], sd['model.layers.0.mlp.gate.weight'].t())
  with pytest.raises(KeyError):
    CK.rename_hf_state(cfg, {**sd, 'model.layers.0.unknown.weight': t(2)})


def test_packed_format_round_trip(tmp_path):
  for cfg, rank in ((ModelConfig('llama3', 2, 96, 64, 128, 4, 16, 2, 10_000, 1e-5, True), 8),
                    (_tiny('qwen3', experts=4), 0)):
    m = QLoRAModel.random_init(cfg, seed=3, group=64, lora_rank=rank, lora_alpha=16.0 if rank else 0.0,
                               lora_targets=('q_proj', 'k_proj', 'v_proj', 'o_proj'), device='cpu')
    path = str(tmp_path / f'{cfg.family}.safetensors')
    CK.save_packed(m, path)
    r = CK.load_packed(path, device='cpu')
    assert r.config == cfg and r.group == 64 and r.lora_rank == rank
    assert (r.head is r.embed) == bool(cfg.weight_tying)
    for a, b in zip(m.layers, r.layers):
      assert set(a.keys()) == set(b.keys())
      for k in a:
        if isinstance(a[k], torch.Tensor):
          assert torch.equal(a[k], b[k])
        else:
          assert (a[k].k, a[k].n, a[k].seg_cols, a[k].rank, a[k].experts) == (b[k].k, b[k].n, b[k].seg_cols, b[k].rank, b[k].experts)
          assert torch.equal(a[k].qweight, b[k].qweight) and torch.equal(a[k].scales, b[k].scales)
          if a[k].lora_a_t is not None:
            assert torch.equal(a[k].lora_a_t, b[k].lora_a_t) and torch.equal(a[k].lora_b, b[k].lora_b)
    assert set(m.lora_state().keys()) == set(r.lora_state().keys())
  with pytest.raises(ValueError):
    from safetensors.torch import save_file
    save_file({'x': torch.zeros(1)}, str(tmp_path / 'other.safetensors'))
    CK.load_packed(str(tmp_path / 'other.safetensors'), device='cpu')
