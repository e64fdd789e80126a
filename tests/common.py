"""Shared builders: one dense synthetic state -> (oracle decoder, product model)."""
import numpy as np

from oracle import int4
from oracle import layers as OL
from oracle import model as OM
from oracle.bf16 import bf16_round


class ToyTokenizer:
  """ids <-> space-separated decimal strings; pad 0, bos 1, eos 2 (the ids the
  reference's MockVocab uses, tunix/tests/test_common.py:396-464)."""

  def __init__(self, pad=0, bos=1, eos=2):
    self._pad, self._bos, self._eos = pad, bos, eos

  def encode(self, text):
    return [int(t) for t in text.split()]

  def decode(self, ids):
    return ' '.join(str(int(i)) for i in ids)

  def pad_id(self):
    return self._pad

  def bos_id(self):
    return self._bos

  def eos_id(self):
    return self._eos


def make_state(cfg, seed=0, lora_rank=0, targets=('q_proj', 'k_proj', 'v_proj', 'o_proj'),
               std=0.02, norm_jitter=0.0):
  """Dense weights under the reference's parameter paths (numpy f32 holding bf16)."""
  rng = np.random.default_rng(seed)
  mat = lambda *s: bf16_round(rng.standard_normal(s).astype(np.float32) * np.float32(std))
  ones = lambda n: bf16_round(np.ones(n, np.float32) + norm_jitter * rng.standard_normal(n).astype(np.float32))
  d, f, n, kh, h = cfg.embed_dim, cfg.hidden_dim, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim
  st = {'embedder.input_embedding': mat(cfg.vocab_size, d), 'final_norm.w': ones(d)}
  if not cfg.tied:
    st['lm_head.w'] = mat(d, cfg.vocab_size)
  for i in range(cfg.num_layers):
    p = f'layers.{i}'
    st[f'{p}.input_layernorm.w'] = ones(d)
    st[f'{p}.post_attention_layernorm.w'] = ones(d)
    shapes = {'q_proj': ((d, n, h), (d,), (n, h)), 'k_proj': ((d, kh, h), (d,), (kh, h)),
              'v_proj': ((d, kh, h), (d,), (kh, h)), 'o_proj': ((n, h, d), (n, h), (d,))}
    for name, (ws, ain, bout) in shapes.items():
      st[f'{p}.attn.{name}.w'] = mat(*ws)
      if lora_rank and name in targets:
        st[f'{p}.attn.{name}.w_lora_a'] = mat(*ain, lora_rank)
        st[f'{p}.attn.{name}.w_lora_b'] = mat(lora_rank, *bout)
    if cfg.family == 'qwen3':
      st[f'{p}.attn.q_norm.w'] = ones(h)
      st[f'{p}.attn.k_norm.w'] = ones(h)
    if cfg.num_experts:
      e = cfg.num_experts
      st[f'{p}.mlp.router.kernel'] = mat(d, e) * np.float32(8)  # spread-out routing scores
      st[f'{p}.mlp.gate_proj'], st[f'{p}.mlp.up_proj'] = mat(e, d, f), mat(e, d, f)
      st[f'{p}.mlp.down_proj'] = mat(e, f, d)
      continue
    for name, (k, o) in {'gate_proj': (d, f), 'up_proj': (d, f), 'down_proj': (f, d)}.items():
      st[f'{p}.mlp.{name}.kernel'] = mat(k, o)
      if lora_rank and name in targets:
        st[f'{p}.mlp.{name}.kernel_lora_a'] = mat(k, lora_rank)
        st[f'{p}.mlp.{name}.kernel_lora_b'] = mat(lora_rank, o)
  return st


def oracle_weights(cfg, st, group, lora_alpha, lora_rank, quantized=True):
  def lin(prefix, name, wkey):
    w = st[f'{prefix}.{name}.{wkey}']
    w2 = w.reshape(-1, w.shape[-1]) if name == 'o_proj' else w.reshape(w.shape[0], -1)
    a = st.get(f'{prefix}.{name}.{wkey}_lora_a')
    b = st.get(f'{prefix}.{name}.{wkey}_lora_b')
    if a is not None:
      a, b = a.reshape(-1, a.shape[-1]), b.reshape(b.shape[0], -1)
    ls = lora_alpha / lora_rank if (a is not None and lora_rank) else 0.0
    if quantized:
      q, s = int4.quantize(w2, group)
      return OL.Linear(q=q, scale=s, group=group, a=a, b=b, lora_scale=ls)
    return OL.Linear(w=w2, a=a, b=b, lora_scale=ls)

  w = {'embed': st['embedder.input_embedding'], 'final_norm': st['final_norm.w'], 'layers': []}
  if not cfg.tied:
    w['lm_head'] = OL.Linear(w=st['lm_head.w'])
  for i in range(cfg.num_layers):
    p = f'layers.{i}'
    lw = {'norm1': st[f'{p}.input_layernorm.w'], 'norm2': st[f'{p}.post_attention_layernorm.w'],
          'q': lin(f'{p}.attn', 'q_proj', 'w'), 'k': lin(f'{p}.attn', 'k_proj', 'w'),
          'v': lin(f'{p}.attn', 'v_proj', 'w'), 'o': lin(f'{p}.attn', 'o_proj', 'w')}
    if cfg.num_experts:
      def elin(w2):
        if not quantized:
          return OL.Linear(w=w2)
        q, s = int4.quantize(w2, group)
        return OL.Linear(q=q, scale=s, group=group)
      lw['router'] = st[f'{p}.mlp.router.kernel']
      lw['experts'] = [(elin(st[f'{p}.mlp.gate_proj'][e]), elin(st[f'{p}.mlp.up_proj'][e]),
                        elin(st[f'{p}.mlp.down_proj'][e])) for e in range(cfg.num_experts)]
    else:
      lw['gate'] = lin(f'{p}.mlp', 'gate_proj', 'kernel')
      lw['up'] = lin(f'{p}.mlp', 'up_proj', 'kernel')
      lw['down'] = lin(f'{p}.mlp', 'down_proj', 'kernel')
    if cfg.family == 'qwen3':
      lw['q_norm'], lw['k_norm'] = st[f'{p}.attn.q_norm.w'], st[f'{p}.attn.k_norm.w']
    w['layers'].append(lw)
  return w


def product_config(cfg):
  from tunix_amd.model import ModelConfig
  return ModelConfig(cfg.family, cfg.num_layers, cfg.vocab_size, cfg.embed_dim, cfg.hidden_dim,
                     cfg.num_heads, cfg.head_dim, cfg.num_kv_heads, cfg.rope_theta, cfg.norm_eps, cfg.tied,
                     cfg.num_experts or None, cfg.experts_per_tok or None)


def product_model(cfg, st, group, lora_alpha, device='cuda'):
  import torch
  from tunix_amd.model import QLoRAModel
  tstate = {k: torch.from_numpy(np.ascontiguousarray(v)) for k, v in st.items()}
  return QLoRAModel.from_state(product_config(cfg), tstate, group=group, lora_alpha=lora_alpha, device=device)


TOY = OM.Config('llama3', 2, 1024, 256, 1024, 4, 64, 4, rope_theta=10000, norm_eps=1e-5, tied=False)
