"""Llama3 / Qwen3 decoder forward with KV cache (test infrastructure only).

Restates tunix/models/llama3/model.py:300-410, 489-496, 546-564, 642-697 and
tunix/models/qwen3/model.py:549-604, 776-809, 894-939, 1199-1208, 1268-1289,
1375-1442 for the call contract
  model(tokens i32[B,T], positions i32[B,T], cache, mask bool[B,T,C]) -> (logits f32[B,T,V], cache).
"""
import dataclasses
import numpy as np

from oracle import layers as L
from oracle import int4
from oracle.bf16 import BF16, bf16_round


@dataclasses.dataclass
class Config:
  family: str            # 'llama3' | 'qwen3'
  num_layers: int
  vocab_size: int
  embed_dim: int
  hidden_dim: int
  num_heads: int
  head_dim: int
  num_kv_heads: int
  rope_theta: float = 1_000_000
  norm_eps: float = 1e-5
  tied: bool = False
  num_experts: int = 0
  experts_per_tok: int = 0

  def effective_theta(self):
    # llama3/model.py:356-365 never forwards config.rope_theta -> default 1e6.
    return 1_000_000 if self.family == 'llama3' else self.rope_theta


def init_cache(cfg, batch, cache_size):
  """tunix/generate/sampler.py:171-202, qwen3/model.py:1359-1373."""
  shape = (batch, cache_size, cfg.num_kv_heads, cfg.head_dim)
  return {
      f'layer_{i}': {
          'k': np.zeros(shape, np.float32),
          'v': np.zeros(shape, np.float32),
          'end_index': np.zeros((batch,), np.int32),
      } for i in range(cfg.num_layers)
  }


class Decoder:
  """weights: dict with
     'embed' [V, D]; 'final_norm' [D]; 'lm_head' Linear [D, V] (absent if tied);
     'layers': list of dict(norm1, norm2, q, k, v, o: Linear (2-D, contraction
     axes flattened), gate/up/down: Linear | router [D, E] + experts list,
     q_norm, k_norm [H] for qwen3)."""

  def __init__(self, cfg, weights, pol=BF16, mode='reference'):
    self.cfg, self.w, self.pol, self.mode = cfg, weights, pol, mode
    self.routed = None

  def _norm(self, x, w):
    if self.cfg.family == 'llama3':
      return L.rmsnorm_llama3(x, w, self.cfg.norm_eps, self.pol)
    return L.rmsnorm_qwen3(x, w, self.cfg.norm_eps, self.pol)

  def _rope(self, x, pos):
    if self.cfg.family == 'llama3':
      return L.rope_llama3(x, pos, self.cfg.effective_theta(), self.pol)
    return L.rope_qwen3(x, pos, self.cfg.effective_theta(), self.pol)

  def _attn(self, lw, x, pos, cache, mask):
    c, pol, mode = self.cfg, self.pol, self.mode
    b, t, _ = x.shape
    q = lw['q'](x, pol, mode).reshape(b, t, c.num_heads, c.head_dim)
    k = lw['k'](x, pol, mode).reshape(b, t, c.num_kv_heads, c.head_dim)
    v = lw['v'](x, pol, mode).reshape(b, t, c.num_kv_heads, c.head_dim)
    if c.family == 'qwen3':
      q = L.rmsnorm_qwen3(q, lw['q_norm'], c.norm_eps, pol)
      k = L.rmsnorm_qwen3(k, lw['k_norm'], c.norm_eps, pol)
    q = self._rope(q, pos)
    k = self._rope(k, pos)
    if cache is not None:
      # dynamic_update_slice at end_index[0] % cache_size for ALL rows.
      slot = int(cache['end_index'][0]) % cache['v'].shape[1]
      kc, vc = cache['k'].copy(), cache['v'].copy()
      kc[:, slot:slot + t] = k
      vc[:, slot:slot + t] = v
      k, v = kc, vc
      new_cache = {'k': k, 'v': v, 'end_index': cache['end_index'] + t}
    else:
      new_cache = None
    if mask is not None and mask.shape[-1] != k.shape[1]:
      raise ValueError('mask / key length mismatch')
    if mask is None:
      mask = np.ones((b, t, k.shape[1]), bool)
    o = L.gqa_attention(q, k, v, mask, pol, mode)
    return new_cache, lw['o'](o.reshape(b, t, -1), pol, mode)

  def __call__(self, tokens, positions, cache, mask):
    c, pol = self.cfg, self.pol
    x = self.w['embed'][tokens]
    new_cache = None if cache is None else {}
    routed = []
    for i, lw in enumerate(self.w['layers']):
      name = f'layer_{i}'
      lc = cache[name] if cache else None
      lc, a = self._attn(lw, self._norm(x, lw['norm1']), positions, lc, mask)
      h = pol.r(a + x)
      hn = self._norm(h, lw['norm2'])
      if c.num_experts:
        m, idx = L.moe_layer(hn, lw['router'], lw['experts'], c.experts_per_tok, pol, self.mode)
        routed.append(idx)
      else:
        m = L.swiglu_mlp(hn, lw['gate'], lw['up'], lw['down'], pol, self.mode)
      x = pol.r(h + m)
      if cache is not None:
        new_cache[name] = lc
    self.routed = routed
    x = self._norm(x, self.w['final_norm'])
    if c.tied:
      logits = pol.r(x @ self.w['embed'].T)
    else:
      logits = self.w['lm_head'](x, pol, 'reference')
    return logits.astype(np.float32), new_cache


def random_weights(cfg, seed=0, group=64, lora_rank=0, lora_alpha=0.0, lora_targets=(),
                   quantize=True, std=0.02, bound=7.5):
  """Synthetic weights: every matrix std * N(0,1) rounded to bf16 (mirrors
  tunix/models/dummy_model_creator.py:29-92), norm weights 1; projections int4
  group-quantised; LoRA A, B std * N(0,1) on the named targets."""
  rng = np.random.default_rng(seed)

  def mat(*shape):
    return bf16_round((rng.standard_normal(shape, dtype=np.float32) * np.float32(std)))

  def lin(name, k, n):
    w = mat(k, n)
    a = b = None
    if lora_rank and name in lora_targets:
      a, b = mat(k, lora_rank), mat(lora_rank, n)
    ls = (lora_alpha / lora_rank) if lora_rank else 0.0
    if quantize:
      q, s = int4.quantize(w, group, bound)
      return L.Linear(q=q, scale=s, group=group, a=a, b=b, lora_scale=ls)
    return L.Linear(w=w, a=a, b=b, lora_scale=ls)

  d, f, n, kh, h = cfg.embed_dim, cfg.hidden_dim, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim
  w = {'embed': mat(cfg.vocab_size, d), 'final_norm': np.ones(d, np.float32), 'layers': []}
  if not cfg.tied:
    w['lm_head'] = L.Linear(w=mat(d, cfg.vocab_size))
  for _ in range(cfg.num_layers):
    lw = {
        'norm1': np.ones(d, np.float32), 'norm2': np.ones(d, np.float32),
        'q': lin('q', d, n * h), 'k': lin('k', d, kh * h), 'v': lin('v', d, kh * h),
        'o': lin('o', n * h, d),
    }
    if cfg.family == 'qwen3':
      lw['q_norm'] = np.ones(h, np.float32)
      lw['k_norm'] = np.ones(h, np.float32)
    if cfg.num_experts:
      lw['router'] = mat(d, cfg.num_experts)
      lw['experts'] = [(lin('gate', d, f), lin('up', d, f), lin('down', f, d))
                       for _ in range(cfg.num_experts)]
    else:
      lw['gate'], lw['up'], lw['down'] = lin('gate', d, f), lin('up', d, f), lin('down', f, d)
    w['layers'].append(lw)
  return w
