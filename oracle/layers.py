"""Decode-step building blocks restated from the reference (test infrastructure only).

All arrays are float32; under the BF16 policy every value that the reference
holds in bfloat16 is rounded to bf16 at the point where the reference's dtype
rules round it.  Under the F32 policy nothing is rounded (library cross-checks).
"""
import numpy as np

from oracle import int4
from oracle.bf16 import BF16

K_MASK = np.float32(-2.3819763e38)  # tunix/models/llama3/model.py:33, qwen3/model.py:41


def rmsnorm_llama3(x, w, eps, pol=BF16):
  """tunix/models/llama3/model.py:290-297: astype(w * x / rms, dtype); w * x is
  evaluated first in the activation dtype, the division by the f32 rms second."""
  rms = np.sqrt(np.mean(np.square(x, dtype=np.float32), axis=-1, keepdims=True, dtype=np.float32)
                + np.float32(eps)).astype(np.float32)
  return pol.r(pol.r(w * x) / rms)


def rmsnorm_qwen3(x, w, eps, pol=BF16):
  """tunix/models/qwen3/model.py:478-484: everything in f32, one cast at the end."""
  rms = np.sqrt(np.mean(np.square(x, dtype=np.float32), axis=-1, keepdims=True, dtype=np.float32)
                + np.float32(eps)).astype(np.float32)
  return pol.r(w.astype(np.float32) * (x / rms))


def _sincos(positions, head_dim, theta):
  frac = (np.float32(2.0) * np.arange(head_dim // 2, dtype=np.float32) / np.float32(head_dim)).astype(np.float32)
  timescale = np.power(np.float32(theta), frac).astype(np.float32)
  ang = (positions[..., None].astype(np.float32) / timescale).astype(np.float32)  # [B, T, H/2]
  ang = ang[..., None, :]  # [B, T, 1, H/2]
  return np.sin(ang).astype(np.float32), np.cos(ang).astype(np.float32)


def rope_llama3(x, positions, theta=1_000_000, pol=BF16):
  """tunix/models/llama3/model.py:249-270.  x [B, T, heads, H]; f32 trig, f32
  products, one cast.  NOTE Attention.block (:356-365) never passes rope_theta,
  so the Llama3 path always uses the default 1_000_000."""
  h = x.shape[-1]
  sin, cos = _sincos(positions, h, theta)
  x1, x2 = x[..., : h // 2], x[..., h // 2:]
  return pol.r(np.concatenate([x1 * cos - x2 * sin, x2 * cos + x1 * sin], axis=-1))


def rope_qwen3(x, positions, theta, pol=BF16):
  """tunix/models/qwen3/model.py:432-453: sin/cos are cast to the input dtype
  before multiplying, so each product and the sum round in that dtype."""
  h = x.shape[-1]
  sin, cos = _sincos(positions, h, theta)
  sin, cos = pol.r(sin), pol.r(cos)
  x1, x2 = x[..., : h // 2], x[..., h // 2:]
  a = pol.r(pol.r(x1 * cos) - pol.r(x2 * sin))
  b = pol.r(pol.r(x2 * cos) + pol.r(x1 * sin))
  return np.concatenate([a, b], axis=-1)


class Linear:
  """A bias-free projection y = x W (+ LoRA), W given dense or int4-quantised.

  Dense: ``w`` [K, N].  Quantised: ``q`` int8 [K, N], ``scale`` [K // G, N],
  ``group``.  LoRA: ``a`` [K, r], ``b`` [r, N], ``lora_scale`` = alpha / rank.
  """

  def __init__(self, w=None, q=None, scale=None, group=None, a=None, b=None, lora_scale=0.0):
    self.w, self.q, self.scale, self.group = w, q, scale, group
    self.a, self.b, self.lora_scale = a, b, np.float32(lora_scale)

  def weight(self):
    if self.w is not None:
      return self.w
    return int4.dequantize(self.q, self.scale, self.group)

  def merged(self):
    """W + A B alpha/r in f32 (the merged-weight identity used as a check)."""
    w = self.weight().astype(np.float32)
    if self.a is not None:
      w = w + (self.a.astype(np.float32) @ self.b.astype(np.float32)) * self.lora_scale
    return w

  def __call__(self, x, pol=BF16, mode='reference'):
    """mode 'reference': dequantise to a bf16 weight, bf16 matmul (f32 accumulate,
    output rounded), LoRA delta (x A) B s rounded at each einsum output and
    added in the activation dtype (a7/a15/a16).  mode 'fused': the same
    mathematics with a single rounding of base + delta at the end and the exact
    f32 product q * scale (what a fused kernel computes)."""
    x = np.asarray(x, np.float32)
    if mode == 'reference':
      y = pol.r(x @ self.weight())
      if self.a is not None:
        t = pol.r(x @ self.a)
        d = pol.r(pol.r(t @ self.b) * self.lora_scale)
        y = pol.r(y + d)
      return y
    if self.w is not None:
      y = x @ self.w
    else:
      s = np.repeat(self.scale.astype(np.float32), self.group, axis=0)
      y = x @ (self.q.astype(np.float32) * s)
    if self.a is not None:
      t = pol.r(x @ self.a)
      y = y + (t @ self.b) * self.lora_scale
    return pol.r(y)


def silu(x, pol=BF16):
  """jax.nn.silu = x * sigmoid(x); each elementwise op output rounds."""
  sg = pol.r(np.float32(1.0) / (np.float32(1.0) + np.exp(-x.astype(np.float32))))
  return pol.r(x * sg)


def swiglu_mlp(x, gate, up, down, pol=BF16, mode='reference'):
  """tunix/models/llama3/model.py:489-496, qwen3/model.py:1199-1208."""
  g = gate(x, pol, mode)
  u = up(x, pol, mode)
  if mode == 'reference':
    act = pol.r(silu(g, pol) * u)
  else:
    act = pol.r(g / (np.float32(1.0) + np.exp(-g)) * u)
  return down(act, pol, mode)


def softmax_f32(s):
  m = s.max(axis=-1, keepdims=True)
  e = np.exp(s - m, dtype=np.float32)
  return (e / e.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float32)


def gqa_attention(q, k, v, mask, pol=BF16, mode='reference'):
  """tunix/models/llama3/model.py:379-396, qwen3/model.py:776-793.

  q [B, T, N, H]; k, v [B, S, K, H] (the whole cache, S = cache_size);
  mask bool [B, T, S].  mode 'reference' rounds scores (einsum output, then the
  multiply by H**-0.5) and probabilities like the reference's bf16 einsums;
  mode 'fused' keeps f32 until the output."""
  b, t, n, h = q.shape
  _, s, kh, _ = k.shape
  g = n // kh
  qg = q.reshape(b, t, kh, g, h)
  scores = np.einsum('bthgd,bshd->bhgts', qg, k, dtype=np.float32, optimize=True)
  scale = np.float32(h ** -0.5)
  if mode == 'reference':
    scores = pol.r(pol.r(scores) * scale)
  else:
    scores = scores * scale
  scores = np.where(mask[:, None, None, :, :], scores, K_MASK).astype(np.float32)
  p = softmax_f32(scores)
  if mode == 'reference':
    p = pol.r(p)
  out = np.einsum('bhgts,bshd->bthgd', p, v, dtype=np.float32, optimize=True)
  return pol.r(out.reshape(b, t, n, h))


def moe_route(x, router_w, top_k, pol=BF16):
  """tunix/models/qwen3/model.py:895-902.  Returns (weights [.., k], idx [.., k]).
  lax.top_k is stable: among equal probabilities the lower expert id wins."""
  scores = pol.r(x @ router_w).astype(np.float32)
  p = softmax_f32(scores)
  idx = np.argsort(-p, axis=-1, kind='stable')[..., :top_k]
  w = np.take_along_axis(p, idx, axis=-1)
  w = pol.r(w / w.sum(axis=-1, keepdims=True, dtype=np.float32))
  return w, idx.astype(np.int32)


def moe_layer(x, router_w, experts, top_k, pol=BF16, mode='reference'):
  """tunix/models/qwen3/model.py:894-939 (the dense fallback), evaluated only
  for routed (token, expert) pairs: the one-hot dispatch makes every other
  pair contribute exactly zero.  experts: list of (gate, up, down) Linear."""
  shp = x.shape
  x2 = x.reshape(-1, shp[-1])
  w, idx = moe_route(x2, router_w, top_k, pol)
  out = np.zeros_like(x2, dtype=np.float32)
  for e in np.unique(idx):
    rows, slot = np.nonzero(idx == e)
    gate, up, down = experts[int(e)]
    y = swiglu_mlp(x2[rows], gate, up, down, pol, mode)
    out[rows] += y * w[rows, slot][:, None]
  return pol.r(out).reshape(shp), idx.reshape(shp[:-1] + (top_k,))
