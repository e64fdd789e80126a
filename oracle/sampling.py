"""Token selection and log-probabilities (test infrastructure only).

Restates tunix/generate/sampler.py:112-168 (sample_top_p, sample_best).
"""
import numpy as np

from oracle import prng


def log_softmax(z):
  z = np.asarray(z, np.float32)
  s = z - z.max(axis=-1, keepdims=True)
  return (s - np.log(np.exp(s).sum(axis=-1, keepdims=True, dtype=np.float32))).astype(np.float32)


def softmax(z):
  z = np.asarray(z, np.float32)
  e = np.exp(z - z.max(axis=-1, keepdims=True))
  return (e / e.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float32)


def apply_forbidden(logits, forbidden):
  """sampler.py:536-537: logits[..., forbidden] = -inf."""
  if forbidden:
    logits = np.array(logits, np.float32, copy=True)
    logits[..., list(forbidden)] = -np.inf
  return logits


def sample_best(logits):
  """sampler.py:158-168.  logits f32 [B, V] -> (token i32 [B], logprob f32 [B])."""
  logits = np.asarray(logits, np.float32)
  tok = np.argmax(logits, axis=-1).astype(np.int32)
  logp = log_softmax(logits)
  return tok, np.take_along_axis(logp, tok[:, None], axis=-1)[:, 0]


def sample_top_p(logits, key, temperature, top_p, top_k=None):
  """sampler.py:112-155.  The logprob is of the temperature-scaled, NOT
  nucleus-renormalised distribution (:131-134, :148-151)."""
  z = (np.asarray(logits, np.float32) / np.float32(temperature)).astype(np.float32)
  no_topk = top_k is None or top_k <= 0
  logp = log_softmax(z)
  if top_p >= 1.0 and no_topk:
    tok = prng.categorical(key, z)
    return tok, np.take_along_axis(logp, tok[:, None], axis=-1)[:, 0]
  k = z.shape[-1] if no_topk else top_k
  # lax.top_k: descending, stable (lower index first among equals).
  order = np.argsort(-z, axis=-1, kind='stable')[:, :k]
  zs = np.take_along_axis(z, order, axis=-1)
  ps = softmax(zs)
  cs = np.cumsum(ps, axis=-1, dtype=np.float32)
  mask = (cs - ps) > np.float32(top_p)
  zs = np.where(mask, -np.inf, zs).astype(np.float32)
  pick = prng.categorical(key, zs)
  tok = np.take_along_axis(order, pick[:, None], axis=-1)[:, 0].astype(np.int32)
  return tok, np.take_along_axis(logp, tok[:, None], axis=-1)[:, 0]


def nucleus_members(z_row, top_p):
  """Set of token ids that survive the top-p filter for one row (z already / T)."""
  z_row = np.asarray(z_row, np.float32)
  order = np.argsort(-z_row, kind='stable')
  ps = softmax(z_row[order][None, :])[0]
  cs = np.cumsum(ps, dtype=np.float32)
  keep = ~((cs - ps) > np.float32(top_p))
  return set(order[keep].tolist())
