"""Teacher-forced per-token log-probabilities (test infrastructure only).

Restates tunix/rl/common.py:426-606 (compute_per_token_logps, the branch without sequence
packing and without chunking) with process_ids (:257-330) and selective_log_softmax
(:207-226): one full-sequence forward over [prompt | completion] without a cache.
"""
import numpy as np

from oracle import masks
from oracle.bf16 import bf16_round


def per_token_logps(model, prompt_tokens, completion_tokens, pad_id, temperature=1.0):
  """model: oracle.model.Decoder.  Returns f32 [B, completion_len]."""
  prompt = np.asarray(prompt_tokens, np.int32)
  comp = np.asarray(completion_tokens, np.int32)
  ids = np.concatenate([prompt, comp], axis=1)               # common.py:284
  valid = ids != pad_id                                       # :302-306
  positions = masks.build_positions_from_mask(valid)          # :311
  t = ids.shape[1]
  attn = masks.make_causal_attn_mask(valid, t)                # :312
  logits, _ = model(ids, positions, None, attn)               # :540, cache=None
  keep = comp.shape[1]
  logits = logits[:, -keep - 1:-1, :]                         # :590
  if temperature not in (0.0, 1.0):
    # :591-592 `logits /= temperature` on the model's bf16 logits: the quotient is a bf16 array
    logits = bf16_round(logits / np.float32(temperature))
  return selective_log_softmax(logits, ids[:, -keep:])


def selective_log_softmax(logits, input_ids):
  """common.py:207-226: NaN logits count as -1e9, the others are clipped to [-1e9, 1e9];
  result = logits[ids] - logsumexp(logits), f32."""
  x = np.asarray(logits, np.float32)
  with np.errstate(invalid='ignore'):
    x = np.where(np.isnan(x), np.float32(-1e9), np.clip(x, np.float32(-1e9), np.float32(1e9))).astype(np.float32)
  # jax.nn.logsumexp: max + log(sum(exp(x - max))), all f32; the target's logit minus that
  # (not the shifted form of log_softmax: at the clip the two differ by log(count))
  mx = x.max(axis=-1, keepdims=True)
  lse = (mx + np.log(np.exp(x - mx).sum(axis=-1, keepdims=True, dtype=np.float32))).astype(np.float32)
  target = np.take_along_axis(x, np.asarray(input_ids)[..., None], axis=-1)
  return (target - lse)[..., 0].astype(np.float32)
