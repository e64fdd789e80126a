"""Teacher-forced per-token log-probabilities (test infrastructure only).

Restates tunix/rl/common.py:426-606 (compute_per_token_logps, the branch without sequence
packing and without chunking) with process_ids (:257-330) and selective_log_softmax
(:207-226): one full-sequence forward over [prompt | completion] without a cache.
"""
import numpy as np

from oracle import masks
from oracle import sampling


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
    logits = logits / np.float32(temperature)                 # :591-592
  logp = sampling.log_softmax(logits)
  return np.take_along_axis(logp, ids[:, -keep:, None], axis=-1)[..., 0]
