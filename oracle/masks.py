"""Mask / position / padding helpers restated (test infrastructure only).

tunix/generate/utils.py:35-59 (compute_attention_masks), :62-84
(make_causal_attn_mask), :87-96 (next_power_of_2, cdiv), :134-174 (pad / eos
finders), :299-312 (build_positions_from_mask), :2200-2229
(left_pad_prompt_tokens).
"""
import numpy as np


def compute_attention_masks(time_step, seq_len, input_mask):
  """input_mask here is the NEGATED token mask (True = padding), exactly as the
  caller passes it (tunix/generate/sampler.py:762-765).  Returns bool [B,1,seq_len],
  True = may attend."""
  input_mask = np.asarray(input_mask, bool)
  b = input_mask.shape[0]
  causal_padding = np.arange(seq_len)[None, :] > np.uint32(time_step)
  max_seq_len = min(input_mask.shape[-1], seq_len)
  start = max(time_step - seq_len + 1, 0)
  # lax.dynamic_slice clamps the start so the slice stays in bounds.
  start = min(start, input_mask.shape[-1] - max_seq_len)
  sl = input_mask[:, start:start + max_seq_len]
  padded = np.zeros((b, seq_len), bool)
  padded[:, :max_seq_len] = sl
  return ~(causal_padding | padded)[:, None, :]


def make_causal_attn_mask(input_mask, cache_size):
  input_mask = np.asarray(input_mask, bool)
  t = input_mask.shape[-1]
  m = input_mask[..., None, :] & np.tril(np.ones((t, t), bool))[None]
  return np.pad(m, ((0, 0), (0, 0), (0, cache_size - t)))


def build_positions_from_mask(input_mask):
  pos = np.cumsum(np.asarray(input_mask, bool), axis=-1).astype(np.int32)
  return pos - (pos >= 1)


def next_power_of_2(x):
  if x == 0:
    return 1
  return int(2 ** int(np.ceil(np.log2(x))))


def cdiv(a, b):
  return -(-a // b)


def find_first_non_pad_idx(ids, pad_id):
  m = np.asarray(ids) != pad_id
  return int(np.argmax(m)) if m.any() else 0


def find_first_eos_idx(ids, eos_ids):
  ids = np.asarray(ids)
  m = np.isin(ids, np.atleast_1d(eos_ids))
  return int(np.argmax(m)) if m.any() else len(ids)


def find_last_non_pad_idx(ids, pad_id):
  ids = np.asarray(ids)
  m = (ids != pad_id)[::-1]
  return len(ids) - int(np.argmax(m)) - 1 if m.any() else len(ids)


def left_pad_prompt_tokens(prompt_ids, max_prompt_length, pad_value, max_allowed_length=None):
  lens = np.array([len(x) for x in prompt_ids], np.int32)
  longest = int(lens.max())
  if max_prompt_length is None or max_prompt_length < longest:
    max_prompt_length = next_power_of_2(longest)
    if max_allowed_length is not None and longest <= max_allowed_length:
      max_prompt_length = min(max_prompt_length, max_allowed_length)
  out = np.full((len(prompt_ids), max_prompt_length), pad_value, np.int32)
  for i, x in enumerate(prompt_ids):
    x = np.asarray(x, np.int32)
    out[i, max_prompt_length - len(x):] = x
  return out, lens, max_prompt_length
