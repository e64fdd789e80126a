"""Host-side helpers of the Sampler (numpy), same names and behaviour as the
reference's tunix/generate/utils.py: compute_attention_masks :35-59,
make_causal_attn_mask :62-84, next_power_of_2 :87-91, cdiv :94-96, pad_to_length
:99-131, find_first_non_pad_idx / find_first_eos_idx / find_last_non_pad_idx
:134-198, build_positions_from_mask :299-312, is_token_id_sequence / as_token_ids
:2116-2137, resolve_prompt_tokens :2164-2197, left_pad_prompt_tokens :2200-2229.
"""
import math

import numpy as np


def compute_attention_masks(time_step, seq_len, input_mask):
  """`input_mask` is True on PADDING (the caller negates the token mask).
  Returns bool [B, 1, seq_len], True where attention is allowed."""
  input_mask = np.asarray(input_mask).astype(bool)
  batch = input_mask.shape[0]
  cols = np.arange(seq_len, dtype=np.int64)[None, :]
  future = cols > int(time_step)
  width = min(input_mask.shape[-1], seq_len)
  first = max(int(time_step) - seq_len + 1, 0)
  first = min(first, input_mask.shape[-1] - width)  # dynamic_slice clamps
  pad = np.zeros((batch, seq_len), dtype=bool)
  pad[:, :width] = input_mask[:, first:first + width]
  return np.logical_not(future | pad)[:, None, :]


def make_causal_attn_mask(input_mask, cache_size):
  input_mask = np.asarray(input_mask).astype(bool)
  seq_len = input_mask.shape[-1]
  if cache_size < seq_len:
    raise AssertionError('cache_size must be at least the sequence length')
  lower = np.tri(seq_len, dtype=bool)
  mask = input_mask[..., None, :] & lower
  out = np.zeros(mask.shape[:-1] + (cache_size,), dtype=bool)
  out[..., :seq_len] = mask
  return out


def next_power_of_2(x):
  if x == 0:
    return 1
  return int(2 ** int(math.ceil(math.log2(x))))


def cdiv(a, b):
  return -(-a // b)


def pad_to_length(x, target_length, pad_value=0, left=False, axis=0):
  x = np.asarray(x)
  length = x.shape[axis]
  if length >= target_length:
    return x
  shape = list(x.shape)
  shape[axis] = target_length - length
  fill = np.full(shape, pad_value, dtype=x.dtype)
  return np.concatenate([fill, x] if left else [x, fill], axis=axis)


def find_first_non_pad_idx(ids, pad_id):
  ids = np.asarray(ids)
  assert ids.ndim == 1, f'ids should be a 1d array. Got: {ids.shape}'
  hits = np.flatnonzero(ids != pad_id)
  return int(hits[0]) if hits.size else 0


np_find_first_non_pad_idx = find_first_non_pad_idx


def find_first_eos_idx(ids, eos_id):
  ids = np.asarray(ids)
  assert ids.ndim == 1, f'ids should be a 1d array. Got: {ids.shape}'
  hits = np.flatnonzero(np.isin(ids, np.atleast_1d(np.asarray(eos_id))))
  return int(hits[0]) if hits.size else int(ids.shape[0])


np_find_first_eos_idx = find_first_eos_idx


def find_last_non_pad_idx(ids, pad_id):
  ids = np.asarray(ids)
  assert ids.ndim == 1, f'ids should be a 1d array. Got: {ids.shape}'
  hits = np.flatnonzero(ids != pad_id)
  return int(hits[-1]) if hits.size else int(ids.shape[-1])


def build_positions_from_mask(input_mask):
  counts = np.cumsum(np.asarray(input_mask).astype(np.int32), axis=-1, dtype=np.int32)
  return counts - (counts >= 1).astype(np.int32)


def is_token_id_sequence(prompt):
  if isinstance(prompt, np.ndarray):
    return prompt.ndim == 1 and np.issubdtype(prompt.dtype, np.integer)
  return (isinstance(prompt, (list, tuple)) and bool(prompt)
          and isinstance(prompt[0], (int, np.integer)))


def as_token_ids(value):
  array = np.array(value, dtype=np.int32)
  if array.ndim != 1:
    raise ValueError(f'token ids must be 1-D, got shape {array.shape}')
  return array


def _token_rows(prompt_token_ids, budget, max_length_name, single_output_per_row):
  """Validated int32 rows of caller-supplied token ids (error texts as the reference's)."""
  if len(prompt_token_ids) == 0:
    raise ValueError('prompt_token_ids must not be empty')
  if not single_output_per_row:
    raise ValueError('prompt_token_ids requires exactly one output per row')
  rows = [as_token_ids(r) for r in prompt_token_ids]
  if budget is not None and max((len(r) for r in rows), default=0) > budget:
    raise ValueError(f'prompt plus max_generation_steps exceeds {max_length_name}')
  return rows


def resolve_prompt_tokens(input_strings, prompt_token_ids, tokenize_fn, *, max_generation_steps=0,
                          max_total_length=None, max_length_name='max_model_len',
                          single_output_per_row=True):
  """One int32 id row per prompt, from text (tokenised here) or from ids given as they are."""
  have_text, have_ids = input_strings is not None, prompt_token_ids is not None
  if have_text == have_ids:
    raise ValueError('Provide exactly one of input_strings or prompt_token_ids')
  if have_ids:
    budget = None if max_total_length is None else max_total_length - max_generation_steps
    return _token_rows(prompt_token_ids, budget, max_length_name, single_output_per_row)
  texts = input_strings.tolist() if isinstance(input_strings, np.ndarray) else input_strings
  texts = [texts] if isinstance(texts, str) else texts
  if len(texts) == 0:
    raise ValueError('input_strings must not be empty')
  return [np.asarray(tokenize_fn(str(t)), dtype=np.int32) for t in texts]


def left_pad_prompt_tokens(prompt_ids, max_prompt_length, pad_value, *, max_allowed_length=None):
  """(left-padded int32 [B, P], true lengths, P).  P is the caller's max_prompt_length when every
  prompt fits it; otherwise the longest prompt rounded up to a power of two (one compiled shape
  per bucket in the reference), capped by max_allowed_length when the longest prompt still fits."""
  lengths = np.fromiter((len(r) for r in prompt_ids), dtype=np.int32, count=len(prompt_ids))
  longest = int(lengths.max())
  width = max_prompt_length
  if width is None or width < longest:
    width = next_power_of_2(longest)
    if max_allowed_length is not None and longest <= max_allowed_length < width:
      width = max_allowed_length
  padded = np.full((len(prompt_ids), width), pad_value, dtype=np.int32)
  for i, r in enumerate(prompt_ids):
    if len(r):
      padded[i, width - len(r):] = np.asarray(r, dtype=np.int32)
  return padded, lengths, width


def _leaf_array(leaf):
  """Array held by a state leaf: variable-like objects (nnx.Param / nnx.LoRAParam) carry it in
  `.value` (newer releases: `get_value()`); bf16 arrays of array libraries without a native
  numpy dtype are taken over by their bit pattern."""
  import torch
  for _ in range(2):
    if isinstance(leaf, (torch.Tensor, np.ndarray)):
      break
    if hasattr(leaf, 'value'):
      leaf = leaf.value
    elif hasattr(leaf, 'get_value'):
      leaf = leaf.get_value()
  if isinstance(leaf, torch.Tensor):
    return leaf
  arr = np.asarray(leaf)
  if arr.dtype.kind == 'V' or arr.dtype.name == 'bfloat16':
    if arr.dtype.itemsize != 2:
      raise ValueError(f'unsupported parameter dtype {arr.dtype}')
    return torch.from_numpy(np.ascontiguousarray(arr).view(np.int16).copy()).view(torch.bfloat16)
  return torch.from_numpy(np.ascontiguousarray(arr))


def flatten_state(tree):
  """Flat {dotted path: tensor} of a parameter tree, the counterpart of the reference's
  to_flat_dict (tunix/rl/utils.py:72-78, keys = tuples of path parts) for what the weight sync
  hands over: nested mappings or state objects (anything with .items()), mappings keyed by
  path tuples, lists / tuples (index as path part), leaves that are arrays or variable-like
  objects with the array in `.value`.  Integer path parts (layer indices) print as digits."""
  out = {}

  def is_node(x):
    return hasattr(x, 'items') and callable(x.items) and not hasattr(x, 'shape')

  def walk(prefix, node):
    if is_node(node):
      for k, v in node.items():
        parts = tuple(k) if isinstance(k, tuple) else (k,)
        walk(prefix + tuple(str(getattr(p, 'key', p)) for p in parts), v)
    elif isinstance(node, (list, tuple)) and not (node and isinstance(node[0], (int, float, np.number))):
      for i, v in enumerate(node):
        walk(prefix + (str(i),), v)
    else:
      name = '.'.join(prefix)
      if name.endswith('.value'):  # pure-dict dumps of variable objects
        name = name[:-len('.value')]
      if name in out:
        raise ValueError(f'duplicate parameter path {name!r}')
      out[name] = _leaf_array(node)

  walk((), tree)
  return out
