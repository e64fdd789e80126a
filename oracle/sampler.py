"""The Sampler's prefill + decode loop restated (test infrastructure only).

tunix/generate/sampler.py:402-509 (init_sample_state), :520-599 (_sample),
:601-730 (_prefill_fn), :732-793 (_decode_fn / _sample_step), :931-1080
(__call__ epilogue).  Beam search, images and logits buffers are not restated.
"""
import numpy as np

from oracle import masks, prng, sampling
from oracle import model as M


class SamplingState:
  pass


def init_sample_state(cfg, all_input_ids, total_sampling_steps, cache_size, pad_id,
                      temperature, top_p, top_k, seed_key, prompt_lengths=None,
                      forbidden=None):
  b, p = all_input_ids.shape
  st = SamplingState()
  st.token_buffer = np.full((b, total_sampling_steps), pad_id, np.int32)
  st.token_buffer[:, :p] = all_input_ids
  st.input_mask = np.ones((b, total_sampling_steps), bool)
  if prompt_lengths is not None:
    st.input_mask[:, :p] = np.arange(p)[None, :] >= (p - np.asarray(prompt_lengths)[:, None])
  else:
    st.input_mask[:, :p] = all_input_ids != pad_id
  st.positions = masks.build_positions_from_mask(st.input_mask)
  st.done = np.zeros((b,), bool)
  st.cache = M.init_cache(cfg, b, cache_size)
  st.logprobs_buffer = np.zeros((b, total_sampling_steps), np.float32)
  st.decoding_step = p - 1
  st.num_input_tokens = p
  st.total_sampling_steps = total_sampling_steps
  st.temperature, st.top_p, st.top_k = temperature, top_p, top_k
  st.sampling_mode = 'greedy' if top_p is None else 'top_p'
  st.seed = seed_key
  st.forbidden = tuple(forbidden) if forbidden else None
  st.margins = []  # top-2 logit margin per step (for tie-aware comparisons)
  st.step_logits = []
  return st


def _sample(logits, eos, st, keep_logits=False):
  """sampler.py:520-599.  logits f32 [B, T, V]; uses the last position."""
  z = sampling.apply_forbidden(logits[:, -1], st.forbidden)
  if st.sampling_mode == 'greedy':
    tok, logp = sampling.sample_best(z)
  else:
    key = prng.fold_in(st.seed, st.decoding_step)
    tok, logp = sampling.sample_top_p(z, key, st.temperature, st.top_p, st.top_k)
  srt = np.sort(z, axis=-1)
  st.margins.append((srt[:, -1] - srt[:, -2]).astype(np.float32))
  if keep_logits:
    st.step_logits.append(z.copy())
  st.token_buffer[:, st.decoding_step + 1] = tok
  st.logprobs_buffer[:, st.decoding_step + 1] = logp
  st.done = st.done | np.isin(st.token_buffer[:, st.decoding_step + 1], eos)
  st.decoding_step += 1
  return st


def prefill(model, st, cache_size, eos, keep_logits=False):
  p = st.num_input_tokens
  mask = masks.make_causal_attn_mask(st.input_mask[:, :p], cache_size)
  logits, st.cache = model(st.token_buffer[:, :p], st.positions[:, :p], st.cache, mask)
  return _sample(logits, eos, st, keep_logits)


def decode(model, st, cache_size, eos, keep_logits=False, max_steps=None):
  n = 0
  while st.decoding_step < st.total_sampling_steps - 1 and not st.done.all():
    if max_steps is not None and n >= max_steps:
      break
    step = st.decoding_step
    last = st.token_buffer[:, step:step + 1]
    pos = st.positions[:, step:step + 1]
    mask = masks.compute_attention_masks(step, cache_size, ~st.input_mask)
    logits, st.cache = model(last, pos, st.cache, mask)
    _sample(logits, eos, st, keep_logits)
    n += 1
  return st


def generate(model, cfg, prompt_ids, max_generation_steps, cache_size, pad_id=0, eos_ids=(-1,),
             max_prompt_length=None, temperature=0.0, top_p=None, top_k=None, seed=None,
             forbidden=None, exact_input=True, keep_logits=False):
  """sampler.py:795-1080 for token-id prompts, echo=False, pad_output=False.
  Returns dict(tokens, logprobs, padded_prompt_tokens, prompt_lengths, state)."""
  eos = np.asarray(list(eos_ids))
  ids, lens, p = masks.left_pad_prompt_tokens(
      prompt_ids, max_prompt_length, pad_id, max_allowed_length=cache_size - max_generation_steps)
  total = p + max_generation_steps
  if total > cache_size:
    raise ValueError(f'Total sampling steps {total} must be less than the cache size {cache_size}.')
  key = prng.prng_key(0 if seed is None else seed)
  st = init_sample_state(cfg, ids, total, cache_size, pad_id, temperature, top_p, top_k, key,
                         prompt_lengths=lens if exact_input else None, forbidden=forbidden)
  prefill(model, st, cache_size, eos, keep_logits)
  decode(model, st, cache_size, eos, keep_logits)
  toks, lps = [], []
  for i in range(ids.shape[0]):
    end = masks.find_first_eos_idx(st.token_buffer[i, p:], eos) + p
    toks.append(st.token_buffer[i, p:end].copy())
    lps.append(st.logprobs_buffer[i, p:end].copy())
  return dict(tokens=toks, logprobs=lps, padded_prompt_tokens=ids, prompt_lengths=lens, state=st)
