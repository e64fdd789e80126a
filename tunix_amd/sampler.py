"""Sampler with the reference's call surface, running the decode loop on the GPU.

Mirrors tunix/generate/sampler.py:205 ``Sampler`` (constructor :208-214,
``__call__`` :795-1080, ``transformer_state`` :267-359, ``update_params`` :361-392,
``tokenize`` :511-518, ``dtype`` :394-400) and base_sampler.py:59 ``BaseSampler``.
The jitted prefill / while_loop pair is replaced by ``tmx_decode_steps``: prompt
positions are walked through the same single-token step without the head (cache
fill), then every generation step runs with the fused head + token selection.
"""
import ctypes
import warnings

import numpy as np
import torch

from tunix_amd import _lib
from tunix_amd import utils
from tunix_amd.configs import CacheConfig, SamplerOutput
from tunix_amd.model import DecodeState, SAMPLE_GREEDY, SAMPLE_TOP_P, SAMPLE_SCORE

_REQUIRED_TOKENIZER_METHODS = ('encode', 'decode', 'bos_id', 'eos_id', 'pad_id')


class TokenizerAdapter:
  """Duck-typed tokenizer wrapper (tunix/generate/tokenizer_adapter.py:34): accepts
  any object with encode / decode / bos_id / eos_id / pad_id."""

  def __init__(self, tokenizer):
    missing = [m for m in _REQUIRED_TOKENIZER_METHODS if not hasattr(tokenizer, m)]
    if missing:
      raise ValueError(
          'Your tokenizer should have the following methods: '
          '`["encode", "decode", "bos_id", "eos_id", "pad_id"]`. Received: '
          f'`type(tokenizer)` = {type(tokenizer)}, with missing methods: {missing}.')
    self._tokenizer = tokenizer

  def encode(self, text, **kw):
    return self._tokenizer.encode(text, **kw)

  def decode(self, ids, **kw):
    return self._tokenizer.decode(ids, **kw)

  def bos_id(self):
    return self._tokenizer.bos_id()

  def eos_id(self):
    return self._tokenizer.eos_id()

  def pad_id(self):
    return self._tokenizer.pad_id()

  def dedup_bos_ids(self, ids):
    i = 0
    while i < len(ids) - 1 and ids[i] == ids[i + 1] == self.bos_id():
      i += 1
    return ids[i:]


def _seed_key(seed):
  """The two threefry key words (hi32, lo32) of a seed.  An int goes through
  jax.random.PRNGKey with 64-bit types disabled, as in the reference (sampler.py:938-941): the
  high word is 0 and the low word the seed's low 32 bits, negative seeds included.  A raw 2-word
  key (uint32[2]) passes through; a typed key array is unwrapped to its key data first."""
  if seed is None:
    seed = 0
  if isinstance(seed, (int, np.integer)):
    return 0, int(seed) & 0xFFFFFFFF
  for attr in ('_base_array', 'key_data'):  # jax typed keys (jax.random.key): the wrapped uint32[2]
    inner = getattr(seed, attr, None)
    if inner is not None and not callable(inner):
      seed = inner
      break
  arr = np.asarray(seed).astype(np.uint32).reshape(-1)
  if arr.size != 2:
    raise ValueError('seed must be an int or a 2-word key')
  return int(arr[0]), int(arr[1])


def shared_prompt_groups(ids, mask, min_len=32, max_group=64):
  """(g, n, c): the largest saving split of the rows into consecutive groups of g whose first c columns agree
  in token ids and mask, n = c rounded down to a multiple of 32; (1, 0, 0) when nothing is worth sharing.  A
  GRPO rollout decodes the G samples of a prompt as consecutive rows (tunix/rl/rl_learner.py:432-435 repeats
  every prompt num_generations times), so the K / V rows of the prompt columns are the same within a group:
  decode attention reads n of them once per group, and the cache fill computes c of them once per group.  The
  saving counted is (g - 1) / g * n cache rows."""
  ids, mask = np.asarray(ids), np.asarray(mask)
  b, p = ids.shape
  if b < 2 or p < min_len:
    return 1, 0, 0
  same = (ids[1:] == ids[:-1]) & (mask[1:] == mask[:-1])          # row i + 1 against row i, per column
  run = np.where(same.all(axis=1), p, np.argmin(same, axis=1))   # columns in which row i + 1 repeats row i
  best, best_gain = (1, 0, 0), 0.0
  for g in range(2, min(b, max_group) + 1):
    if b % g:
      continue
    inner = np.arange(1, b) % g != 0                              # pairs (i, i + 1) inside one group
    c = int(run[inner[: b - 1]].min())
    n = c // 32 * 32
    if n >= min_len and (g - 1) / g * n > best_gain:
      best, best_gain = (g, n, c), (g - 1) / g * n
  return best


class Sampler:
  """Sampler for an int4 QLoRA decoder resident on one MI355X."""

  # decode steps enqueued between two host checks of the `done` flags
  CHECK_EVERY = 32

  def __init__(self, transformer, tokenizer, cache_config: CacheConfig, image_processor=None):
    if image_processor is not None:
      raise NotImplementedError('image inputs are outside this decode path')
    self.tokenizer = tokenizer if isinstance(tokenizer, TokenizerAdapter) else TokenizerAdapter(tokenizer)
    self.cache_config = cache_config
    self._transformer = transformer
    c = transformer.config
    if (cache_config.num_layers, cache_config.num_kv_heads, cache_config.head_dim) != (
        c.num_layers, c.num_kv_heads, c.head_dim):
      raise ValueError('cache_config does not match the transformer configuration')
    self._lib = _lib.lib()  # raises if the HIP library is missing
    self._cache = None
    self._workspace = None
    self._nucleus_ws = None
    # replay one recorded decode step instead of launching every kernel: measured neutral on
    # MI355X (the steps are bound by the device, not by host launches), so off by default
    self.use_graph = False
    # read the cache rows of prompt columns once per group of rows with the same prompt (GRPO samples)
    self.share_prompt_kv = True
    self.eos_ids = None
    self.last_step_logits = None

  # -- reference surface -----------------------------------------------------
  @property
  def transformer(self):
    return self._transformer

  @property
  def transformer_state(self):
    """Flat dict of parameters: LoRA tensors by the reference's parameter paths."""
    return self._transformer.lora_state()

  @transformer_state.setter
  def transformer_state(self, state):
    self._transformer.update_lora(utils.flatten_state(state))

  def update_params(self, updated_weights, filter_types=None):
    """LoRA weight sync between rollouts.  RLEngine.sync_weights passes
    nnx.state(actor, nnx.LoRAParam) (tunix/rl/rl_cluster.py:1279-1294); the reference flattens
    it with to_flat_dict, casts to the rollout precision and merges it over the old parameters
    (tunix/generate/sampler.py:361-392).  Accepted here: a flat mapping under dotted names, a
    mapping keyed by path tuples, or a nested mapping / state object (anything with .items()),
    with array leaves or variable-like leaves that carry the array in `.value`.  Tensors are
    cast to bf16; a path the model does not have, or a tensor of another shape, raises the
    reference's "same structure" / "same shape" errors."""
    del filter_types
    flat = utils.flatten_state(updated_weights)
    merged = dict(self._transformer.lora_state())
    unknown = set(flat) - set(merged)
    if unknown:
      raise ValueError(f'New state must have the same structure as the old state. Unknown: {sorted(unknown)[:3]}')
    merged.update(flat)
    self._transformer.update_lora(merged)

  @property
  def dtype(self):
    return self._transformer.dtype

  def tokenize(self, input_string):
    ids = self.tokenizer.encode(input_string)
    bos = [self.tokenizer.bos_id()] if self.tokenizer.bos_id() else []
    return np.array(self.tokenizer.dedup_bos_ids(bos + list(ids)), dtype=np.int32)

  def delete_cache(self):
    self._cache = None
    self._lead_cache = None
    self._workspace = None

  def reinitialize_cache(self):
    pass

  # -- state ----------------------------------------------------------------
  def init_sample_state(self, all_input_ids, total_sampling_steps, include_logits,
                        forbidden_token_ids, temperature, top_p, top_k, seed, beam_size=None,
                        include_logprobs=False, prompt_lengths=None):
    """Device-side _SamplingState (tunix/generate/sampler.py:402-509)."""
    if beam_size is not None:
      raise NotImplementedError('beam search is outside this decode path')
    dev = self._transformer.device
    ids = np.asarray(all_input_ids, dtype=np.int32)
    b, p = ids.shape
    pad = self.tokenizer.pad_id()
    # Every column of the buffer is gathered from the embedding table at some step (pad columns
    # included), so every id must be a valid row.  The reference's JAX gather clamps silently.
    vocab = self._transformer.config.vocab_size
    if ids.size and (ids.min() < 0 or ids.max() >= vocab):
      bad = ids[(ids < 0) | (ids >= vocab)]
      raise ValueError(f'token id {int(bad[0])} is outside the vocabulary [0, {vocab}) '
                       '(prompt ids and the tokenizer\'s pad_id must be valid embedding rows)')
    if not 0 <= pad < vocab:
      raise ValueError(f'pad_id {pad} is outside the vocabulary [0, {vocab})')
    token_buffer = np.full((b, total_sampling_steps), pad, dtype=np.int32)
    token_buffer[:, :p] = ids
    input_mask = np.ones((b, total_sampling_steps), dtype=bool)
    if prompt_lengths is not None:
      lens = np.asarray(prompt_lengths).reshape(-1, 1)
      input_mask[:, :p] = np.arange(p)[None, :] >= (p - lens)
    else:
      input_mask[:, :p] = ids != pad
    positions = utils.build_positions_from_mask(input_mask)
    share = shared_prompt_groups(ids, input_mask[:, :p]) if self.share_prompt_kv else (1, 0, 0)
    c = self._transformer.config
    need = (c.num_layers, 2, b, self.cache_config.cache_size, c.num_kv_heads, c.head_dim)
    if self._cache is None or tuple(self._cache.shape) != need:
      self._cache = None
      self._cache = self._transformer.init_cache(b, self.cache_config.cache_size)
    else:
      self._cache.zero_()
    st = {
        'token_buffer': torch.from_numpy(token_buffer).to(dev),
        'input_mask_host': input_mask,
        'input_mask': torch.from_numpy(input_mask.astype(np.uint8)).to(dev),
        'positions_host': positions,
        'positions': torch.from_numpy(positions.astype(np.int32)).to(dev),
        'done': torch.zeros(b, dtype=torch.uint8, device=dev),
        'logprobs': torch.zeros(b, total_sampling_steps, dtype=torch.float32, device=dev)
                    if include_logprobs else None,
        'step': torch.zeros(1, dtype=torch.int32, device=dev),
        'cache': self._cache,
        'num_input_tokens': p,
        'share_group': share[0], 'share_len': share[1], 'share_common': share[2],
        'fresh': True,  # nothing walked yet: the cache fill may start with one pass per group of equal prompts
        'total_sampling_steps': total_sampling_steps,
        'sampling_mode': 'greedy' if top_p is None else 'top_p',
        'temperature': float(temperature),
        'top_p': top_p, 'top_k': top_k,
        'seed': _seed_key(seed),
        'forbidden': torch.tensor(list(forbidden_token_ids), dtype=torch.int32, device=dev)
                     if forbidden_token_ids else None,
        'eos': torch.tensor(np.asarray(self.eos_ids).reshape(-1), dtype=torch.int32, device=dev),
        'logits': torch.zeros(b, c.vocab_size, dtype=torch.float32, device=dev) if include_logits else None,
    }
    return st

  def _c_state(self, st, tokens_per_pass=1):
    b, total = st['token_buffer'].shape
    rows = b * max(tokens_per_pass, 1)
    if rows > self._max_rows():
      raise ValueError(
          f'{b} sequences x {max(tokens_per_pass, 1)} tokens per pass: this model takes at most {self._max_rows()} rows '
          '(4096 when every projection has K % 128 == 0, MoE models 8192 / experts per token, else 128)')
    ws_bytes = self._lib.tmx_decode_workspace_bytes(
        ctypes.byref(self._transformer.desc()), b * tokens_per_pass, self.cache_config.cache_size)
    if self._workspace is None or self._workspace.numel() < ws_bytes:
      # zero-filled: the first 256 bytes hold the status word tmx_decode_status reads
      self._workspace = torch.zeros(ws_bytes, dtype=torch.uint8, device=self._transformer.device)
    s = DecodeState()
    s.tokens_per_pass = tokens_per_pass
    s.share_group, s.share_len = st.get('share_group', 1), st.get('share_len', 0)
    s.batch, s.buf_len, s.cache_size = b, total, self.cache_config.cache_size
    s.token_buffer, s.positions = st['token_buffer'].data_ptr(), st['positions'].data_ptr()
    s.input_mask, s.done, s.step = st['input_mask'].data_ptr(), st['done'].data_ptr(), st['step'].data_ptr()
    s.logprobs = st['logprobs'].data_ptr() if st['logprobs'] is not None else None
    s.kv_cache = st['cache'].data_ptr()
    s.sampling_mode = {'greedy': SAMPLE_GREEDY, 'top_p': SAMPLE_TOP_P, 'score': SAMPLE_SCORE}[st['sampling_mode']]
    s.temperature = st['temperature']
    s.top_p = 1.0 if st['top_p'] is None else float(st['top_p'])
    s.top_k = int(st['top_k']) if st['top_k'] else 0
    s.seed_hi, s.seed_lo = st['seed']
    s.eos_ids, s.n_eos = st['eos'].data_ptr(), st['eos'].numel()
    if st['forbidden'] is not None:
      s.forbidden, s.n_forbidden = st['forbidden'].data_ptr(), st['forbidden'].numel()
    s.logits_out = st['logits'].data_ptr() if st['logits'] is not None else None
    s.workspace, s.workspace_bytes = self._workspace.data_ptr(), self._workspace.numel()
    if s.sampling_mode == SAMPLE_TOP_P and (s.top_p < 1.0 or s.top_k > 0):
      # the sorting branch of sample_top_p needs room for one sort key per logit
      nb = self._lib.tmx_nucleus_workspace_bytes(b, self._transformer.config.vocab_size)
      if nb == 0:
        raise _lib.TmxError('tmx_nucleus_workspace_bytes returned 0 (no device, or batch x vocab too large)')
      if self._nucleus_ws is None or self._nucleus_ws.numel() < nb:
        self._nucleus_ws = torch.empty(nb, dtype=torch.uint8, device=self._transformer.device)
      s.nucleus_workspace, s.nucleus_workspace_bytes = self._nucleus_ws.data_ptr(), self._nucleus_ws.numel()
    return s

  MAX_ROWS = 128        # rows of one pass that chooses tokens (sequences x tokens per pass)
  MAX_FILL_ROWS = 4096  # rows of one cache-fill or scoring pass of a dense model (256-row projection blocks)

  MAX_MOE_PAIRS = 8192  # routed (token, expert) pairs of one pass of a MoE model
  MAX_PASSES_IN_FLIGHT = 64  # passes a walk enqueues before it waits for the stream

  def _max_rows(self):
    """Rows one pass can take: more than 128 need the 256-row projection blocks (every attention /
    dense-MLP projection with K % 128 == 0); MoE models are bounded by the routed pairs per pass."""
    cfg = self._transformer.config
    ks = [cfg.embed_dim, cfg.num_heads * cfg.head_dim] + ([] if cfg.num_experts else [cfg.hidden_dim])
    if not all(k % 128 == 0 for k in ks):
      return 128
    if cfg.num_experts:
      return max(128, min(4096, self.MAX_MOE_PAIRS // cfg.num_experts_per_tok))
    return 4096

  def _many_rows_ok(self):
    return self._max_rows() > 128

  def _fill_rows(self):
    return max(self.MAX_ROWS, min(self.MAX_FILL_ROWS, self._max_rows()))

  def walk(self, st, n_tokens, sample=False):
    """Advances every sequence by n_tokens known tokens (cache fill over a prompt, or scoring
    when st['sampling_mode'] == 'score') in passes of as many tokens per sequence as fit
    MAX_ROWS rows (MAX_FILL_ROWS without the head, where the model allows), instead of one
    token per launch sequence."""
    b = st['token_buffer'].shape[0]
    if st.get('fresh') and not sample and st.get('share_group', 1) > 1:
      n_lead = min(n_tokens, st['share_common'])
      if n_lead >= 32:
        self._walk_group_leaders(st, n_lead)
        n_tokens -= n_lead
    st['fresh'] = False
    # the head chooses tokens for up to MAX_ROWS rows; scoring takes as many rows as a cache fill
    choose = sample and st['sampling_mode'] != 'score'
    per = min(128, max(1, (self.MAX_ROWS if choose else self._fill_rows()) // b))
    passes = 0
    while n_tokens > 0:
      t = min(per, n_tokens)
      self.run_steps(st, 1, sample=sample, tokens_per_pass=t)
      n_tokens -= t
      passes += 1
      if passes % self.MAX_PASSES_IN_FLIGHT == 0:
        # bound the queue of pending launches (a pass is a few hundred of them): a walk of
        # thousands of short passes otherwise leaves tens of thousands of dispatches pending at once
        torch.cuda.current_stream().synchronize()

  def _walk_group_leaders(self, st, n):
    """Cache fill over the first n columns, which every group of st['share_group'] consecutive rows has in
    common (the samples of one prompt): the first row of every group is walked, in a cache of its own, and
    its K / V rows are copied to the cache rows of the whole group, so the prompt is computed once per group
    instead of once per sample.  Advances st['step'] by n like a walk over all rows."""
    g = st['share_group']
    b = st['token_buffer'].shape[0]
    dev = self._transformer.device
    lead = torch.arange(0, b, g, device=dev)
    c = self._transformer.config
    need = (c.num_layers, 2, b // g, self.cache_config.cache_size, c.num_kv_heads, c.head_dim)
    if getattr(self, '_lead_cache', None) is None or tuple(self._lead_cache.shape) != need:
      self._lead_cache = None
      self._lead_cache = self._transformer.init_cache(b // g, self.cache_config.cache_size)
    sub = dict(st)
    sub.update({
        'token_buffer': st['token_buffer'][lead].contiguous(), 'positions': st['positions'][lead].contiguous(),
        'input_mask': st['input_mask'][lead].contiguous(), 'done': torch.zeros(b // g, dtype=torch.uint8, device=dev),
        'logprobs': None, 'logits': None, 'step': torch.zeros(1, dtype=torch.int32, device=dev),
        'cache': self._lead_cache, 'share_group': 1, 'share_len': 0, 'share_common': 0, 'fresh': False})
    self.walk(sub, n)
    for r in range(g):  # rows r, r + g, ... of the cache <- the leaders' rows (strided copies, no temporary)
      st['cache'][:, :, r::g, :n].copy_(self._lead_cache[:, :, :, :n])
    st['step'].fill_(n)

  def run_steps(self, st, n_steps, sample=True, graph=False, tokens_per_pass=1):
    """Runs n decode-loop iterations on the current stream.  graph=False only enqueues (no host
    sync); graph=True replays one recorded step and returns when the steps have run.
    tokens_per_pass > 1: every iteration consumes that many known tokens of each sequence
    (cache fill or scoring only)."""
    if n_steps <= 0:
      return
    st['fresh'] = False
    cs = self._c_state(st, tokens_per_pass)
    fn = self._lib.tmx_decode_steps_graph if graph else self._lib.tmx_decode_steps
    rc = fn(ctypes.byref(self._transformer.desc()), ctypes.byref(cs), _lib.stream(), int(n_steps),
            1 if sample else 0)
    _lib.check(rc, 'tmx_decode_steps_graph' if graph else 'tmx_decode_steps')

  def check_device_status(self, st):
    """Waits for the stream and raises if a bounded wait inside a kernel ran out since the last
    check (tmx_decode_status); called before results are handed to the caller."""
    cs = self._c_state(st)
    rc = self._lib.tmx_decode_status(ctypes.byref(self._transformer.desc()), ctypes.byref(cs), _lib.stream())
    _lib.check(rc, 'tmx_decode_status')

  def per_token_logps(self, prompt_tokens, completion_tokens, pad_id=None, temperature=1.0, token_mask=None):
    """Teacher-forced log-probabilities of the completion tokens, f32 [B, completion_len]:
    log_softmax(logits / temperature)[token] at every completion position given everything
    before it (tunix/rl/common.py:426-606 compute_per_token_logps without sequence packing;
    positions and the attention mask follow process_ids, :257-330: valid = token != pad_id or
    `token_mask`).  Entries at padded completion positions are computed like the reference's
    and meant to be masked by the caller.  The sequence is walked token by token through the
    decode kernels."""
    prompt = np.asarray(prompt_tokens, dtype=np.int32)
    comp = np.asarray(completion_tokens, dtype=np.int32)
    if prompt.ndim != 2 or comp.ndim != 2 or prompt.shape[0] != comp.shape[0]:
      raise ValueError('prompt_tokens and completion_tokens must be [B, P] and [B, T]')
    pad = self.tokenizer.pad_id() if pad_id is None else pad_id
    ids = np.concatenate([prompt, comp], axis=1)
    b, total = ids.shape
    p, t = prompt.shape[1], comp.shape[1]
    if total > self.cache_config.cache_size:
      raise ValueError(f'Total sampling steps {total} must be less than the cache size'
                       f' {self.cache_config.cache_size}.')
    if p == 0:
      raise ValueError('prompt_tokens must hold at least one column (packed sequences are not supported)')
    if t == 0:
      return np.zeros((b, 0), np.float32)
    valid = (ids != pad) if token_mask is None else np.asarray(token_mask).astype(bool)
    if valid.shape != ids.shape:
      raise ValueError('token_mask must match the full prompt/completion shape')
    self.eos_ids = np.array([-1])
    st = self.init_sample_state(ids, total, False, None, temperature if temperature not in (0.0, 1.0) else 1.0,
                                1.0, None, 0, include_logprobs=True)
    dev = self._transformer.device
    st['input_mask'] = torch.from_numpy(valid.astype(np.uint8)).to(dev)
    st['positions'] = torch.from_numpy(utils.build_positions_from_mask(valid).astype(np.int32)).to(dev)
    st['sampling_mode'] = 'score'
    self.walk(st, p - 1)
    self.walk(st, t, sample=True)
    self.check_device_status(st)
    return st['logprobs'][:, p:p + t].cpu().numpy()

  # -- the call ---------------------------------------------------------------
  def __call__(self, input_strings=None, max_generation_steps=0, max_prompt_length=None, echo=False,
               return_logits=False, return_logprobs=False, eos_tokens=None, forbidden_tokens=None,
               temperature=0.0, top_p=None, top_k=None, beam_size=None, seed=None, pad_output=False,
               images=None, audios=None, max_audio_length=None, max_audio_clips=None, *,
               prompt_token_ids=None):
    if images is not None or audios is not None:
      raise NotImplementedError('image / audio inputs are outside this decode path')
    if return_logits and echo:
      # the reference slices its logits buffer from the first prompt token on (sampler.py:1045-1052);
      # the cache fill here computes no prompt logits, so only generated-step logits exist
      raise NotImplementedError('return_logits with echo=True needs prompt-position logits, which the cache fill '
                                'does not compute; call with echo=False')
    self.eos_ids = np.array(list(eos_tokens) if eos_tokens else [self.tokenizer.eos_id()])
    exact_input = prompt_token_ids is not None
    tokens = utils.resolve_prompt_tokens(
        input_strings, prompt_token_ids, self.tokenize,
        max_generation_steps=max_generation_steps,
        max_total_length=self.cache_config.cache_size,
        max_length_name='cache_size',
        single_output_per_row=beam_size is None)
    if beam_size is not None:
      raise NotImplementedError('beam search is outside this decode path')
    forbidden = tuple(forbidden_tokens) if forbidden_tokens else None
    all_input_ids, prompt_lengths, max_prompt_length = utils.left_pad_prompt_tokens(
        tokens, max_prompt_length, self.tokenizer.pad_id(),
        max_allowed_length=self.cache_config.cache_size - max_generation_steps)
    total = max_prompt_length + max_generation_steps
    if total > self.cache_config.cache_size:
      raise ValueError(f'Total sampling steps {total} must be less than the cache size'
                       f' {self.cache_config.cache_size}.')
    st = self.init_sample_state(
        all_input_ids, total, return_logits, forbidden, temperature, top_p, top_k, seed, beam_size,
        include_logprobs=return_logprobs, prompt_lengths=prompt_lengths if exact_input else None)
    p = max_prompt_length
    logits_steps = []
    if max_generation_steps > 0:
      # cache fill over prompt columns 0 .. P-2, then P-1 produces generated token #1
      self.walk(st, p - 1)
      remaining = max_generation_steps
      while remaining > 0:
        n = 1 if return_logits else min(self.CHECK_EVERY, remaining)
        self.run_steps(st, n, sample=True, graph=self.use_graph)
        remaining -= n
        if return_logits:
          logits_steps.append(st['logits'].clone())
        if remaining > 0 and bool(st['done'].all().item()):
          break
    self.check_device_status(st)
    token_buffers = st['token_buffer'].cpu().numpy()
    logprob_buffers = st['logprobs'].cpu().numpy() if return_logprobs else None
    if return_logits and logits_steps:
      self.last_step_logits = logits_steps[-1]
      gen_logits = torch.stack(logits_steps, dim=1).cpu().numpy()  # [B, steps, V]
    else:
      gen_logits = None
    pad = self.tokenizer.pad_id()

    def bounds(row, prompt_length):
      if not echo:
        start = p
      elif exact_input:
        start = p - int(prompt_length)
      else:
        start = utils.find_first_non_pad_idx(row, pad)
      end = utils.find_first_eos_idx(row[p:], self.eos_ids) + p
      return start, end

    out_tokens, out_logits, out_logprobs = [], [], []
    max_len = total if echo else max_generation_steps
    for i, row in enumerate(token_buffers):
      start, end = bounds(row, prompt_lengths[i])
      toks = row[start:end]
      if pad_output:
        toks = utils.pad_to_length(toks, max_len, pad)
      out_tokens.append(toks)
      if gen_logits is not None:
        lg = gen_logits[i][: max(end - p, 0)]
        out_logits.append(lg)
      if return_logprobs:
        lp = logprob_buffers[i][start:end]
        if pad_output:
          lp = np.pad(lp, (0, max_len - len(lp)), mode='constant', constant_values=0.0)
        out_logprobs.append(lp.tolist())
    if pad_output:
      lengths = [bounds(r, prompt_lengths[i])[1] - bounds(r, prompt_lengths[i])[0]
                 for i, r in enumerate(token_buffers)]
      decoded = [self.tokenizer.decode(t[:n].tolist()) for t, n in zip(out_tokens, lengths)]
      out_tokens = np.stack(out_tokens) if out_tokens else out_tokens
    else:
      decoded = [self.tokenizer.decode(t.tolist()) for t in out_tokens]
    return SamplerOutput(
        text=decoded,
        logits=out_logits if return_logits else [],
        tokens=out_tokens,
        padded_prompt_tokens=all_input_ids,
        logprobs=out_logprobs if return_logprobs else None,
        prompt_lengths=prompt_lengths,
    )
