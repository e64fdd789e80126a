"""Benchmark of the decode path: generated tokens/s of an int4 QLoRA rollout on one MI355X.

A "step" is one decode-loop iteration over the whole batch (one new token per
sequence).  Default workload: Llama-3.1-8B shape, 64 sequences (8 prompts x 8
samples), 256-token prompts, temperature 0.9, top-p 1.0, per-token logprobs,
bf16 KV cache.  The timed region is centred on the workload's mean context
(prompt + new / 2): the default run times nearly the whole generation (context
271 -> 767); a shorter run (--steps 20) first fills the cache up to the start of its
window with known tokens, in multi-token passes, so it measures the same mean context.
Prints one JSON line.

  python bench.py --pmc-summary CSV COUNTER [--match TEXT]   per-kernel means of one hardware
      counter from a rocprofv3 counter-collection CSV (how profiles/ summaries are made)
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: (config factory, batch, prompt, new tokens, group, rank, temperature, top_p)
    'llama3.1-8b-grpo': ('llama3p1_8b', 64, 256, 512, 64, 16, 0.9, 1.0),
    'llama3.2-1b-b1': ('llama3p2_1b', 1, 256, 512, 64, 16, 1.0, 1.0),
    'toy': ('toy', 4, 32, 32, 64, 8, 0.9, 1.0),
    # large-batch rollout with nucleus sampling, and the MoE shape (LoRA on attention only)
    'qwen3-8b-b128': ('qwen3_8b', 128, 512, 1024, 128, 32, 1.0, 0.95),
    'qwen3-30b-a3b-moe': ('qwen3_30b_a3b', 32, 256, 512, 64, 8, 0.9, 1.0),
}
ATTN_ONLY_LORA = {'qwen3-30b-a3b-moe'}
LABELS = {'llama3.1-8b-grpo': '8B', 'llama3.2-1b-b1': '1B single-sequence', 'toy': 'toy',
          'qwen3-8b-b128': 'Qwen3-8B 128-sequence', 'qwen3-30b-a3b-moe': 'Qwen3-30B-A3B MoE'}

CLASS_NAMES = ['row_norm', 'qkv_linear', 'rope_kvwrite', 'attention', 'o_linear', 'gate_up_linear',
               'swiglu', 'down_linear', 'head_sample', 'advance_step', 'empty_launch', 'router']


def linear_bytes(pl, batch, frac=1.0):
  """int4 + scales + LoRA A, B (+ activations in and out, counted for the GEMM regime).
  frac: expected fraction of a stacked expert matrix that a step touches."""
  b = int((pl.k * pl.n // 2 + (pl.k // pl.group) * pl.n * 2) * (frac if pl.experts > 1 else 1.0))
  if pl.lora_a_t is not None:
    b += 2 * pl.rank * (pl.k * len(pl.seg_cols) + pl.n)
  return b + batch * (pl.k + pl.n) * 2


def cpu_baseline(workload, n_layers=2):
  """One decode step of the CPU oracle (dequantise -> bf16 matmul, attention over the whole
  cache, f32 log-softmax) at the workload's shapes on `n_layers` layers + head, scaled to
  the full depth.  Reported beside the GPU number, not a target."""
  import torch
  from oracle import model as OM
  from oracle import masks as OMK
  from oracle import sampling as OS
  name, batch, prompt, new, group, rank, temp, _ = WORKLOADS[workload]
  from tunix_amd.model import ModelConfig
  c = getattr(ModelConfig, name)()
  full_layers = c.num_layers
  # the layers are timed with a tiny vocabulary (the embedding is only gathered); the head
  # matrix of the real shape is a tiled random block (values do not affect the timing)
  ocfg = OM.Config(c.family, min(n_layers, full_layers), 32, c.embed_dim, c.hidden_dim,
                   c.num_heads, c.head_dim, c.num_kv_heads, c.rope_theta, c.norm_eps, True)
  w = OM.random_weights(ocfg, 0, group, rank, 2.0 * rank,
                        ('q', 'k', 'v', 'o', 'gate', 'up', 'down'))
  dec = OM.Decoder(ocfg, w)
  cache_size = prompt + new
  step = prompt + new // 2
  cache = OM.init_cache(ocfg, batch, cache_size)
  rng = np.random.default_rng(0)
  for lc in cache.values():
    lc['end_index'][:] = step
    lc['k'][:, :step] = rng.standard_normal((batch, step, c.num_kv_heads, c.head_dim), dtype=np.float32)
    lc['v'][:, :step] = lc['k'][:, :step]
  block = (rng.standard_normal((c.embed_dim, 1002), dtype=np.float32) * np.float32(0.02))
  reps = -(-c.vocab_size // 1002)
  head = np.ascontiguousarray(np.tile(block, (1, reps))[:, :c.vocab_size])
  x = rng.standard_normal((batch, 1, c.embed_dim), dtype=np.float32)
  pos = np.full((batch, 1), step, np.int32)
  mask = OMK.compute_attention_masks(step, cache_size, np.zeros((batch, cache_size), bool))
  from oracle import layers as L
  t_layers0 = time.perf_counter()
  for i, lw in enumerate(dec.w['layers']):
    lc, a = dec._attn(lw, dec._norm(x, lw['norm1']), pos, cache[f'layer_{i}'], mask)
    h = dec.pol.r(a + x)
    m = L.swiglu_mlp(dec._norm(h, lw['norm2']), lw['gate'], lw['up'], lw['down'], dec.pol, 'reference')
    x = dec.pol.r(h + m)
  t_layers = time.perf_counter() - t_layers0
  t_head0 = time.perf_counter()
  xn = dec._norm(x, dec.w['final_norm'])
  logits = dec.pol.r(xn @ head)
  OS.log_softmax(logits[:, -1] / np.float32(temp))
  t_head = time.perf_counter() - t_head0
  step_s = t_layers * full_layers / ocfg.num_layers + t_head
  return {
      'value': batch / step_s,
      'unit': 'tokens/s',
      'cores': int(os.environ.get('OMP_NUM_THREADS', torch.get_num_threads())),
      'kind': 'port',
      'sample': (f'CPU restatement (numpy), not tunix/JAX: 1 decode step at context {step}, '
                 f'{ocfg.num_layers} of {full_layers} layers timed ({t_layers:.2f} s) and scaled, '
                 f'+ head ({t_head:.2f} s); os.cpu_count()={os.cpu_count()}'),
  }


def pmc_summary(path, counter, match=None, top=16):
  """Prints, for every kernel symbol of a rocprofv3 counter-collection CSV, the number of
  dispatches and the mean / max of `counter` over them (template arguments kept, argument
  lists dropped)."""
  import collections
  import csv
  agg = collections.defaultdict(list)
  with open(path) as f:
    for row in csv.DictReader(f):
      if row['Counter_Name'] != counter or (match and match not in row['Kernel_Name']):
        continue
      agg[row['Kernel_Name'].split('(')[0]].append(float(row['Counter_Value']))
  rows = sorted(agg.items(), key=lambda kv: -sum(kv[1]))[:top]
  for k, v in rows:
    print(f"{counter} {k[:80]:80s} launches {len(v):7d} mean {sum(v) / len(v):14.1f} max {max(v):14.1f}")


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument('--pmc-summary', nargs=2, metavar=('CSV', 'COUNTER'), default=None,
                  help='summarise one counter of a rocprofv3 counter-collection CSV per kernel and exit (no GPU)')
  ap.add_argument('--match', default=None, help='--pmc-summary: only kernels whose name contains this text')
  ap.add_argument('--gpus', type=int, default=1)
  ap.add_argument('--steps', type=int, default=496)
  ap.add_argument('--warmup', type=int, default=16)
  ap.add_argument('--workload', default='llama3.1-8b-grpo', choices=sorted(WORKLOADS))
  ap.add_argument('--sequences', type=int, default=0,
                  help='override the number of sequences of the workload (the headline metric is the default)')
  ap.add_argument('--scoring', action='store_true',
                  help='time the scoring pass instead (Sampler.per_token_logps over prompt + new tokens of every '
                       'sequence): a separate JSON line, not the headline metric')
  ap.add_argument('--no-kv-sharing', action='store_true',
                  help='read the prompt slots per sequence even where consecutive rows hold samples of one prompt')
  ap.add_argument('--no-cpu-baseline', action='store_true')
  ap.add_argument('--no-profile', action='store_true')
  ap.add_argument('--graph', action='store_true', help='replay one recorded decode step (tmx_decode_steps_graph)')
  ap.add_argument('--sync-steps', action='store_true',
                  help='synchronise after every decode step (counter-collection runs: the profiler '
                       'cannot hold tens of thousands of pending dispatches)')
  ap.add_argument('--pmc-calibrate', action='store_true',
                  help='also run one 1 GiB device copy (a kernel of known traffic) to scale PMC counters')
  args = ap.parse_args()
  if args.pmc_summary:
    pmc_summary(args.pmc_summary[0], args.pmc_summary[1], args.match)
    return
  if args.gpus != 1:
    print('bench.py: this build runs on ONE GPU (no collectives, no sharding); --gpus must be 1',
          file=sys.stderr)
    sys.exit(2)

  import torch
  from tunix_amd import _lib
  from tunix_amd.configs import CacheConfig
  from tunix_amd.model import ModelConfig, QLoRAModel
  from tunix_amd.sampler import Sampler

  name, batch, prompt, new, group, rank, temp, top_p = WORKLOADS[args.workload]
  if args.sequences > 0:
    batch = args.sequences
  if args.steps + args.warmup > new:
    print(f'bench.py: steps + warmup must be <= {new} new tokens of the workload', file=sys.stderr)
    sys.exit(2)
  cfg = getattr(ModelConfig, name)()
  torch.cuda.set_device(0)
  targets = ('q_proj', 'k_proj', 'v_proj', 'o_proj')
  if args.workload not in ATTN_ONLY_LORA:
    targets += ('gate_proj', 'up_proj', 'down_proj')
  model = QLoRAModel.random_init(cfg, seed=0, group=group, lora_rank=rank, lora_alpha=2.0 * rank,
                                 lora_targets=targets)
  cache_size = prompt + new

  class _Tok:  # ids only: the benchmark feeds token ids and never decodes text
    def encode(self, s): return [int(t) for t in s.split()]
    def decode(self, ids): return ''
    def pad_id(self): return 0
    def bos_id(self): return 1
    def eos_id(self): return -1

  sampler = Sampler(model, _Tok(), CacheConfig(cache_size, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim))
  sampler.eos_ids = np.array([-1])  # unreachable: every row runs the full length
  sampler.share_prompt_kv = not args.no_kv_sharing
  rng = np.random.default_rng(0)
  # GRPO workloads: G = 8 samples of a prompt are consecutive rows; the others: distinct prompts
  n_prompts = max((batch + 7) // 8, 1) if 'grpo' in args.workload else batch
  base = rng.integers(3, cfg.vocab_size, (n_prompts, prompt)).astype(np.int32)
  ids = np.repeat(base, -(-batch // n_prompts), axis=0)[:batch]  # G samples of a prompt are consecutive rows

  if args.scoring:
    # Teacher forcing over whole sequences (tunix/rl/common.py:426-606): prompt cache fill + scored completion.
    comp = rng.integers(3, cfg.vocab_size, (batch, new)).astype(np.int32)
    times = []
    for _ in range(3):
      torch.cuda.synchronize()
      t0 = time.perf_counter()
      lp = sampler.per_token_logps(ids, comp, pad_id=0, temperature=1.0)
      torch.cuda.synchronize()
      times.append(time.perf_counter() - t0)
    assert lp.shape == (batch, new) and np.isfinite(lp).all() and (lp <= 0).all()
    dt = min(times[1:])
    print(json.dumps({
        'metric': 'scored tokens/s at 1 GPU, int4 QLoRA scoring pass (per-token log-probs)',
        'value': batch * (prompt + new) / dt, 'unit': 'tokens/s', 'n_gpus': 1, 'ms_per_pass': dt * 1e3,
        'higher_is_better': True, 'vs_baseline': None,
        'dtype': 'bf16 activations / int4 weights / f32 accumulate',
        'data': 'synthetic (random-init weights, uniform-random token ids)',
        'config': {'workload': args.workload, 'shape': name, 'sequences': batch, 'prompt_len': prompt,
                   'scored_tokens': new, 'quant': f'int4 group {group}', 'lora_rank': rank,
                   'rows_per_pass': min(sampler._fill_rows() // batch, 128) * batch},
    }))
    return

  walk_ms = []
  # The timed window [start + warmup, start + warmup + steps) is centred on the workload's mean
  # context prompt + new / 2.  A run shorter than the generation stands in for its middle: the
  # columns between the prompt and `start` hold known (random) tokens, as if already generated,
  # and are walked by the same cache fill as the prompt.
  start = max(prompt, prompt + (new - args.steps) // 2 - args.warmup)
  filled = np.concatenate([ids, rng.integers(3, cfg.vocab_size, (batch, start - prompt)).astype(np.int32)], axis=1)

  def fresh_state():
    st = sampler.init_sample_state(filled, prompt + new, False, None, temp, top_p, None, 0,
                                   include_logprobs=True, prompt_lengths=np.full(batch, start))
    # cache fill over the known tokens (outside the timed region), in multi-token passes
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    if args.sync_steps:
      run(st, start - 1, False)
    else:
      sampler.walk(st, start - 1)
    torch.cuda.synchronize()
    walk_ms.append((time.perf_counter() - t0) * 1e3)
    return st

  def run(st, n, sample=True):
    if not args.sync_steps:
      return sampler.run_steps(st, n, sample=sample, graph=args.graph)
    for _ in range(n):
      sampler.run_steps(st, 1, sample=sample)
      torch.cuda.synchronize()

  if args.pmc_calibrate:
    src = torch.empty(1 << 30, dtype=torch.uint8, device='cuda')
    dst = torch.empty_like(src)
    dst.copy_(src)  # reads 1 GiB, writes 1 GiB
    torch.cuda.synchronize()
    del src, dst
  def timed_run():
    st = fresh_state()
    run(st, args.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run(st, args.steps)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    toks = st['token_buffer'][:, start:start + args.warmup + args.steps]
    assert int(st['step'].item()) == start - 1 + args.warmup + args.steps
    assert bool(((toks >= 0) & (toks < cfg.vocab_size)).all().item())
    lps = st['logprobs'][:, start:start + args.warmup + args.steps]
    assert bool(torch.isfinite(lps).all().item()) and bool((lps <= 0).all().item())
    # a hand-over inside a launch whose bounded wait ran out would have dropped a LoRA term: raises if so
    sampler.check_device_status(st)
    return st, dt

  # The product's own path first: where consecutive rows hold samples of one prompt (the GRPO workload), decode
  # attention reads the prompt slots once per group.  Every roofline figure below prices the K/V bytes at
  # sequences x context and therefore comes from a second run WITHOUT that sharing (the same launches otherwise).
  st, dt = timed_run()
  shared = (st['share_group'], st['share_len']) if st['share_group'] > 1 else None
  dt_product, walk_product = dt, walk_ms[0]
  if shared:
    sampler.share_prompt_kv = False
    walk_ms.clear()
    st, dt = timed_run()

  result = {
      'metric': f'generated tokens/s at 1 GPU, int4 QLoRA {LABELS[args.workload]} rollout (decode)',
      'value': batch * args.steps / dt_product,
      'unit': 'tokens/s',
      'n_gpus': 1,
      'steps': args.steps,
      'warmup': args.warmup,
      'ms_per_step': dt_product / args.steps * 1e3,
      'higher_is_better': True,
      'scaling': 'weak',
      'vs_baseline': None,
      'cache_fill_ms': walk_product,
      'dtype': 'bf16 activations / int4 weights / f32 accumulate',
      'data': 'synthetic (random-init weights, uniform-random prompt ids)',
      'config': {
          'workload': args.workload,
          'shape': name, 'sequences': batch, 'prompt_len': prompt, 'new_tokens': new,
          'quant': f'int4 group {group}', 'lora_rank': rank, 'temperature': temp, 'top_p': top_p,
          'context_range': [start - 1 + args.warmup, start - 1 + args.warmup + args.steps],
          'cache_filled_to': start,
      },
  }

  # Whole-step algorithmic bytes at the mean context of the timed region.
  wbytes, hbytes = model.weight_bytes(batch)
  s_mean = start + args.warmup + args.steps / 2.0
  kv_per_tok = cfg.num_layers * cfg.num_kv_heads * cfg.head_dim * 2 * 2
  step_bytes = wbytes + hbytes + batch * s_mean * kv_per_tok
  result['step_hbm'] = {'algorithmic_bytes': step_bytes,
                        'achieved_GBps': step_bytes / (dt / args.steps) / 1e9,
                        'frac_of_8TBps': step_bytes / (dt / args.steps) / 8e12}
  if shared:
    # beside, not inside, the figures priced at sequences x context: step_hbm, roofline and kernel_ms_per_step are
    # the run without sharing; `value` / `ms_per_step` are the product's default path (sharing on)
    result['prompt_kv_sharing'] = {
        'share_group': shared[0], 'share_len': shared[1],
        'value': batch * args.steps / dt_product, 'ms_per_step': dt_product / args.steps * 1e3,
        'value_without': batch * args.steps / dt, 'ms_per_step_without': dt / args.steps * 1e3,
        'kv_rows_read_per_step_ratio': (batch * (s_mean - shared[1]) + batch / shared[0] * shared[1]) / (batch * s_mean),
        'cache_fill_ms': walk_product, 'cache_fill_ms_without': walk_ms[0],
        'note': 'step_hbm, roofline* and kernel_ms_per_step below are measured WITHOUT sharing (K/V bytes priced at '
                'sequences x context); value and ms_per_step are the default path, which reads the prompt slots '
                'once per group of samples of one prompt'}

  if not args.no_profile:
    # Replay the same rollout with HIP events around every launch: every 8th step of a long run,
    # every step of a short one.
    lib = _lib.lib()
    st = fresh_state()
    sampler.run_steps(st, args.warmup, sample=True)
    ms = np.zeros(len(CLASS_NAMES), np.float32)
    cnt = np.zeros(len(CLASS_NAMES), np.int32)
    tot_ms = np.zeros_like(ms)
    tot_cnt = np.zeros_like(cnt)
    ctx_sum, ctx_n = 0.0, 0
    done_steps = 0
    stride = 8 if args.steps >= 128 else 1
    while done_steps < args.steps:
      skip = min(stride - 1, args.steps - done_steps)
      sampler.run_steps(st, skip, sample=True)
      done_steps += skip
      if done_steps >= args.steps:
        break
      ctx_sum += start + args.warmup + done_steps
      ctx_n += 1
      cs = sampler._c_state(st)
      rc = lib.tmx_decode_steps_profiled(ctypes.byref(model.desc()), ctypes.byref(cs), _lib.stream(), 1, 1,
                                         ms.ctypes.data_as(ctypes.c_void_p), cnt.ctypes.data_as(ctypes.c_void_p))
      _lib.check(rc, 'tmx_decode_steps_profiled')
      tot_ms += ms
      tot_cnt += cnt
      done_steps += 1
    sampler.check_device_status(st)  # the profiled steps too
    result['device_status'] = 'ok: no bounded in-kernel wait ran out (timed window and profiled replay)'
    per_step = tot_ms / max(ctx_n, 1)
    result['kernel_ms_per_step'] = {n: round(float(v), 4) for n, v in zip(CLASS_NAMES, per_step)}
    layer0 = model.layers[0]
    ctx = ctx_sum / max(ctx_n, 1)
    alg = {
        'qkv_linear': linear_bytes(layer0['qkv'], batch), 'o_linear': linear_bytes(layer0['o'], batch),
        'gate_up_linear': linear_bytes(layer0['gate_up'], batch, model.expert_fraction(batch)),
        'down_linear': linear_bytes(layer0['down'], batch, model.expert_fraction(batch)),
        'attention': batch * ctx * cfg.num_kv_heads * cfg.head_dim * 2 * 2,
        'head_sample': hbytes,
    }
    if not cfg.num_experts and tot_cnt[CLASS_NAMES.index('swiglu')] == 0:
      alg['gate_up_linear'] -= batch * cfg.hidden_dim * 2  # fused SwiGLU: [M, F] goes out, not [M, 2 F]
    # multiply-add work of the dense projections (2 M K N, + the LoRA products): above the ridge of
    # 2.5 PFLOP/s / 8 TB/s = 312 flop per byte a kernel is priced against the bf16 MFMA peak instead
    def linear_flops(pl):
      f = 2.0 * batch * pl.k * pl.n
      if pl.lora_a_t is not None:
        f += 2.0 * batch * pl.rank * (pl.k * len(pl.seg_cols) + pl.n)
      return f
    flops = {}
    if not cfg.num_experts:
      flops = {'qkv_linear': linear_flops(layer0['qkv']), 'o_linear': linear_flops(layer0['o']),
               'gate_up_linear': linear_flops(layer0['gate_up']), 'down_linear': linear_flops(layer0['down'])}
    # kernel symbols (as rocprofv3 names them) and the launch classes each one serves
    mt = 1 if batch <= 32 else (2 if batch <= 64 else 4)
    # K % 256 == 0 below 8192 with fewer than 16 column blocks runs the 4-wave kernel, the rest the
    # direct-to-LDS k-way kernel (K % 256 == 0) or the plain k-way kernel.  An unsplit gate|up with
    # LoRA rank <= 16 runs the fused LoRA + SwiGLU kernel (8 waves up to 64 rows with K % 512 == 0).
    four = lambda pl: pl.k % 256 == 0 and pl.k < 8192 and (pl.n + 127) // 128 < 16
    dense = [('qkv_linear', 'qkv'), ('o_linear', 'o')]
    symbols = {}
    if cfg.num_experts:
      symbols['tmx::moe_stream_kernel<false>'] = ['gate_up_linear']
      symbols['tmx::moe_stream_kernel<true>'] = ['down_linear']
    else:
      gu = layer0['gate_up']
      fused = (tot_cnt[CLASS_NAMES.index('swiglu')] == 0 and gu.k % 256 == 0 and gu.k < 8192)
      if fused:
        lora = gu.lora_a_t is not None
        if batch <= 64 and gu.k % 512 == 0:   # 8 waves per workgroup, activation slab by direct-to-LDS loads
          # LoRA mode: 0 none, 1 every workgroup multiplies x by A itself, 2 a few workgroups do it once and
          # hand t over (K / 256 <= 32 producers that fit beside the F / 64 main workgroups within 256)
          cus = torch.cuda.get_device_properties(0).multi_processor_count
          mode = 0 if not lora else (2 if gu.k // 256 <= 32 and cfg.hidden_dim // 64 + gu.k // 256 <= cus else 1)
          sym = f'tmx::qlinear_gate_up8_kernel<{mt}, {mode}>'
        else:
          sym = f'tmx::qlinear_gate_up_kernel<{mt}>' if lora else f'tmx::qlinear_mfma4_kernel<{mt}>'
        symbols.setdefault(sym, []).append('gate_up_linear')
      else:
        dense.append(('gate_up_linear', 'gate_up'))
      dense.append(('down_linear', 'down'))
    def kway_symbol(pl):
      if pl.k % 256 == 0:
        return f'tmx::qlinear_mfma_dma_kernel<{mt}>'
      return f'tmx::qlinear_mfma_kernel<{mt}, 2>'
    if batch > 128 and not cfg.num_experts:
      # more than 128 sequences (--sequences): every projection runs the 256-row kernel, the head in
      # 256 x 256 blocks (the byte-based fractions below then understate these MFMA-bound kernels)
      symbols = {'tmx::qlinear_mfma_wide_kernel': ['qkv_linear', 'o_linear', 'gate_up_linear', 'down_linear']}
      dense = []
    for cls_name, key in dense:
      sym = f'tmx::qlinear_mfma4_kernel<{mt}>' if four(layer0[key]) else kway_symbol(layer0[key])
      symbols.setdefault(sym, []).append(cls_name)
    small = batch <= 4 and not cfg.num_experts and tot_cnt[CLASS_NAMES.index('rope_kvwrite')] == 0
    if small:
      # 1..4 rows: five launches per layer, norm / LoRA / residual / SwiGLU inside the projections
      # (template arguments: prologue 0 plain, 1 norm, 2 attention merge; epilogue 0 plain, 1 residual, 2 SwiGLU)
      symbols = {'tmx::sb_linear_kernel<1, 0>': ['qkv_linear'], 'tmx::sb_linear_kernel<2, 1>': ['o_linear'],
                 'tmx::sb_linear_kernel<1, 2>': ['gate_up_linear'], 'tmx::sb_linear_kernel<0, 1>': ['down_linear'],
                 f'tmx::sb_attn_kernel<{cfg.head_dim}, {cfg.num_heads // cfg.num_kv_heads}>': ['attention']}
    # the walk of the run without shared slots: on the matrix pipe for 4 or 8 query heads per kv head while three
    # workgroups per CU hold every (sequence, kv head) pair at once (+ gqa_combine_kernel where a row is split),
    # else on the vector ALU
    g_heads = cfg.num_heads // cfg.num_kv_heads
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    on_tile = g_heads in (4, 8) and batch * cfg.num_kv_heads <= 3 * cus
    symbols.update({} if small else {
        f"tmx::gqa_{'tile' if on_tile else 'decode'}_kernel<{cfg.head_dim}, {g_heads}>": ['attention']})
    symbols.update({
        # more than 64 rows: the head in 256 x 256 blocks (template argument: the sampling mode, 1 = top-p branch);
        # with top_p < 1 the class also holds the three selection launches of nucleus.hip
        ('tmx::head_wide_kernel<1>' if batch > 64 else f'tmx::head_kernel<{min(mt, 2)}, true>'): ['head_sample'],
    })
    idx = {n: i for i, n in enumerate(CLASS_NAMES)}
    # An event pair around a launch also times the packet processing on both sides of it, so it
    # reads a few microseconds above rocprofv3's kernel trace (which brackets the dispatch
    # alone).  The pair around a kernel that does nothing is reported beside it as the upper
    # bound of that excess; the roofline figures use the uncorrected (longer) event time.
    pair_ms = float(tot_ms[idx['empty_launch']] / max(tot_cnt[idx['empty_launch']], 1))
    per_symbol = {}
    for sym, classes in symbols.items():
      t = float(sum(tot_ms[idx[c]] for c in classes))
      n = int(sum(tot_cnt[idx[c]] for c in classes))
      if n == 0:
        continue
      launches_per_class = {c: int(tot_cnt[idx[c]]) for c in classes}
      byts = float(sum(alg[c] * launches_per_class[c] for c in classes)) / n
      avg = t / n
      per_symbol[sym] = {'classes': classes, 'total_ms_per_step': avg * n / max(ctx_n, 1), 'launches_per_step': n / max(ctx_n, 1),
                         'avg_launch_ms': avg, 'bound': 'hbm',
                         'algorithmic_bytes_per_launch': byts,
                         'achieved_GBps': byts / (avg * 1e-3) / 1e9, 'frac': byts / (avg * 1e-3) / 8e12}
      if all(c in flops for c in classes):
        fl = float(sum(flops[c] * launches_per_class[c] for c in classes)) / n
        per_symbol[sym].update({'flops_per_launch': fl, 'achieved_TFLOPs': fl / (avg * 1e-3) / 1e12,
                                'frac_of_2500_TFLOPs': fl / (avg * 1e-3) / 2.5e15})
        if fl / byts > 2.5e15 / 8e12:
          per_symbol[sym]['bound'] = 'mfma'
    dom = max(per_symbol, key=lambda k: per_symbol[k]['total_ms_per_step'])
    traffic = None
    tpath = os.path.join(ROOT, 'profiles', 'traffic.json')
    if os.path.exists(tpath):  # HBM bytes per launch from the rocprofv3 --pmc runs (see profiles/)
      traffic = json.load(open(tpath)).get(args.workload, {}).get(dom)
    d = per_symbol[dom]
    mf = d['bound'] == 'mfma'
    result['roofline'] = {'bound': d['bound'], 'achieved': d['achieved_TFLOPs'] if mf else d['achieved_GBps'],
                          'peak': 2500.0 if mf else 8000.0, 'unit': 'TFLOP/s' if mf else 'GB/s',
                          'frac': d['frac_of_2500_TFLOPs'] if mf else d['frac'], 'traffic': traffic, 'kernel': dom,
                          'avg_launch_ms': d['avg_launch_ms'],
                          'empty_launch_event_pair_ms': pair_ms,
                          'algorithmic_bytes_per_launch': d['algorithmic_bytes_per_launch'],
                          'note': 'mean HIP-event time around the launches of this kernel in the sampled '
                                  'steps (includes event packet processing, see empty_launch_event_pair_ms); '
                                  'classes per kernel symbol are listed in roofline_kernels'}
    result['roofline_kernels'] = per_symbol
    result['roofline_all'] = {}
    for i, n in enumerate(CLASS_NAMES):
      if n in alg and tot_cnt[i] > 0:
        avg = float(tot_ms[i] / tot_cnt[i])
        result['roofline_all'][n] = {'avg_launch_ms': avg, 'achieved_GBps': alg[n] / (avg * 1e-3) / 1e9,
                                     'frac': alg[n] / (avg * 1e-3) / 8e12}

  if not args.no_profile and not cfg.num_experts and sampler._fill_rows() > 128:
    # Cache fill (outside the headline metric): the prompt walk above, and the projection kernel that
    # carries it (256-row blocks, MFMA-bound) timed alone on the gate|up shape at the rows of one pass.
    lib = _lib.lib()
    rows = min(sampler._fill_rows() // batch, 128, start - 1) * batch
    pl = model.layers[0]['gate_up']
    xs = torch.randn(rows, pl.k, device='cuda').to(torch.bfloat16)
    ns = lib.tmx_qlora_linear_num_splits(rows, pl.k, pl.n)
    yp = torch.empty(ns, rows, pl.n, dtype=torch.float32, device='cuda')
    tp = torch.empty(32, rows, 128, dtype=torch.float32, device='cuda')
    a_t = pl.lora_a_t.data_ptr() if pl.lora_a_t is not None else None
    def gemm():
      _lib.check(lib.tmx_qlora_linear_planes(_lib.stream(), xs.data_ptr(), pl.qweight.data_ptr(), pl.scales.data_ptr(),
                                             a_t, yp.data_ptr(), tp.data_ptr(), rows, pl.k, pl.n, group,
                                             pl.r_pad if a_t else 0, ns), 'tmx_qlora_linear_planes')
    for _ in range(2):
      gemm()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(8):
      gemm()
    e1.record()
    torch.cuda.synchronize()
    g_ms = e0.elapsed_time(e1) / 8
    flops = 2.0 * rows * pl.k * pl.n
    result['prefill'] = {
        'prompt_tokens_per_s': batch * (start - 1) / (walk_ms[0] * 1e-3), 'walk_ms': walk_ms[0],
        'walked_tokens_per_sequence': start - 1,
        'rows_per_pass': rows,
        'roofline': {'bound': 'mfma', 'kernel': 'tmx::qlinear_mfma_wide_kernel',
                     'shape': f'{rows} x {pl.k} x {pl.n} (gate|up)', 'avg_launch_ms': g_ms,
                     'achieved': flops / (g_ms * 1e-3) / 1e12, 'peak': 2500.0, 'unit': 'TFLOP/s',
                     'frac': flops / (g_ms * 1e-3) / 2.5e15},
    }
    del xs, yp, tp

  if shared and not args.no_profile:
    # the attention launch of the default path, timed the same way over a few steps
    sampler.share_prompt_kv = True
    lib = _lib.lib()
    st = fresh_state()
    n_prof = min(8, args.steps)
    # at the middle of the timed window: the mean context, where the unshared replay's mean sits too
    sampler.run_steps(st, args.warmup + (args.steps - n_prof) // 2, sample=True)
    ms = np.zeros(len(CLASS_NAMES), np.float32)
    cnt = np.zeros(len(CLASS_NAMES), np.int32)
    tot = 0.0
    for _ in range(n_prof):
      cs = sampler._c_state(st)
      rc = lib.tmx_decode_steps_profiled(ctypes.byref(model.desc()), ctypes.byref(cs), _lib.stream(), 1, 1,
                                         ms.ctypes.data_as(ctypes.c_void_p), cnt.ctypes.data_as(ctypes.c_void_p))
      _lib.check(rc, 'tmx_decode_steps_profiled')
      tot += float(ms[CLASS_NAMES.index('attention')])
    sampler.check_device_status(st)
    result['prompt_kv_sharing']['attention_ms_per_step'] = tot / n_prof
    result['prompt_kv_sharing']['attention_ms_per_step_without'] = result['kernel_ms_per_step']['attention']
  if args.steps + args.warmup >= new and not args.sync_steps:
    # The whole rollout through the call a user makes (Sampler.__call__): padding, cache fill over the prompt,
    # every decode step, the device status check, device-to-host copies and per-row slicing.  Beside `value`,
    # which times decode steps alone.
    sampler.share_prompt_kv = not args.no_kv_sharing
    prompts = [row for row in ids]
    best = None
    for rep in range(2):
      torch.cuda.synchronize()
      t0 = time.perf_counter()
      out = sampler(prompt_token_ids=prompts, max_generation_steps=new, return_logprobs=True, eos_tokens=[-1],
                    temperature=temp, top_p=top_p, seed=rep)
      torch.cuda.synchronize()
      sec = time.perf_counter() - t0
      n_tok = int(sum(len(t) for t in out.tokens))
      assert n_tok == batch * new
      best = sec if best is None else min(best, sec)
    result['sampler_call'] = {'tokens_per_s': n_tok / best, 'seconds': best, 'generated_tokens': n_tok,
                              'includes': 'prompt padding, cache fill, decode steps, status check, copies to the host'}
  if not args.no_cpu_baseline and not cfg.num_experts:
    st = None
    result['cpu_baseline'] = cpu_baseline(args.workload)
  print(json.dumps(result))


if __name__ == '__main__':
  main()
