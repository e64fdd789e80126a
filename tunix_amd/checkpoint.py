"""Local checkpoints -> QLoRAModel, and a packed on-disk format of the quantised model.

Two loaders (both read local paths only, through `safetensors`, which executes nothing):

* ``load_hf_safetensors(dir, config)``: Hugging Face Llama / Qwen3 / Qwen3-MoE weights
  (``*.safetensors`` under `dir`) renamed and reshaped to the reference's parameter paths with
  the rules of tunix/models/llama3/params.py:23-80 and tunix/models/qwen3/params.py:25-121
  (torch ``[out, in]`` -> transpose -> reshape ``[D, N, H]`` / ``[N, H, D]``; MoE experts stacked
  to ``[E, D, F]`` / ``[E, F, D]``), ready for ``QLoRAModel.from_state`` (which quantises).
* ``save_packed(model, path)`` / ``load_packed(path, device)``: the device layout itself (q4t
  nibble tiles, bf16 scales, LoRA tensors, norms, embedding / head) in one safetensors file
  with the configuration in its metadata, so a served model is not re-quantised at start-up.

File format of ``save_packed`` (version 1): tensors ``embed``, ``head`` (absent when tied),
``final_norm``, and per layer i ``layers.i.{norm1,norm2,q_norm,k_norm,router}`` and per
projection p in {qkv, o, gate_up, down} ``layers.i.p.{qweight,scales,lora_a_t,lora_b}``;
metadata: ``format`` = "tunix_amd.q4t.v1", ``config`` (JSON of ModelConfig), ``group``,
``lora_rank``, ``lora_alpha`` and per projection ``layers.i.p.meta`` = JSON
{k, n, seg_cols, rank, lora_scale, experts}.
"""
import dataclasses
import glob
import json
import os
import re

import torch

from tunix_amd import quant
from tunix_amd.model import ModelConfig, QLoRAModel

FORMAT = 'tunix_amd.q4t.v1'


def hf_key_rules(cfg):
  """(regex on the torch key, tunix path template, transpose?, reshape or None)."""
  d, n, kh, h = cfg.embed_dim, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim
  L = r'model\.layers\.([0-9]+)\.'
  return [
      (r'model\.embed_tokens\.weight', 'embedder.input_embedding', False, None),
      (L + r'self_attn\.q_proj\.weight', r'layers.\1.attn.q_proj.w', True, (d, n, h)),
      (L + r'self_attn\.k_proj\.weight', r'layers.\1.attn.k_proj.w', True, (d, kh, h)),
      (L + r'self_attn\.v_proj\.weight', r'layers.\1.attn.v_proj.w', True, (d, kh, h)),
      (L + r'self_attn\.o_proj\.weight', r'layers.\1.attn.o_proj.w', True, (n, h, d)),
      (L + r'mlp\.(gate|up|down)_proj\.weight', r'layers.\1.mlp.\2_proj.kernel', True, None),
      (L + r'mlp\.gate\.weight', r'layers.\1.mlp.router.kernel', True, None),
      (L + r'mlp\.experts\.([0-9]+)\.(gate|up|down)_proj\.weight', r'layers.\1.mlp.experts.\2.\3_proj.kernel', True, None),
      (r'model\.norm\.weight', 'final_norm.w', False, None),
      (L + r'self_attn\.(q|k)_norm\.weight', r'layers.\1.attn.\2_norm.w', False, None),
      (L + r'(input|post_attention)_layernorm\.weight', r'layers.\1.\2_layernorm.w', False, None),
      (r'lm_head\.weight', 'lm_head.w', True, None),
  ]


def rename_hf_state(cfg, tensors):
  """dict torch key -> tensor  =>  dict tunix path -> tensor (float32 on CPU)."""
  rules = [(re.compile(pat + '$'), tmpl, tr, shape) for pat, tmpl, tr, shape in hf_key_rules(cfg)]
  out = {}
  for key, t in tensors.items():
    for pat, tmpl, tr, shape in rules:
      m = pat.match(key)
      if not m:
        continue
      t = t.to(torch.float32)
      if tr:
        t = t.t()
      if shape is not None:
        t = t.reshape(shape)
      out[m.expand(tmpl)] = t.contiguous()
      break
    else:
      if 'rotary_emb' in key or key.endswith('.bias'):
        continue  # buffers the reference's mapping also drops
      raise KeyError(f'no rule for checkpoint key {key!r}')
  if cfg.num_experts:
    # stack the per-expert matrices (qwen3/params.py:25-44)
    for i in range(cfg.num_layers):
      for kw in ('gate', 'up', 'down'):
        keys = [f'layers.{i}.mlp.experts.{e}.{kw}_proj.kernel' for e in range(cfg.num_experts)]
        out[f'layers.{i}.mlp.{kw}_proj'] = torch.stack([out.pop(k) for k in keys], 0)
  if cfg.weight_tying:
    out.pop('lm_head.w', None)
  elif 'lm_head.w' not in out:
    raise KeyError('checkpoint has no lm_head.weight but the configuration is not tied')
  return out


def load_hf_safetensors(file_dir, cfg):
  """Reads every *.safetensors under file_dir (a local directory) and renames the tensors."""
  from safetensors import safe_open
  files = sorted(glob.glob(os.path.join(file_dir, '*.safetensors')))
  if not files:
    raise FileNotFoundError(f'no *.safetensors under {file_dir}')
  tensors = {}
  for f in files:
    with safe_open(f, framework='pt', device='cpu') as sf:
      for k in sf.keys():
        tensors[k] = sf.get_tensor(k)
  return rename_hf_state(cfg, tensors)


def model_from_hf(file_dir, cfg, group=64, device='cuda', lora_state=None, lora_alpha=0.0, bound=7.5):
  """HF checkpoint -> int4 QLoRA model on the device (optionally with LoRA tensors under the
  reference's `<weight>_lora_a/_lora_b` names)."""
  state = load_hf_safetensors(file_dir, cfg)
  if lora_state:
    state.update(lora_state)
  return QLoRAModel.from_state(cfg, state, group=group, lora_alpha=lora_alpha, device=device, bound=bound)


_PROJ = ('qkv', 'o', 'gate_up', 'down')


def save_packed(model, path):
  from safetensors.torch import save_file
  tensors = {'embed': model.embed, 'final_norm': model.final_norm}
  if model.head is not model.embed:
    tensors['head'] = model.head
  meta = {'format': FORMAT, 'config': json.dumps(dataclasses.asdict(model.config)), 'group': str(model.group),
          'lora_rank': str(model.lora_rank), 'lora_alpha': repr(float(model.lora_alpha))}
  for i, layer in enumerate(model.layers):
    for k in ('norm1', 'norm2', 'q_norm', 'k_norm', 'router'):
      if k in layer:
        tensors[f'layers.{i}.{k}'] = layer[k]
    for p in _PROJ:
      pl = layer[p]
      tensors[f'layers.{i}.{p}.qweight'] = pl.qweight
      tensors[f'layers.{i}.{p}.scales'] = pl.scales
      if pl.lora_a_t is not None:
        tensors[f'layers.{i}.{p}.lora_a_t'] = pl.lora_a_t
        tensors[f'layers.{i}.{p}.lora_b'] = pl.lora_b
      meta[f'layers.{i}.{p}.meta'] = json.dumps({'k': pl.k, 'n': pl.n, 'seg_cols': pl.seg_cols, 'rank': pl.rank,
                                                 'lora_scale': pl.lora_scale, 'experts': pl.experts})
  save_file({k: v.detach().contiguous().cpu() for k, v in tensors.items()}, path, metadata=meta)


def load_packed(path, device='cuda'):
  from safetensors import safe_open
  with safe_open(path, framework='pt', device='cpu') as sf:
    meta = sf.metadata() or {}
    if meta.get('format') != FORMAT:
      raise ValueError(f'{path}: not a {FORMAT} file')
    cfg = ModelConfig(**json.loads(meta['config']))
    m = QLoRAModel(cfg, device)
    m.group, m.lora_rank, m.lora_alpha = int(meta['group']), int(meta['lora_rank']), float(meta['lora_alpha'])
    get = lambda k: sf.get_tensor(k).to(m.device)
    keys = set(sf.keys())
    m.embed, m.final_norm = get('embed'), get('final_norm')
    m.head = get('head') if 'head' in keys else m.embed
    for i in range(cfg.num_layers):
      layer = {}
      for k in ('norm1', 'norm2', 'q_norm', 'k_norm', 'router'):
        if f'layers.{i}.{k}' in keys:
          layer[k] = get(f'layers.{i}.{k}')
      for p in _PROJ:
        pm = json.loads(meta[f'layers.{i}.{p}.meta'])
        has_lora = f'layers.{i}.{p}.lora_a_t' in keys
        pl = quant.PackedLinear(pm['k'], pm['n'], m.group, get(f'layers.{i}.{p}.qweight'),
                                get(f'layers.{i}.{p}.scales'), pm['seg_cols'], pm['rank'],
                                get(f'layers.{i}.{p}.lora_a_t') if has_lora else None,
                                get(f'layers.{i}.{p}.lora_b') if has_lora else None, pm['lora_scale'])
        pl.experts = pm['experts']
        layer[p] = pl
      m.layers.append(layer)
  return m
