"""Device-resident int4 QLoRA decoder weights in the layout the HIP kernels read.

Stands where the reference has a qwix-wrapped ``Llama3`` / ``Qwen3`` nnx module
(tunix/models/llama3/model.py:590, tunix/models/qwen3/model.py:1318 after
tunix/cli/utils/model.py:31-77): same configuration fields, same parameter
names in the state dict it is built from, same LoRA-only update contract.
"""
import ctypes
import dataclasses
from typing import Optional

import torch

from tunix_amd import quant
from tunix_amd import _lib

FAMILY_LLAMA3, FAMILY_QWEN3 = 0, 1
SAMPLE_GREEDY, SAMPLE_TOP_P, SAMPLE_SCORE = 0, 1, 2
MAX_RPAD = 128


@dataclasses.dataclass
class ModelConfig:
  """Field names follow the reference's ModelConfig dataclasses
  (llama3/model.py:85-101, qwen3/model.py:163-186)."""
  family: str
  num_layers: int
  vocab_size: int
  embed_dim: int
  hidden_dim: int
  num_heads: int
  head_dim: int
  num_kv_heads: int
  rope_theta: float = 500_000
  norm_eps: float = 1e-5
  weight_tying: bool = False
  num_experts: Optional[int] = None
  num_experts_per_tok: Optional[int] = None

  @classmethod
  def from_reference(cls, cfg, family=None):
    """From one of the reference's own ModelConfig objects (llama3/model.py:85-101,
    qwen3/model.py:160-185), read by attribute name; `family` is taken from the defining module or
    from the Qwen3-only fields when not given."""
    if family is None:
      mod = type(cfg).__module__ or ''
      family = 'qwen3' if ('qwen3' in mod or hasattr(cfg, 'use_tied_embedding')) else 'llama3'
    if family not in ('llama3', 'qwen3'):
      raise ValueError(f'unknown model family {family!r}')
    tied = bool(getattr(cfg, 'weight_tying', False) or getattr(cfg, 'use_tied_embedding', False))
    return cls(family, int(cfg.num_layers), int(cfg.vocab_size), int(cfg.embed_dim), int(cfg.hidden_dim),
               int(cfg.num_heads), int(cfg.head_dim), int(cfg.num_kv_heads), float(cfg.rope_theta),
               float(cfg.norm_eps), tied, getattr(cfg, 'num_experts', None), getattr(cfg, 'num_experts_per_tok', None))

  @classmethod
  def llama3p2_1b(cls):
    return cls('llama3', 16, 128256, 2048, 8192, 32, 64, 8, 500_000, 1e-5, True)

  @classmethod
  def llama3p1_8b(cls):
    return cls('llama3', 32, 128256, 4096, 14336, 32, 128, 8, 500_000, 1e-5, False)

  @classmethod
  def qwen3_8b(cls):
    return cls('qwen3', 36, 151936, 4096, 12288, 32, 128, 8, 1_000_000, 1e-6, False)

  @classmethod
  def qwen3_30b_a3b(cls):
    return cls('qwen3', 48, 151936, 2048, 768, 32, 128, 4, 1_000_000, 1e-6, False, 128, 8)

  @classmethod
  def toy(cls):
    """The 2-layer CPU-runnable configuration of the benchmark description."""
    return cls('llama3', 2, 1024, 256, 1024, 4, 64, 4, 10_000, 1e-5, False)


class QLinearDesc(ctypes.Structure):
  _fields_ = [('qweight', ctypes.c_void_p), ('scales', ctypes.c_void_p), ('lora_a_t', ctypes.c_void_p),
              ('lora_b', ctypes.c_void_p), ('K', ctypes.c_int), ('N', ctypes.c_int), ('G', ctypes.c_int),
              ('rank', ctypes.c_int), ('r_pad', ctypes.c_int), ('lora_scale', ctypes.c_float)]


class LayerDesc(ctypes.Structure):
  _fields_ = [('norm1_w', ctypes.c_void_p), ('norm2_w', ctypes.c_void_p), ('q_norm_w', ctypes.c_void_p),
              ('k_norm_w', ctypes.c_void_p), ('qkv', QLinearDesc), ('o', QLinearDesc),
              ('gate_up', QLinearDesc), ('down', QLinearDesc), ('router_w', ctypes.c_void_p)]


class ModelDesc(ctypes.Structure):
  _fields_ = [('family', ctypes.c_int), ('num_layers', ctypes.c_int), ('vocab_size', ctypes.c_int),
              ('embed_dim', ctypes.c_int), ('hidden_dim', ctypes.c_int), ('num_heads', ctypes.c_int),
              ('num_kv_heads', ctypes.c_int), ('head_dim', ctypes.c_int), ('num_experts', ctypes.c_int),
              ('experts_per_tok', ctypes.c_int), ('rope_theta', ctypes.c_float),
              ('norm_eps', ctypes.c_float), ('embed', ctypes.c_void_p), ('final_norm_w', ctypes.c_void_p),
              ('head', ctypes.c_void_p), ('layers', ctypes.POINTER(LayerDesc)), ('head_tiles', ctypes.c_void_p)]


class DecodeState(ctypes.Structure):
  _fields_ = [('batch', ctypes.c_int), ('buf_len', ctypes.c_int), ('cache_size', ctypes.c_int),
              ('token_buffer', ctypes.c_void_p), ('positions', ctypes.c_void_p),
              ('input_mask', ctypes.c_void_p), ('logprobs', ctypes.c_void_p), ('done', ctypes.c_void_p),
              ('step', ctypes.c_void_p), ('kv_cache', ctypes.c_void_p), ('sampling_mode', ctypes.c_int),
              ('temperature', ctypes.c_float), ('top_p', ctypes.c_float), ('top_k', ctypes.c_int),
              ('seed_hi', ctypes.c_uint32), ('seed_lo', ctypes.c_uint32), ('eos_ids', ctypes.c_void_p),
              ('n_eos', ctypes.c_int), ('forbidden', ctypes.c_void_p), ('n_forbidden', ctypes.c_int),
              ('logits_out', ctypes.c_void_p), ('workspace', ctypes.c_void_p),
              ('workspace_bytes', ctypes.c_size_t), ('nucleus_workspace', ctypes.c_void_p),
              ('nucleus_workspace_bytes', ctypes.c_size_t), ('tokens_per_pass', ctypes.c_int),
              ('share_group', ctypes.c_int), ('share_len', ctypes.c_int)]


def _qdesc(pl):
  d = QLinearDesc()
  d.qweight, d.scales = pl.qweight.data_ptr(), pl.scales.data_ptr()
  d.lora_a_t = pl.lora_a_t.data_ptr() if pl.lora_a_t is not None else None
  d.lora_b = pl.lora_b.data_ptr() if pl.lora_b is not None else None
  d.K, d.N, d.G, d.rank, d.r_pad, d.lora_scale = pl.k, pl.n // pl.experts, pl.group, pl.rank, pl.r_pad, pl.lora_scale
  return d


_ATTN = ('q_proj', 'k_proj', 'v_proj', 'o_proj')
_MLP = ('gate_proj', 'up_proj', 'down_proj')


class QLoRAModel:
  """int4 group-quantised base weights + bf16 LoRA adapters on one GPU.

  Build with ``from_state`` (a flat dict of dense float tensors under the
  reference's parameter paths) or ``random_init``.
  """

  def __init__(self, config, device='cuda'):
    self.config = config
    self.device = torch.device(device)
    self.layers = []          # list of dict name -> tensor / PackedLinear
    self.embed = None         # bf16 [V, D]
    self.head = None          # bf16 [V, D] (is self.embed when tied)
    self.head_tiles = None    # the head once more in the streaming layout (tmx_head_tiles_pack), made by desc()
    self.stream_head = True   # False: decode steps read the row-major head
    self.final_norm = None
    self.lora_rank = 0
    self.lora_alpha = 0.0
    self.group = 0
    self._desc = None
    self._keep = None

  # -- construction --------------------------------------------------------
  @staticmethod
  def _flat2d(name, w, cfg):
    """Flattens the reference's 3-D Einsum weights to [K_in, N_out] (contraction
    axes first; o_proj 'NHD' contracts over N and H)."""
    if w.dim() == 3:
      if name == 'o_proj':
        return w.reshape(w.shape[0] * w.shape[1], w.shape[2])
      return w.reshape(w.shape[0], w.shape[1] * w.shape[2])
    return w

  @classmethod
  def from_state(cls, config, state, group=64, lora_alpha=0.0, device='cuda', bound=7.5):
    """state: dict path -> tensor with the reference's names, e.g.
    'layers.0.attn.q_proj.w' [D, N, H], '...q_proj.w_lora_a' [D, r], '...w_lora_b' [r, N, H],
    'layers.0.mlp.gate_proj.kernel' [D, F], '...kernel_lora_a', '...kernel_lora_b',
    'layers.0.input_layernorm.w', 'embedder.input_embedding' [V, D], 'final_norm.w',
    'lm_head.w' [D, V] (untied)."""
    m = cls(config, device)
    m.group, m.lora_alpha = group, float(lora_alpha)
    dev = m.device
    bf = lambda t: torch.as_tensor(t).to(dev).to(torch.bfloat16).contiguous()
    m.embed = bf(state['embedder.input_embedding'])
    m.final_norm = bf(state['final_norm.w'])
    m.head = m.embed if config.weight_tying else bf(torch.as_tensor(state['lm_head.w']).to(dev).t())

    def proj(prefix, names, wkey):
      ws, loras = [], []
      for n in names:
        w = cls._flat2d(n, torch.as_tensor(state[f'{prefix}.{n}.{wkey}']), config)
        ws.append(w)
        ka, kb = f'{prefix}.{n}.{wkey}_lora_a', f'{prefix}.{n}.{wkey}_lora_b'
        if ka in state:
          a, b = torch.as_tensor(state[ka]), torch.as_tensor(state[kb])
          a = a.reshape(-1, a.shape[-1])          # [K, r]  (o_proj: [N, H, r])
          b = b.reshape(b.shape[0], -1)            # [r, N_out]
          loras.append((a, b))
          m.lora_rank = a.shape[1]
        else:
          loras.append(None)
      ls = (m.lora_alpha / m.lora_rank) if m.lora_rank else 0.0
      return quant.PackedLinear.from_dense(ws, group, dev, loras, ls, bound)

    for i in range(config.num_layers):
      p = f'layers.{i}'
      layer = {
          'norm1': bf(state[f'{p}.input_layernorm.w']),
          'norm2': bf(state[f'{p}.post_attention_layernorm.w']),
          'qkv': proj(f'{p}.attn', ('q_proj', 'k_proj', 'v_proj'), 'w'),
          'o': proj(f'{p}.attn', ('o_proj',), 'w'),
      }
      if config.num_experts:
        # MoELayer params (tunix/models/qwen3/model.py:863-891): router.kernel [D, E],
        # gate_proj / up_proj [E, D, F], down_proj [E, F, D]; no LoRA on experts
        e = config.num_experts
        g_, u_ = (torch.as_tensor(state[f'{p}.mlp.{n}']).to(dev) for n in ('gate_proj', 'up_proj'))
        gu = torch.stack([g_, u_], dim=2).permute(1, 0, 2, 3).reshape(g_.shape[1], -1)  # [D, E * (F | F)]
        dn = torch.as_tensor(state[f'{p}.mlp.down_proj']).to(dev).permute(1, 0, 2).reshape(g_.shape[2], -1)
        layer['gate_up'] = quant.PackedLinear.from_dense([gu], group, dev, None, 0.0, bound)
        layer['down'] = quant.PackedLinear.from_dense([dn], group, dev, None, 0.0, bound)
        layer['gate_up'].experts = layer['down'].experts = e
        layer['router'] = bf(state[f'{p}.mlp.router.kernel'])
      else:
        layer['gate_up'] = proj(f'{p}.mlp', ('gate_proj', 'up_proj'), 'kernel')
        layer['down'] = proj(f'{p}.mlp', ('down_proj',), 'kernel')
      if config.family == 'qwen3':
        layer['q_norm'] = bf(state[f'{p}.attn.q_norm.w'])
        layer['k_norm'] = bf(state[f'{p}.attn.k_norm.w'])
      m.layers.append(layer)
    return m

  @classmethod
  def from_state_tree(cls, config, tree, group=64, lora_alpha=0.0, device='cuda', bound=7.5):
    """The same from what a tunix caller holds: nnx.state(model) of a (LoRA-wrapped, not yet
    quantised) Llama3 / Qwen3 module, its pure-dict dump, or any nested mapping with the
    reference's path parts ('layers', 0, 'attn', 'q_proj', 'w', ...).  Leaves may be arrays or
    variable objects with the array in `.value`; the tree is flattened to dotted paths
    (tunix/rl/utils.py:72-78 to_flat_dict) and quantised like from_state."""
    from tunix_amd import utils
    return cls.from_state(config, utils.flatten_state(tree), group=group, lora_alpha=lora_alpha, device=device,
                          bound=bound)

  @classmethod
  def random_init(cls, config, seed=0, group=64, lora_rank=0, lora_alpha=0.0,
                  lora_targets=_ATTN + _MLP, std=0.02, device='cuda'):
    """Synthetic weights generated layer by layer on the device: every matrix
    std * N(0, 1) in bf16 (the reference's dummy-model recipe,
    tunix/models/dummy_model_creator.py:29-92), norm weights 1."""
    c = config
    g = torch.Generator(device=device).manual_seed(seed)
    rnd = lambda *s: (torch.randn(*s, generator=g, device=device, dtype=torch.float32) * std).to(torch.bfloat16)
    m = cls(config, device)
    m.group, m.lora_alpha, m.lora_rank = group, float(lora_alpha), lora_rank
    m.embed = rnd(c.vocab_size, c.embed_dim)
    m.final_norm = torch.ones(c.embed_dim, dtype=torch.bfloat16, device=device)
    m.head = m.embed if c.weight_tying else rnd(c.vocab_size, c.embed_dim)
    ls = lora_alpha / lora_rank if lora_rank else 0.0
    d, f, nh, kh = c.embed_dim, c.hidden_dim, c.num_heads * c.head_dim, c.num_kv_heads * c.head_dim

    def proj(k, outs, names):
      ws = [rnd(k, n) for n in outs]
      loras = [(rnd(k, lora_rank), rnd(lora_rank, n)) if (lora_rank and nm in lora_targets) else None
               for n, nm in zip(outs, names)]
      return quant.PackedLinear.from_dense(ws, group, device, loras, ls)

    for _ in range(c.num_layers):
      layer = {
          'norm1': torch.ones(d, dtype=torch.bfloat16, device=device),
          'norm2': torch.ones(d, dtype=torch.bfloat16, device=device),
          'qkv': proj(d, (nh, kh, kh), ('q_proj', 'k_proj', 'v_proj')),
          'o': proj(nh, (d,), ('o_proj',)),
      }
      if c.num_experts:
        e = c.num_experts
        layer['gate_up'] = quant.PackedLinear.from_dense([rnd(d, e * 2 * f)], group, device)
        layer['down'] = quant.PackedLinear.from_dense([rnd(f, e * d)], group, device)
        layer['gate_up'].experts = layer['down'].experts = e
        layer['router'] = rnd(d, e)
      else:
        layer['gate_up'] = proj(d, (f, f), ('gate_proj', 'up_proj'))
        layer['down'] = proj(f, (d,), ('down_proj',))
      if c.family == 'qwen3':
        layer['q_norm'] = torch.ones(c.head_dim, dtype=torch.bfloat16, device=device)
        layer['k_norm'] = torch.ones(c.head_dim, dtype=torch.bfloat16, device=device)
      m.layers.append(layer)
    return m

  # -- reference-shaped surface --------------------------------------------
  @property
  def num_embed(self):
    return self.config.vocab_size

  @property
  def dtype(self):
    return torch.bfloat16

  def init_cache(self, batch_size, cache_size, dtype=torch.bfloat16):
    """One allocation [layers][k|v][B][C][Kh][H]; layer i's 'k' is cache[i, 0].
    (tunix/generate/sampler.py:171-202, qwen3/model.py:1359-1373.)"""
    c = self.config
    return torch.zeros(c.num_layers, 2, batch_size, cache_size, c.num_kv_heads, c.head_dim,
                       dtype=dtype, device=self.device)

  def lora_state(self):
    """Flat dict of the LoRA tensors (the nnx.LoRAParam leaves of the reference)."""
    out = {}
    for i, layer in enumerate(self.layers):
      for key, names, pre, wk in (('qkv', ('q_proj', 'k_proj', 'v_proj'), 'attn', 'w'),
                                  ('o', ('o_proj',), 'attn', 'w'),
                                  ('gate_up', ('gate_proj', 'up_proj'), 'mlp', 'kernel'),
                                  ('down', ('down_proj',), 'mlp', 'kernel')):
        pl = layer[key]
        if pl.lora_a_t is None:
          continue
        col = 0
        for j, (n, width) in enumerate(zip(names, pl.seg_cols)):
          a = pl.lora_a_dense()[:, j * pl.rank:(j + 1) * pl.rank].contiguous()
          b = pl.lora_b[:, col:col + width].contiguous()
          out[f'layers.{i}.{pre}.{n}.{wk}_lora_a'] = a
          out[f'layers.{i}.{pre}.{n}.{wk}_lora_b'] = b
          col += width
    return out

  @staticmethod
  def check_lora_state(cur, state):
    """The reference's checks on a replacement state (tunix/generate/sampler.py:281-332): same
    paths, same shapes (3-D Einsum shapes are accepted for their flattened 2-D counterparts)."""
    if set(state.keys()) != set(cur.keys()):
      raise ValueError('New state must have the same structure as the old state.'
                       f' {sorted(cur.keys())[:3]}... vs {sorted(state.keys())[:3]}...')
    for k, v in state.items():
      v = torch.as_tensor(v)
      ok = v.numel() == cur[k].numel() and v.dim() >= 2 and (
          v.reshape(cur[k].shape[0], -1).shape == cur[k].shape or v.reshape(-1, cur[k].shape[-1]).shape == cur[k].shape)
      # a flattened axis must be one the Einsum layout really has: first or last dimension kept
      ok = ok and (v.shape[0] == cur[k].shape[0] or v.shape[-1] == cur[k].shape[-1])
      if not ok:
        raise ValueError('New state must have the same shape, dtype and sharding as the old state.'
                         f' {k}: {tuple(v.shape)} vs {tuple(cur[k].shape)}')

  def update_lora(self, state):
    """LoRA-only replacement (tunix/generate/sampler.py:340-354): `state` must have
    exactly the keys and shapes of lora_state(); base int4 weights are untouched."""
    self.check_lora_state(self.lora_state(), state)
    for i, layer in enumerate(self.layers):
      for key, names, pre, wk in (('qkv', ('q_proj', 'k_proj', 'v_proj'), 'attn', 'w'),
                                  ('o', ('o_proj',), 'attn', 'w'),
                                  ('gate_up', ('gate_proj', 'up_proj'), 'mlp', 'kernel'),
                                  ('down', ('down_proj',), 'mlp', 'kernel')):
        pl = layer[key]
        if pl.lora_a_t is None:
          continue
        loras = []
        for n in names:
          a = torch.as_tensor(state[f'layers.{i}.{pre}.{n}.{wk}_lora_a'])
          b = torch.as_tensor(state[f'layers.{i}.{pre}.{n}.{wk}_lora_b'])
          loras.append((a.reshape(-1, a.shape[-1]), b.reshape(b.shape[0], -1)))
        pl.set_lora(loras)

  # -- C ABI descriptor -------------------------------------------------------
  def desc(self):
    """ctypes tmx_model_desc (cached; device pointers stay valid because LoRA
    updates are in place)."""
    if self._desc is not None:
      return self._desc
    c = self.config
    arr = (LayerDesc * c.num_layers)()
    for i, layer in enumerate(self.layers):
      arr[i].norm1_w = layer['norm1'].data_ptr()
      arr[i].norm2_w = layer['norm2'].data_ptr()
      arr[i].q_norm_w = layer['q_norm'].data_ptr() if 'q_norm' in layer else None
      arr[i].k_norm_w = layer['k_norm'].data_ptr() if 'k_norm' in layer else None
      arr[i].qkv, arr[i].o = _qdesc(layer['qkv']), _qdesc(layer['o'])
      arr[i].gate_up, arr[i].down = _qdesc(layer['gate_up']), _qdesc(layer['down'])
      arr[i].router_w = layer['router'].data_ptr() if 'router' in layer else None
    d = ModelDesc()
    d.family = FAMILY_LLAMA3 if c.family == 'llama3' else FAMILY_QWEN3
    d.num_layers, d.vocab_size, d.embed_dim, d.hidden_dim = c.num_layers, c.vocab_size, c.embed_dim, c.hidden_dim
    d.num_heads, d.num_kv_heads, d.head_dim = c.num_heads, c.num_kv_heads, c.head_dim
    d.num_experts, d.experts_per_tok = c.num_experts or 0, c.num_experts_per_tok or 0
    d.rope_theta, d.norm_eps = float(c.rope_theta), float(c.norm_eps)
    d.embed, d.final_norm_w, d.head = self.embed.data_ptr(), self.final_norm.data_ptr(), self.head.data_ptr()
    if self.stream_head and c.vocab_size % 32 == 0 and c.embed_dim % 64 == 0 and c.vocab_size <= 32 * 65535:
      # one more copy of the head (V * D * 2 bytes) that one-token steps of up to 64 sequences stream
      if self.head_tiles is None:
        self.head_tiles = torch.empty_like(self.head)
        _lib.check(_lib.lib().tmx_head_tiles_pack(_lib.stream(), _lib.ptr(self.head), _lib.ptr(self.head_tiles),
                                                  c.vocab_size, c.embed_dim), 'tmx_head_tiles_pack')
      d.head_tiles = self.head_tiles.data_ptr()
    d.layers = ctypes.cast(arr, ctypes.POINTER(LayerDesc))
    self._desc, self._keep = d, arr
    return d

  def expert_fraction(self, batch):
    """Expected fraction of a layer's experts that a step of `batch` tokens touches under
    uniform routing: 1 - (1 - k / E) ** batch (1 for dense models)."""
    c = self.config
    if not c.num_experts:
      return 1.0
    return 1.0 - (1.0 - c.num_experts_per_tok / c.num_experts) ** batch

  def weight_bytes(self, batch=1):
    """Algorithmic bytes one decode step streams from the weights:
    int4 + scales + LoRA A, B per projection, plus the bf16 head.  Routed-expert
    matrices count by the expected fraction of experts touched (data dependent)."""
    total = 0
    for layer in self.layers:
      if 'router' in layer:
        total += layer['router'].numel() * 2
      for key in ('qkv', 'o', 'gate_up', 'down'):
        pl = layer[key]
        frac = self.expert_fraction(batch) if pl.experts > 1 else 1.0
        total += int((pl.k * pl.n // 2 + (pl.k // pl.group) * pl.n * 2) * frac)
        if pl.lora_a_t is not None:
          total += 2 * pl.rank * (pl.k * len(pl.seg_cols) + pl.n)
    return total, self.head.numel() * 2
