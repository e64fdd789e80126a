"""Host-side (offline) int4 group quantisation and packing into the q4t tile format.

Mirrors what the reference obtains from qwix through
tunix/cli/utils/model.py:31-77 (LoraProvider(weight_qtype='int4', tile_size=G)):
symmetric absmax calibration per group of G elements along the contraction axis,
q = clip(round_half_even(w / scale), -8, 7), bf16 scales.  The calibration bound
(absmax / bound) is a parameter because qwix's constant cannot be checked here.
Runs as torch tensor ops on whatever device the weight lives on.
"""
import torch


def quantize_int4(w, group, bound=7.5):
  """w [K, N] float/bf16 -> (q int8 [K, N], scale bf16 [K // group, N])."""
  k, n = w.shape
  if k % group:
    raise ValueError(f'K={k} is not a multiple of the group size {group}')
  wg = w.float().reshape(k // group, group, n)
  absmax = wg.abs().amax(dim=1)
  scale = (absmax / bound).to(torch.bfloat16)
  scale = torch.where(scale == 0, torch.ones_like(scale), scale)
  q = torch.round(wg / scale.float()[:, None, :]).clamp_(-8, 7)
  return q.reshape(k, n).to(torch.int8), scale


def pack_q4t(q):
  """q int8 [K, N] in [-8, 7] -> int32 [N // 32, K // 64, 64, 4] (the q4t tiles)."""
  k, n = q.shape
  if k % 64 or n % 32:
    raise ValueError(f'q4t needs K % 64 == 0 and N % 32 == 0, got {k}x{n}')
  kt, nt = k // 64, n // 32
  # k_in_tile = 16 t + 8 h + j with j = 2 p + c; nibble index i = p + 4 c.
  u = (q.to(torch.int64) + 8).reshape(kt, 4, 2, 4, 2, nt, 32)  # [kt, t, h, p, c, nt, nl]
  p = torch.arange(4, device=q.device).view(4, 1)
  c = torch.arange(2, device=q.device).view(1, 2)
  shift = (4 * (p + 4 * c)).view(1, 1, 1, 4, 2, 1, 1)
  words = (u << shift).sum(dim=(3, 4))  # [kt, t, h, nt, nl]
  words = words.permute(3, 0, 2, 4, 1).reshape(nt, kt, 64, 4)
  words = torch.where(words >= 2**31, words - 2**32, words)
  return words.to(torch.int32).contiguous()


def pack_scales(scale):
  """scale bf16 [K // G, N] -> bf16 [N // 32, K // G, 32]."""
  g, n = scale.shape
  return scale.reshape(g, n // 32, 32).permute(1, 0, 2).contiguous()


def pad32(r):
  return (r + 31) // 32 * 32


def pack_lora_a(a_list, k):
  """[A_i [K, r]] -> bf16 [K // 64, r_pad // 32, 4, 64, 8]: the A matrices side by side,
  zero-padded to a multiple of 32 columns, in MFMA B-fragment order: element
  A[64 kb + 16 t + 8 h + j][32 ct + c] at [kb][ct][t][32 h + c][j] (the operand of MFMA step
  t of a tile is 1 KiB contiguous: lane 32 h + c reads 16 bytes at 16 * lane)."""
  a = torch.cat([x.to(torch.bfloat16) for x in a_list], dim=1)  # [K, R]
  r = a.shape[1]
  rp = pad32(r)
  full = torch.zeros(k, rp, dtype=torch.bfloat16, device=a.device)
  full[:, :r] = a
  t = full.reshape(k // 64, 4, 2, 8, rp // 32, 32)  # [kb, t, h, j, ct, c]
  return t.permute(0, 4, 1, 2, 5, 3).reshape(k // 64, rp // 32, 4, 64, 8).contiguous()


class PackedLinear:
  """Device-resident q4t weight (+ optional LoRA) of one (possibly fused) projection.

  Several projections that share their input (q/k/v, gate/up) are fused by
  concatenating their columns; ``seg_cols`` lists the column count of each so
  that consumers pick the matching slice of t = x . [A_0 | A_1 | ...].
  """

  def __init__(self, k, n, group, qweight, scales, seg_cols, rank=0, lora_a_t=None, lora_b=None,
               lora_scale=0.0):
    self.k, self.n, self.group = k, n, group
    self.qweight, self.scales = qweight, scales
    self.seg_cols = list(seg_cols)
    self.rank = rank
    self.lora_a_t, self.lora_b, self.lora_scale = lora_a_t, lora_b, float(lora_scale)
    # > 1: `n` columns hold that many equally wide per-expert matrices side by side; a tile
    # column never straddles experts, so expert e's q4t tiles and scales are one contiguous
    # slice (the stacked layout the routed-expert kernel reads)
    self.experts = 1

  @property
  def r_pad(self):
    return 0 if self.lora_a_t is None else self.lora_a_t.shape[1] * 32

  def lora_a_dense(self):
    """[K, r_pad] view of the packed A (inverse of pack_lora_a)."""
    kt, ct = self.lora_a_t.shape[0], self.lora_a_t.shape[1]
    t = self.lora_a_t.reshape(kt, ct, 4, 2, 32, 8).permute(0, 2, 3, 5, 1, 4)  # [kb, t, h, j, ct, c]
    return t.reshape(kt * 64, ct * 32)

  @classmethod
  def from_dense(cls, ws, group, device, loras=None, lora_scale=0.0, bound=7.5):
    """ws: list of [K, N_i] float weights sharing K; loras: list of (A [K, r], B [r, N_i]) or None."""
    qs, ss = [], []
    for w in ws:
      q, s = quantize_int4(w.to(device), group, bound)
      qs.append(q)
      ss.append(s)
    return cls.from_quantized(qs, ss, group, device, loras, lora_scale)

  @classmethod
  def from_quantized(cls, qs, ss, group, device, loras=None, lora_scale=0.0):
    q = torch.cat([x.to(device) for x in qs], dim=1)
    s = torch.cat([x.to(device) for x in ss], dim=1)
    k, n = q.shape
    rank, a_t, b = 0, None, None
    if loras is not None and any(l is not None for l in loras):
      if not all(l is not None for l in loras):
        raise ValueError('either every fused projection has LoRA or none')
      rank = loras[0][0].shape[1]
      a_t = pack_lora_a([l[0].to(device) for l in loras], k)
      b = torch.cat([l[1].to(device).to(torch.bfloat16) for l in loras], dim=1).contiguous()
    return cls(k, n, group, pack_q4t(q), pack_scales(s.to(torch.bfloat16)), [x.shape[1] for x in qs],
               rank, a_t, b, lora_scale)

  def set_lora(self, loras):
    """Replaces A/B in place (the LoRA-only weight sync of Sampler.update_params)."""
    a_t = pack_lora_a([l[0].to(self.lora_a_t.device) for l in loras], self.k)
    b = torch.cat([l[1].to(self.lora_b.device).to(torch.bfloat16) for l in loras], dim=1)
    if a_t.shape != self.lora_a_t.shape or b.shape != self.lora_b.shape:
      raise ValueError('New state must have the same shape, dtype and sharding as the old state.')
    self.lora_a_t.copy_(a_t)
    self.lora_b.copy_(b)
