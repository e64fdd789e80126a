"""int4 group quantisation, dequantisation and the packed tile format.

Test infrastructure only (see oracle/__init__.py).

Reference arithmetic: the QLoRA recipe tunix/cli/utils/model.py:31-77 hands the
weights to the third-party module ``qwix`` (qwix>=0.1.6, pyproject.toml:48, not
vendored).  Its published weight-only rule is: symmetric per-tile absmax
calibration along the contraction axis, ``q = clip(round(w / scale), -8, 7)``,
and at call time ``w_deq = q.astype(scale.dtype) * scale`` followed by the
ordinary einsum.  ``quantize`` below restates that with the calibration bound as
a parameter (parity unpinned); ``dequantize`` is fully determined by (q, scale)
and is what the GPU must reproduce bit for bit.

Packed tile format (defined by this build, restated here independently of the
product's packer so that the two can be checked against each other):

  logical weight  W[K, N], K % 64 == 0, N % 32 == 0, nibble u = q + 8 in 0..15
  tile (nb, kb) covers k in [64 kb, 64 kb + 64), n in [32 nb, 32 nb + 32) and
  occupies 1024 bytes at byte offset ((nb * (K // 64)) + kb) * 1024
  inside a tile, "lane" l = 32 h + nl (h in {0,1}, nl = n % 32) owns 16 bytes at
  l * 16: four little-endian 32-bit words t = 0..3; nibble i (bits 4i..4i+3) of
  word t holds  k = 64 kb + 16 t + 8 h + 2 (i % 4) + (i // 4),  n = 32 nb + nl
  scales: bf16 [N // 32][K // G][32]  (n-tile major, group, column in tile)
"""
import numpy as np

from oracle.bf16 import bf16_round, bf16_bits, bf16_from_bits


def quantize(w, group, bound=7.5):
  """Symmetric absmax int4 quantisation of W[K, N] along K in groups.

  Returns (q int8 [K, N] in [-8, 7], scale float32-holding-bf16 [K // group, N]).
  A zero group gets scale 1 so that the quotient stays finite.
  """
  w = np.asarray(w, np.float32)
  k, n = w.shape
  assert k % group == 0
  wg = w.reshape(k // group, group, n)
  absmax = np.abs(wg).max(axis=1)
  scale = bf16_round(absmax / np.float32(bound))
  scale = np.where(scale == 0, np.float32(1.0), scale).astype(np.float32)
  q = np.rint(wg / scale[:, None, :])  # rint = round half to even
  q = np.clip(q, -8, 7).astype(np.int8).reshape(k, n)
  return q, scale


def dequantize(q, scale, group):
  """w_deq = bf16(q) * scale evaluated in bf16: one RNE rounding of the product.

  The float32 product of an int4 and a bf16 is exact (4 + 8 significant bits),
  so rounding it once to bf16 equals a native bf16 multiply.
  """
  k, n = q.shape
  s = np.repeat(np.asarray(scale, np.float32), group, axis=0)
  return bf16_round(q.astype(np.float32) * s)


def pack_tiles(q):
  """q int8 [K, N] -> uint8 [K * N // 2] in the tile format (plain loops)."""
  k, n = q.shape
  assert k % 64 == 0 and n % 32 == 0
  kt, nt = k // 64, n // 32
  words = np.zeros((nt, kt, 64, 4), dtype=np.uint32)
  u = (q.astype(np.int32) + 8).astype(np.uint32)
  for h in range(2):
    for t in range(4):
      for i in range(8):
        kk = 16 * t + 8 * h + 2 * (i % 4) + (i // 4)
        # rows kk of every k-tile, all columns -> [kt, n] -> [nt, kt, 32]
        sel = u[kk::64, :].reshape(kt, nt, 32).transpose(1, 0, 2)
        words[:, :, 32 * h:32 * h + 32, t] |= sel << np.uint32(4 * i)
  return words.reshape(-1).view(np.uint8).copy()


def unpack_tiles(packed, k, n):
  """Inverse of pack_tiles: uint8 buffer -> q int8 [K, N]."""
  kt, nt = k // 64, n // 32
  words = np.ascontiguousarray(packed).view(np.uint32).reshape(nt, kt, 64, 4)
  q = np.zeros((k, n), dtype=np.int8)
  for h in range(2):
    for t in range(4):
      for i in range(8):
        kk = 16 * t + 8 * h + 2 * (i % 4) + (i // 4)
        nib = (words[:, :, 32 * h:32 * h + 32, t] >> np.uint32(4 * i)) & np.uint32(15)
        val = nib.astype(np.int32) - 8  # [nt, kt, 32]
        q[kk::64, :] = val.transpose(1, 0, 2).reshape(kt, n).astype(np.int8)
  return q


def pack_scales(scale):
  """scale [K // G, N] (bf16 values) -> uint16 [N // 32, K // G, 32]."""
  g, n = scale.shape
  bits = bf16_bits(scale)
  return np.ascontiguousarray(bits.reshape(g, n // 32, 32).transpose(1, 0, 2))


def unpack_scales(packed, groups, n):
  bits = np.asarray(packed, np.uint16).reshape(n // 32, groups, 32)
  return bf16_from_bits(np.ascontiguousarray(bits.transpose(1, 0, 2)).reshape(groups, n))
