"""bfloat16 emulation on float32 numpy arrays (test infrastructure only).

A bf16 value is represented as a float32 whose low 16 bits are zero.
"""
import numpy as np


def bf16_round(x):
  """Round float32 -> nearest bf16 (ties to even), returned as float32.

  This is the rounding XLA applies for ``astype(bfloat16)`` and for the result
  of any op whose output dtype is bfloat16.
  """
  x = np.ascontiguousarray(x, dtype=np.float32)
  u = x.view(np.uint32)
  bias = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
  r = ((u + bias) & np.uint32(0xFFFF0000)).view(np.float32)
  nan = np.isnan(x)
  if nan.any():
    r = np.where(nan, x, r)
  return r


def bf16_bits(x):
  """float32 holding bf16 values -> uint16 bit patterns."""
  x = np.ascontiguousarray(x, dtype=np.float32)
  u = x.view(np.uint32)
  assert not np.any(u & np.uint32(0xFFFF)), 'value is not bf16-representable'
  return (u >> np.uint32(16)).astype(np.uint16)


def bf16_from_bits(b):
  """uint16 bit patterns -> float32 holding the bf16 values."""
  b = np.ascontiguousarray(b, dtype=np.uint16)
  return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


class Policy:
  """Where activations are rounded.

  ``bf16``: every op output is rounded to bf16 exactly where the reference's
  dtype rules round it ("reference rounding").  ``f32``: no rounding at all,
  used for cross-checks against fp32/fp64 library code.
  """

  def __init__(self, act='bf16'):
    assert act in ('bf16', 'f32')
    self.act = act

  def r(self, x):
    return bf16_round(x) if self.act == 'bf16' else np.asarray(x, np.float32)


BF16 = Policy('bf16')
F32 = Policy('f32')
