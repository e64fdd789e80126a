"""Helpers for the GPU parity tests: numpy <-> device tensors and thin C-ABI callers."""
import ctypes

import numpy as np
import torch

from tunix_amd import _lib

DEV = 'cuda'


def bf(x):
  """numpy f32 holding bf16 values -> device bf16 tensor."""
  return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.bfloat16).to(DEV)


def f32(x):
  return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(DEV)


def i32(x):
  return torch.from_numpy(np.ascontiguousarray(x, dtype=np.int32)).to(DEV)


def u8(x):
  return torch.from_numpy(np.ascontiguousarray(x, dtype=np.uint8)).to(DEV)


def host(t):
  return t.float().cpu().numpy()


def p(t):
  return None if t is None else t.data_ptr()


def ulp_bf16(ref):
  """One bf16 ulp at the magnitude of ref (elementwise)."""
  a = np.maximum(np.abs(ref), 2.0 ** -120).astype(np.float32)
  return np.exp2(np.floor(np.log2(a)) - 7).astype(np.float32)


def assert_bf16_close(got, ref, ulps=1.0, extra=0.0, min_exact=0.0, what='', stragglers=0):
  """|got - ref| <= ulps bf16 ulp + extra everywhere; `stragglers` elements (coincidences of several
  rounding flips in samples of millions) may reach three times that bound."""
  d = np.abs(got - ref)
  bound = ulps * ulp_bf16(np.maximum(np.abs(ref), np.abs(got))) + extra
  bad = d > bound
  if stragglers and 0 < bad.sum() <= stragglers:
    bad = d > 3.0 * bound
  assert not bad.any(), f'{what}: {bad.sum()} of {bad.size} beyond {ulps} bf16 ulp; worst {d.max()} at ref {ref.flat[d.argmax()]}'
  if min_exact:
    assert (d == 0).mean() >= min_exact, f'{what}: only {(d == 0).mean():.5f} exact'


def call(name, *args):
  lib = _lib.lib()
  rc = getattr(lib, name)(*args)
  _lib.check(rc, name)


def sync():
  torch.cuda.synchronize()


class Keep:
  """Creates device tensors and keeps them alive until the arena is dropped, returning raw
  pointers (a temporary tensor would be recycled by the caching allocator before the launch)."""

  def __init__(self):
    self.t = []

  def _k(self, t):
    self.t.append(t)
    return t.data_ptr()

  def bf(self, x):
    return self._k(bf(x))

  def f32(self, x):
    return self._k(f32(x))

  def i32(self, x):
    return self._k(i32(x))

  def u8(self, x):
    return self._k(u8(x))
