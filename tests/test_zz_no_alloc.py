"""The entry point that allocates nothing (static device scratch) against tmx_qlora_linear, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle.bf16 import bf16_round
from tunix_amd import _lib
from tunix_amd import quant

import gpu_util as G

pytestmark = pytest.mark.gpu
S = _lib.stream


def _case(M, K, N, group, r, seed):
  rng = np.random.default_rng(seed)
  w = bf16_round(rng.standard_normal((K, N)).astype(np.float32) * 0.02)
  x = bf16_round(rng.standard_normal((M, K)).astype(np.float32))
  res = bf16_round(rng.standard_normal((M, N)).astype(np.float32))
  a = bf16_round(rng.standard_normal((K, r)).astype(np.float32) * 0.02)
  b = bf16_round(rng.standard_normal((r, N)).astype(np.float32) * 0.02)
  pl = quant.PackedLinear.from_dense([torch.from_numpy(w)], group, G.DEV,
                                     [(torch.from_numpy(a), torch.from_numpy(b))], 2.0)
  return pl, G.bf(x), G.bf(res)


def _both(pl, xt, rs, M, K, N, group, r):
  lib = _lib.lib()
  ws = torch.empty(lib.tmx_qlora_linear_workspace_bytes(M, K, N), dtype=torch.uint8, device=G.DEV)
  want = torch.empty(M, N, dtype=torch.bfloat16, device=G.DEV)
  got = torch.full((M, N), float('nan'), dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_qlora_linear', S(), G.p(xt), G.p(pl.qweight), G.p(pl.scales), G.p(pl.lora_a_t), G.p(pl.lora_b),
         G.p(rs), G.p(want), G.p(ws), M, K, N, group, r, pl.r_pad, 2.0)
  G.call('tmx_qlora_linear_noalloc', S(), G.p(xt), G.p(pl.qweight), G.p(pl.scales), G.p(pl.lora_a_t),
         G.p(pl.lora_b), G.p(rs), G.p(got), M, K, N, group, r, pl.r_pad, 2.0)
  G.sync()
  return got, want


def test_noalloc_linear_equals_the_workspace_entry_point_twice_in_a_row():
  # two calls in a row on the same static buffer, the second smaller (stale planes of the first must not leak)
  for (M, K, N, group, r, seed) in [(64, 4096, 1024, 64, 16, 1), (7, 512, 96, 64, 8, 2)]:
    print('noalloc case', M, K, N, group, r, flush=True)
    pl, xt, rs = _case(M, K, N, group, r, seed)
    before = torch.cuda.memory_allocated()
    got, want = _both(pl, xt, rs, M, K, N, group, r)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, K, N)
    assert not torch.isnan(got.float()).any()
    del got, want
    assert torch.cuda.memory_allocated() <= before + 0  # nothing of the test itself stays allocated


def test_noalloc_rejects_requests_beyond_the_static_buffer():
  lib = _lib.lib()
  cap = lib.tmx_qlora_linear_noalloc_max_bytes()
  M, K, N = 4096, 4096, 28672
  assert lib.tmx_qlora_linear_workspace_bytes(M, K, N) > cap
  one = torch.zeros(8, dtype=torch.uint8, device=G.DEV)  # never dereferenced: the size check comes first
  rc = lib.tmx_qlora_linear_noalloc(S(), G.p(one), G.p(one), G.p(one), None, None, None, G.p(one), M, K, N, 64, 0,
                                    0, 0.0)
  assert rc == -5
  assert b'static buffer' in lib.tmx_status_string(rc)
