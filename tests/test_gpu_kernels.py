"""GPU parity of every kernel against the CPU oracle, called through the C ABI."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import int4
from oracle import layers as L
from oracle import prng
from oracle import sampling as OS
from oracle.bf16 import BF16, bf16_round, bf16_from_bits
from tunix_amd import _lib
from tunix_amd import quant

import gpu_util as G

pytestmark = pytest.mark.gpu
S = _lib.stream


def _packed(w, group, loras=None, ls=0.0):
  return quant.PackedLinear.from_dense([torch.from_numpy(w)], group, G.DEV,
                                       None if loras is None else [tuple(torch.from_numpy(m) for m in loras)], ls)


def test_int4_dequant_bit_exact_exhaustive():
  T = G.Keep()
  # every nibble value against 640 distinct bf16 scales, G = 64 and 128
  scales = bf16_from_bits(np.arange(0x3800, 0x3D00, 2, dtype=np.uint16))  # 640 scales
  n = scales.size
  rng = np.random.default_rng(0)
  for group in (64, 128):
    k = 2 * group
    q = rng.integers(-8, 8, (k, n)).astype(np.int8)
    q[:16, :] = np.arange(-8, 8, dtype=np.int8)[:, None]  # every nibble under every scale
    s = np.stack([scales, scales[::-1]])
    qw = quant.pack_q4t(torch.from_numpy(q)).to(G.DEV)
    st = quant.pack_scales(torch.from_numpy(s).to(torch.bfloat16)).to(G.DEV)
    out = torch.empty(k, n, dtype=torch.bfloat16, device=G.DEV)
    G.call('tmx_int4_dequant', S(), G.p(qw), G.p(st), G.p(out), k, n, group)
    G.sync()
    np.testing.assert_array_equal(G.host(out), int4.dequantize(q, s, group))


@pytest.mark.parametrize('M,K,N,group,r', [
    (1, 256, 96, 64, 0), (4, 256, 256, 64, 8), (7, 512, 96, 64, 8), (33, 1024, 160, 128, 16),
    (64, 2048, 1024, 64, 16), (100, 512, 256, 64, 32), (128, 4096, 512, 128, 32), (64, 14336, 256, 64, 16),
    # more than 128 rows: 256-row blocks (one partial, several, a ragged tail), with and without K-slices
    (129, 256, 96, 64, 8), (256, 512, 160, 64, 16), (300, 1024, 256, 128, 16), (700, 4096, 512, 64, 32),
    (1024, 2048, 384, 64, 0), (520, 1152, 4096, 128, 16),
    # unsplit at many rows: LoRA inside the projection's epilogue (ranks 8, 16 and 32, ragged rows)
    (1024, 256, 12288, 64, 8), (1030, 384, 12288, 128, 32), (1024, 256, 12288, 64, 0),
])
def test_qlora_linear_matches_oracle(M, K, N, group, r):
  T = G.Keep()
  rng = np.random.default_rng(M * 7 + N)
  w = bf16_round(rng.standard_normal((K, N)).astype(np.float32) * 0.02)
  x = bf16_round(rng.standard_normal((M, K)).astype(np.float32))
  res = bf16_round(rng.standard_normal((M, N)).astype(np.float32))
  a = b = None
  if r:
    a = bf16_round(rng.standard_normal((K, r)).astype(np.float32) * 0.02)
    b = bf16_round(rng.standard_normal((r, N)).astype(np.float32) * 0.02)
  pl = _packed(w, group, (a, b) if r else None, 2.0)
  qo, so = int4.quantize(w, group)
  lin = L.Linear(q=qo, scale=so, group=group, a=a, b=b, lora_scale=2.0)
  lib = _lib.lib()
  ws = torch.empty(lib.tmx_qlora_linear_workspace_bytes(M, K, N), dtype=torch.uint8, device=G.DEV)
  xt, rs = G.bf(x), G.bf(res)
  for use_res in (False, True):
    y = torch.empty(M, N, dtype=torch.bfloat16, device=G.DEV)
    G.call('tmx_qlora_linear', S(), G.p(xt), G.p(pl.qweight), G.p(pl.scales), G.p(pl.lora_a_t), G.p(pl.lora_b),
           G.p(rs) if use_res else None, G.p(y), G.p(ws), M, K, N, group, r, pl.r_pad, 2.0)
    G.sync()
    out = lin(x, BF16)
    ref = bf16_round(out + res) if use_res else out
    # f32 accumulation order differs: at most one bf16 ulp of the base projection (which the
    # LoRA / residual adds can turn into several ulps of a small sum), and only rarely
    base = bf16_round(x @ lin.weight())
    # a one-ulp flip of the base or of base + LoRA (before the residual is added) carries through
    # (both at once, in one element of millions: the two add)
    extra = G.ulp_bf16(base) + G.ulp_bf16(out) if (use_res or r) else 0.0
    if r:  # and a flip of the LoRA delta itself (rank sum in another order), scaled by lora_scale = 2
      extra = extra + 2.0 * G.ulp_bf16(out - base)
    # sums that cancel to far below their terms: the f32 accumulation error itself (eps32 x sum |x w|)
    extra = extra + 2.0 ** -23 * (np.abs(x) @ np.abs(lin.weight()))
    G.assert_bf16_close(G.host(y), ref, ulps=1.0, extra=extra,
                        min_exact=0.995, what=f'linear {M}x{K}x{N}')


def test_qlora_linear_planes_sum_and_rejects():
  T = G.Keep()
  rng = np.random.default_rng(1)
  M, K, N, group = 16, 1024, 128, 64
  w = bf16_round(rng.standard_normal((K, N)).astype(np.float32) * 0.02)
  x = bf16_round(rng.standard_normal((M, K)).astype(np.float32))
  pl = _packed(w, group)
  qo, so = int4.quantize(w, group)
  lib = _lib.lib()
  for ns in (1, 2, 4):
    yp = torch.zeros(ns, M, N, dtype=torch.float32, device=G.DEV)
    G.call('tmx_qlora_linear_planes', S(), T.bf(x), G.p(pl.qweight), G.p(pl.scales), None, G.p(yp), None,
           M, K, N, group, 0, ns)
    G.sync()
    exact = x.astype(np.float64) @ int4.dequantize(qo, so, group).astype(np.float64)
    np.testing.assert_allclose(G.host(yp.sum(0)), exact, rtol=0, atol=2e-5 * np.abs(exact).max())
  assert lib.tmx_qlora_linear_planes(S(), 1, 1, 1, None, 1, None, 129, 192, N, 64, 0, 1) == -2   # M > 128 needs K % 128 == 0
  assert lib.tmx_qlora_linear_planes(S(), 1, 1, 1, None, 1, None, M, K, N, 96, 0, 1) == -2      # G not a power of two
  assert lib.tmx_qlora_linear_planes(S(), 1, 1, 1, None, 1, None, M, K, N, group, 0, 3) == -2   # empty K-slice
  # LoRA slices: whole groups of 4 k-tiles for narrow projections, of 8 from 16 column blocks on
  assert lib.tmx_qlora_linear_num_lora_splits(4096, 1024) == 16 and lib.tmx_qlora_linear_num_lora_splits(14336, 4096) == 28
  assert lib.tmx_qlora_linear_num_lora_splits(4096, 6144) == 8 and lib.tmx_qlora_linear_num_lora_splits(4096, 4096) == 8


@pytest.mark.parametrize('family', [0, 1])
@pytest.mark.parametrize('M,D', [(1, 256), (5, 2048), (64, 4096), (3, 5120)])
def test_rmsnorm(family, M, D):
  T = G.Keep()
  rng = np.random.default_rng(D + family)
  x = bf16_round(rng.standard_normal((M, D)).astype(np.float32) * 3)
  w = bf16_round(rng.uniform(0.5, 1.5, D).astype(np.float32))
  y = torch.empty(M, D, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_rmsnorm', S(), T.bf(x), T.bf(w), G.p(y), M, D, 1e-5, family)
  G.sync()
  ref = (L.rmsnorm_llama3 if family == 0 else L.rmsnorm_qwen3)(x, w, 1e-5, BF16)
  G.assert_bf16_close(G.host(y), ref, ulps=1.0, min_exact=0.99, what='rmsnorm')


@pytest.mark.parametrize('family', [0, 1])
def test_lora_residual_rmsnorm_planes(family):
  T = G.Keep()
  rng = np.random.default_rng(3)
  M, D, r, ns = 9, 1024, 16, 3
  yp = rng.standard_normal((ns, M, D)).astype(np.float32)
  tp = rng.standard_normal((5, M, 128)).astype(np.float32)  # 5 LoRA planes: the generic sum
  b = bf16_round(rng.standard_normal((r, D)).astype(np.float32) * 0.05)
  res = bf16_round(rng.standard_normal((M, D)).astype(np.float32))
  w = bf16_round(rng.uniform(0.5, 1.5, D).astype(np.float32))
  x_out = torch.empty(M, D, dtype=torch.bfloat16, device=G.DEV)
  xn = torch.empty(M, D, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_lora_residual_rmsnorm', S(), None, T.f32(yp), ns, T.f32(tp), 5, 128, T.bf(b), r, 1.5,
         T.bf(res), G.p(x_out), T.bf(w), G.p(xn), M, D, 1e-6, family)
  G.sync()
  y = bf16_round(yp.sum(0))
  t = bf16_round(tp.sum(0)[:, :r])
  d = bf16_round(bf16_round(t @ b) * np.float32(1.5))
  h = bf16_round(bf16_round(y + d) + res)
  G.assert_bf16_close(G.host(x_out), h, ulps=1.0, min_exact=0.99, what='residual stream')
  got_h = G.host(x_out)
  ref = (L.rmsnorm_llama3 if family == 0 else L.rmsnorm_qwen3)(got_h, w, 1e-6, BF16)
  G.assert_bf16_close(G.host(xn), ref, ulps=1.0, min_exact=0.99, what='norm of residual')


@pytest.mark.parametrize('family,H,N,Kh', [(0, 64, 4, 4), (0, 128, 8, 2), (1, 128, 4, 2), (1, 64, 8, 8)])
def test_rope_kv_write(family, H, N, Kh):
  T = G.Keep()
  rng = np.random.default_rng(H + N)
  B, C, Lbuf, r, ns, step = 3, 12, 10, 8, 2, 5
  ntot = (N + 2 * Kh) * H
  qkv = rng.standard_normal((ns, B, ntot)).astype(np.float32)
  tp = rng.standard_normal((16, B, 128)).astype(np.float32)
  lb = bf16_round(rng.standard_normal((r, ntot)).astype(np.float32) * 0.05)
  qn = bf16_round(rng.uniform(0.5, 1.5, H).astype(np.float32))
  kn = bf16_round(rng.uniform(0.5, 1.5, H).astype(np.float32))
  positions = rng.integers(0, 700, (B, Lbuf)).astype(np.int32)
  kc = torch.full((B, C, Kh, H), 7.0, dtype=torch.bfloat16, device=G.DEV)
  vc = torch.full((B, C, Kh, H), 7.0, dtype=torch.bfloat16, device=G.DEV)
  q_out = torch.empty(B, N * H, dtype=torch.bfloat16, device=G.DEV)
  theta = 1_000_000.0 if family == 0 else 10_000.0
  G.call('tmx_rope_kv_write', S(), None, T.f32(qkv), ns, T.f32(tp), 16, 128, T.bf(lb), r, 2.0,
         T.bf(qn) if family else None, T.bf(kn) if family else None, T.i32(positions),
         T.i32([step]), Lbuf, G.p(q_out), G.p(kc), G.p(vc), B, N, Kh, H, C, theta, 1e-6, family)
  G.sync()
  y = bf16_round(qkv.sum(0))
  t = bf16_round(tp.sum(0))
  cols = np.arange(ntot)
  seg = np.where(cols < N * H, 0, np.where(cols < (N + Kh) * H, 1, 2))
  d = np.zeros_like(y)
  for s in range(3):
    d[:, seg == s] = bf16_round(bf16_round(t[:, s * r:(s + 1) * r] @ lb[:, seg == s]) * np.float32(2.0))
  y = bf16_round(y + d)
  q = y[:, :N * H].reshape(B, 1, N, H)
  k = y[:, N * H:(N + Kh) * H].reshape(B, 1, Kh, H)
  v = y[:, (N + Kh) * H:].reshape(B, Kh, H)
  pos = positions[:, step:step + 1]
  if family:
    q, k = L.rmsnorm_qwen3(q, qn, 1e-6, BF16), L.rmsnorm_qwen3(k, kn, 1e-6, BF16)
    q, k = L.rope_qwen3(q, pos, theta, BF16), L.rope_qwen3(k, pos, theta, BF16)
  else:
    q, k = L.rope_llama3(q, pos, theta, BF16), L.rope_llama3(k, pos, theta, BF16)
  # trig of angles up to ~700 rad: GPU and numpy sin/cos agree to ~1e-6 relative of the angle
  G.assert_bf16_close(G.host(q_out), q.reshape(B, -1), ulps=1.0, extra=2e-3, min_exact=0.97, what='q')
  kc_h, vc_h = G.host(kc), G.host(vc)
  G.assert_bf16_close(kc_h[:, step], k[:, 0], ulps=1.0, extra=2e-3, min_exact=0.97, what='k row')
  np.testing.assert_array_equal(vc_h[:, step], v)
  others = [i for i in range(C) if i != step]
  assert np.all(kc_h[:, others] == 7.0) and np.all(vc_h[:, others] == 7.0)


@pytest.mark.parametrize('M,F,ns,lora', [
    (3, 1024, 0, False), (64, 14336, 2, True), (5, 768, 1, True), (5, 768, 0, True),
    # more than 128 rows of bf16 input: 16 rows per workgroup, ragged last block and column tail
    (300, 2304, 0, True), (200, 1024, 0, False), (129, 4096, 0, True),
])
def test_swiglu(M, F, ns, lora):
  T = G.Keep()
  rng = np.random.default_rng(F + M)
  r = 16
  lb = bf16_round(rng.standard_normal((r, 2 * F)).astype(np.float32) * 0.05)
  act = torch.empty(M, F, dtype=torch.bfloat16, device=G.DEV)
  tp = rng.standard_normal((28, M, 128)).astype(np.float32)
  lora_args = (T.f32(tp), 28, 128, T.bf(lb), r, 2.0) if lora else (None, 0, 0, None, 0, 0.0)
  if ns == 0:
    y = bf16_round(rng.standard_normal((M, 2 * F)).astype(np.float32) * 2)
    G.call('tmx_swiglu', S(), T.bf(y), None, 0, *lora_args, G.p(act), M, F)
  else:
    gp = rng.standard_normal((ns, M, 2 * F)).astype(np.float32)
    G.call('tmx_swiglu', S(), None, T.f32(gp), ns, *lora_args, G.p(act), M, F)
    y = bf16_round(gp.sum(0))
  if lora:
    t = bf16_round(tp.sum(0))
    dg = bf16_round(bf16_round(t[:, :r] @ lb[:, :F]) * np.float32(2.0))
    du = bf16_round(bf16_round(t[:, r:2 * r] @ lb[:, F:]) * np.float32(2.0))
    y = np.concatenate([bf16_round(y[:, :F] + dg), bf16_round(y[:, F:] + du)], axis=1)
  G.sync()
  ref = bf16_round(L.silu(y[:, :F], BF16) * y[:, F:])
  G.assert_bf16_close(G.host(act), ref, ulps=1.0, min_exact=0.98, what='swiglu')


@pytest.mark.parametrize('M,K,F,group,r', [
    (4, 256, 128, 64, 8), (33, 768, 192, 64, 0), (64, 512, 256, 64, 16), (17, 1024, 320, 128, 16),
    (64, 2048, 1024, 64, 0), (40, 4096, 512, 64, 16), (100, 1024, 256, 64, 8), (128, 512, 128, 128, 0),
])
def test_fused_gate_up_swiglu_matches_oracle(M, K, F, group, r):
  """One launch for gate | up + LoRA + SwiGLU against the oracle's separate projections (K in
  multiples of 512 up to 64 rows runs the 8-wave kernel, the rest the 4-wave one)."""
  rng = np.random.default_rng(M + K + F)
  x = bf16_round(rng.standard_normal((M, K)).astype(np.float32))
  ws = [bf16_round(rng.standard_normal((K, F)).astype(np.float32) * 0.03) for _ in range(2)]
  loras = None
  if r:
    loras = [(bf16_round(rng.standard_normal((K, r)).astype(np.float32) * 0.03),
              bf16_round(rng.standard_normal((r, F)).astype(np.float32) * 0.03)) for _ in range(2)]
  pl = quant.PackedLinear.from_dense([torch.from_numpy(w) for w in ws], group, G.DEV,
                                     None if loras is None else [tuple(torch.from_numpy(m) for m in l) for l in loras],
                                     2.0)
  ys, flips = [], []
  for i, w in enumerate(ws):
    qo, so = int4.quantize(w, group)
    lin = L.Linear(q=qo, scale=so, group=group, a=loras[i][0] if r else None, b=loras[i][1] if r else None,
                   lora_scale=2.0)
    ys.append(lin(x, BF16))
    # how far rounding flips can move g or u: one ulp of the base projection, of the LoRA delta (times
    # lora_scale = 2) and of their sum, which may be far smaller than its terms
    base = bf16_round(x @ lin.weight())
    flips.append(G.ulp_bf16(base) + 2.0 * G.ulp_bf16(ys[i] - base) + G.ulp_bf16(ys[i]))
    if r:  # a flip of a bf16(x . A) value (its K-slices are summed in another order) moves the whole delta row
      flips[-1] = flips[-1] + 2.0 * (G.ulp_bf16(bf16_round(x @ loras[i][0])) @ np.abs(loras[i][1]))
  ref = bf16_round(L.silu(ys[0], BF16) * ys[1])
  xt = G.bf(x)
  act = torch.empty(M, F, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_qlora_gate_up_swiglu', S(), G.p(xt), G.p(pl.qweight), G.p(pl.scales), G.p(pl.lora_a_t),
         G.p(pl.lora_b), G.p(act), M, K, F, group, r, 2.0)
  G.sync()
  # a one-ulp flip of g or u (f32 summation order) moves the product by about one ulp of it,
  # silu' <= 1.1 adds a little, and both can flip; rare
  # (with the flips of g and u themselves as derived above: d(silu)/dg <= 1.1)
  extra = 2.5 * np.maximum(G.ulp_bf16(ref), G.ulp_bf16(ys[0]) * np.abs(ys[1]))
  extra = np.maximum(extra, 1.1 * flips[0] * np.abs(ys[1]) + flips[1] * np.abs(L.silu(ys[0], BF16)) + G.ulp_bf16(ref))
  G.assert_bf16_close(G.host(act), ref, ulps=1.0, extra=extra, min_exact=0.97, what=f'gate_up {M}x{K}x{F}')
  assert _lib.lib().tmx_qlora_gate_up_swiglu(S(), G.p(xt), G.p(pl.qweight), G.p(pl.scales), None, None, G.p(act),
              M, K, F + 32, group, 0, 0.0) != 0


@pytest.mark.parametrize('M,K,F,group,r', [
    (5, 1024, 256, 64, 8), (32, 512, 128, 64, 16), (33, 2048, 512, 64, 16), (48, 4096, 256, 128, 16),
    (64, 1024, 1024, 64, 16), (64, 4096, 1024, 64, 12),
])
def test_fused_gate_up_handover_matches_oracle(M, K, F, group, r):
  """tmx_qlora_gate_up_swiglu_handover: the form of the fused gate | up launch that the decode step runs with
  LoRA at up to 64 rows (x . A computed once by K / 256 extra workgroups and handed over through memory;
  8 producers of 8 k-tiles up to 32 rows, 16 of 4 above) against the oracle's separate projections
  (tunix/models/llama3/model.py:489-496), twice in a row on one workspace: its state must be back at zero."""
  lib = _lib.lib()
  rng = np.random.default_rng(M + K + F + 1)
  x = bf16_round(rng.standard_normal((M, K)).astype(np.float32))
  ws = [bf16_round(rng.standard_normal((K, F)).astype(np.float32) * 0.03) for _ in range(2)]
  loras = [(bf16_round(rng.standard_normal((K, r)).astype(np.float32) * 0.03),
            bf16_round(rng.standard_normal((r, F)).astype(np.float32) * 0.03)) for _ in range(2)]
  pl = quant.PackedLinear.from_dense([torch.from_numpy(w) for w in ws], group, G.DEV,
                                     [tuple(torch.from_numpy(m) for m in l) for l in loras], 2.0)
  ys, flips = [], []
  for i, w in enumerate(ws):
    qo, so = int4.quantize(w, group)
    lin = L.Linear(q=qo, scale=so, group=group, a=loras[i][0], b=loras[i][1], lora_scale=2.0)
    ys.append(lin(x, BF16))
    base = bf16_round(x @ lin.weight())
    f = G.ulp_bf16(base) + 2.0 * G.ulp_bf16(ys[i] - base) + G.ulp_bf16(ys[i])
    flips.append(f + 2.0 * (G.ulp_bf16(bf16_round(x @ loras[i][0])) @ np.abs(loras[i][1])))
  ref = bf16_round(L.silu(ys[0], BF16) * ys[1])
  nb = lib.tmx_qlora_gate_up_swiglu_handover_bytes(M, K, F, r)
  assert nb > 0
  wsb = torch.full((nb,), 0xAB, dtype=torch.uint8, device=G.DEV)  # the call clears the state block itself
  xt = G.bf(x)
  outs = []
  for _ in range(2):
    act = torch.full((M, F), float('nan'), dtype=torch.bfloat16, device=G.DEV)
    G.call('tmx_qlora_gate_up_swiglu_handover', S(), G.p(xt), G.p(pl.qweight), G.p(pl.scales), G.p(pl.lora_a_t),
           G.p(pl.lora_b), G.p(act), G.p(wsb), M, K, F, group, r, 2.0)
    G.call('tmx_handover_status', S(), G.p(wsb))
    outs.append(G.host(act))
  np.testing.assert_array_equal(outs[0], outs[1])
  assert int(wsb[:256].view(torch.int32).abs().sum().item()) == 0
  extra = 2.5 * np.maximum(G.ulp_bf16(ref), G.ulp_bf16(ys[0]) * np.abs(ys[1]))
  extra = np.maximum(extra, 1.1 * flips[0] * np.abs(ys[1]) + flips[1] * np.abs(L.silu(ys[0], BF16)) + G.ulp_bf16(ref))
  G.assert_bf16_close(outs[1], ref, ulps=1.0, extra=extra, min_exact=0.97, what=f'gate_up hand-over {M}x{K}x{F}')
  # and against the form in which every workgroup multiplies by A itself: the same t up to the order its K-slices are added in
  act1 = torch.empty(M, F, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_qlora_gate_up_swiglu', S(), G.p(xt), G.p(pl.qweight), G.p(pl.scales), G.p(pl.lora_a_t),
         G.p(pl.lora_b), G.p(act1), M, K, F, group, r, 2.0)
  G.sync()
  assert (G.host(act1) == outs[1]).mean() > 0.97


def test_handover_status_word_and_shape_limits():
  """tmx_handover_status reports a set "wait ran out" word once and clears it (the word is written here from
  the host: no kernel is made to wait); shapes outside the hand-over form are refused with a zero size."""
  lib = _lib.lib()
  assert lib.tmx_qlora_gate_up_swiglu_handover_bytes(64, 4096, 14336, 16) > 0
  assert lib.tmx_qlora_gate_up_swiglu_handover_bytes(65, 4096, 14336, 16) == 0   # more than 64 rows
  assert lib.tmx_qlora_gate_up_swiglu_handover_bytes(64, 4096 + 256, 14336, 16) == 0  # K % 512
  assert lib.tmx_qlora_gate_up_swiglu_handover_bytes(64, 4096, 14336, 17) == 0   # 2 r > 32
  assert lib.tmx_qlora_gate_up_swiglu_handover_bytes(64, 4096, 64 * 300, 16) == 0  # more workgroups than compute units
  assert lib.tmx_qlora_gate_up_swiglu_handover(S(), 1, 1, 1, 1, 1, 1, 1, 65, 4096, 14336, 64, 16, 2.0) == -4
  ws = torch.zeros(1024, dtype=torch.uint8, device=G.DEV)
  assert lib.tmx_handover_status(S(), G.p(ws)) == 0
  ws[252:256] = torch.tensor([1, 0, 0, 0], dtype=torch.uint8, device=G.DEV)
  assert lib.tmx_handover_status(S(), G.p(ws)) == -6
  assert lib.tmx_handover_status(S(), G.p(ws)) == 0
  assert lib.tmx_handover_status(S(), None) == -1


@pytest.mark.parametrize('B,N,Kh,H,C,step', [
    (2, 4, 4, 64, 64, 40), (3, 8, 2, 64, 96, 95), (2, 8, 4, 64, 33, 0), (4, 32, 8, 128, 300, 257),
    (2, 8, 1, 128, 128, 100), (1, 32, 8, 64, 768, 700), (2, 16, 8, 128, 520, 519), (1, 4, 4, 128, 16, 7),
    # the 8B Qwen3 workload's cache (512-token prompts + 1024 new tokens) near its end and at an early step
    (3, 32, 8, 128, 1536, 1500), (2, 32, 8, 128, 1536, 513),
])
def test_gqa_decode_attention(B, N, Kh, H, C, step):
  T = G.Keep()
  rng = np.random.default_rng(B * 1000 + C)
  Lbuf = C
  q = bf16_round(rng.standard_normal((B, 1, N, H)).astype(np.float32))
  k = bf16_round(rng.standard_normal((B, C, Kh, H)).astype(np.float32))
  v = bf16_round(rng.standard_normal((B, C, Kh, H)).astype(np.float32))
  in_mask = np.ones((B, Lbuf), bool)
  for b in range(B):  # left padding of different lengths plus a hole (a pad id inside a prompt)
    in_mask[b, : (b * 5) % max(step, 1)] = False
  if step > 3:
    in_mask[0, step // 2] = False
  in_mask[:, step] = True
  lib = _lib.lib()
  ws_bytes = lib.tmx_gqa_decode_workspace_bytes(B, N, Kh, H, C)
  ws = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=G.DEV)
  out = torch.empty(B, N * H, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_gqa_decode_attention', S(), T.bf(q), T.bf(k), T.bf(v), T.u8(in_mask),
         T.i32([step]), Lbuf, G.p(out), G.p(ws), B, N, Kh, H, C)
  G.sync()
  from oracle import masks as OMK
  mask = OMK.compute_attention_masks(step, C, ~in_mask)
  fused = L.gqa_attention(q, k, v, mask, BF16, 'fused').reshape(B, -1)
  ref = L.gqa_attention(q, k, v, mask, BF16, 'reference').reshape(B, -1)
  got = G.host(out)
  # kernel keeps f32 inside: 1 ulp against the f32-internal oracle, bf16 noise against the
  # reference-rounding oracle (scores and probabilities rounded to bf16 there)
  G.assert_bf16_close(got, fused, ulps=1.0, extra=1e-3, what='attention vs f32-internal oracle')
  assert np.abs(got - ref).max() < 2e-2


@pytest.mark.parametrize('B,N,Kh,H,C,step,gs,sl', [
    (8, 8, 2, 64, 96, 70, 4, 32),        # two groups of four, one block of shared slots
    (6, 4, 4, 128, 200, 150, 3, 64),     # one query head per kv head, groups of three
    (16, 16, 8, 64, 300, 100, 16, 128),  # the step has not left the shared slots yet: they are walked up to it
    (8, 32, 8, 128, 128, 63, 8, 64),     # first decode step after the prompt: no private slot yet
    (12, 8, 2, 128, 400, 333, 6, 50),    # shared length that is no multiple of 32, two query blocks per group
    (64, 32, 8, 128, 768, 520, 8, 256),  # the 8B rollout: 8 prompts x 8 samples at mid-generation
    (64, 32, 8, 128, 768, 767, 8, 256),
    (128, 32, 8, 128, 512, 300, 32, 224),  # four query blocks per group, one split of the shared slots
])
def test_gqa_decode_attention_with_shared_prompt_slots(B, N, Kh, H, C, step, gs, sl):
  """tmx_gqa_decode_attention_shared: groups of gs sequences whose first sl cache slots and mask entries are
  the same (the samples of one prompt, tunix/rl/rl_learner.py:432-435) against the oracle's attention of
  every sequence over its own cache (tunix/models/llama3/model.py:379-396, mask of
  tunix/generate/utils.py:35-59).  The shared slots of every sequence but a group's first are poisoned with
  NaN in the device copy: the result stays finite, i.e. those rows are read once per group."""
  T = G.Keep()
  rng = np.random.default_rng(B * 1000 + C + gs)
  q = bf16_round(rng.standard_normal((B, 1, N, H)).astype(np.float32))
  k = bf16_round(rng.standard_normal((B, C, Kh, H)).astype(np.float32))
  v = bf16_round(rng.standard_normal((B, C, Kh, H)).astype(np.float32))
  in_mask = np.ones((B, C), bool)
  lead = (np.arange(B) // gs) * gs
  for b in range(B):
    in_mask[b, : (lead[b] * 5 + 3) % max(min(step, sl) - 1, 1)] = False     # left padding, the same within a group
    if step > sl + 8:
      in_mask[b, sl + (b % 5)] = False                                      # and a private hole behind the prompt
  in_mask[0, min(step, sl) // 2] = False
  in_mask[:gs] &= in_mask[0]
  in_mask[:, step] = True
  k[:, :sl], v[:, :sl] = k[lead, :sl], v[lead, :sl]
  in_mask[:, :sl] = in_mask[lead, :sl]
  lib = _lib.lib()
  ws = torch.empty(lib.tmx_gqa_decode_shared_workspace_bytes(B, N, Kh, H, C), dtype=torch.uint8, device=G.DEV)
  out = torch.full((B, N * H), float('nan'), dtype=torch.bfloat16, device=G.DEV)
  kd, vd = G.bf(k), G.bf(v)
  follower = torch.from_numpy(np.arange(B) != lead).to(G.DEV)
  kd[follower, :sl] = float('nan')
  vd[follower, :sl] = float('nan')
  G.call('tmx_gqa_decode_attention_shared', S(), T.bf(q), G.p(kd), G.p(vd), T.u8(in_mask), T.i32([step]), C,
         G.p(out), G.p(ws), B, N, Kh, H, C, gs, sl)
  G.sync()
  from oracle import masks as OMK
  mask = OMK.compute_attention_masks(step, C, ~in_mask)
  fused = L.gqa_attention(q, k, v, mask, BF16, 'fused').reshape(B, -1)
  ref = L.gqa_attention(q, k, v, mask, BF16, 'reference').reshape(B, -1)
  got = G.host(out)
  assert np.isfinite(got).all()
  G.assert_bf16_close(got, fused, ulps=1.0, extra=1e-3, what='shared attention vs f32-internal oracle')
  assert np.abs(got - ref).max() < 2e-2
  # what the shared walk does not serve is refused, not silently run per row
  assert lib.tmx_gqa_decode_attention_shared(S(), 1, 1, 1, 1, 1, 1, C, 1, 1, B, N, Kh, H, C, gs, 16) == -4
  assert lib.tmx_gqa_decode_attention_shared(S(), 1, 1, 1, 1, 1, 1, C, 1, 1, B + 1, N, Kh, H, C, gs, sl) == -4


@pytest.mark.parametrize('nseq,T,N,Kh,H,C,step', [
    (2, 40, 4, 4, 64, 64, 3), (3, 9, 8, 2, 64, 96, 50), (2, 33, 32, 8, 128, 300, 200), (1, 64, 8, 1, 128, 128, 0),
    (2, 5, 16, 8, 128, 96, 60), (1, 128, 4, 4, 128, 200, 31), (2, 3, 8, 4, 64, 64, 20),
])
def test_gqa_attention_rows(nseq, T, N, Kh, H, C, step):
  """T consecutive query tokens per sequence against the per-token oracle (row t sees slots <= step + t)."""
  Tk = G.Keep()
  rng = np.random.default_rng(nseq * 1000 + C + T)
  q = bf16_round(rng.standard_normal((nseq, T, N, H)).astype(np.float32))
  k = bf16_round(rng.standard_normal((nseq, C, Kh, H)).astype(np.float32))
  v = bf16_round(rng.standard_normal((nseq, C, Kh, H)).astype(np.float32))
  in_mask = np.ones((nseq, C), bool)
  for b in range(nseq):  # left padding of different lengths plus a hole
    in_mask[b, : (b * 5 + 2) % max(step, 1)] = False
  in_mask[0, (step + T) // 2] = False
  in_mask[:, step] = True
  lib = _lib.lib()
  ws = torch.empty(max(lib.tmx_gqa_decode_workspace_bytes(nseq * T, N, Kh, H, C), 4), dtype=torch.uint8, device=G.DEV)
  out = torch.empty(nseq * T, N * H, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_gqa_attention_rows', S(), Tk.bf(q.reshape(nseq * T, N * H)), Tk.bf(k), Tk.bf(v), Tk.u8(in_mask),
         Tk.i32([step]), C, G.p(out), G.p(ws), nseq, T, N, Kh, H, C)
  G.sync()
  from oracle import masks as OMK
  got = G.host(out).reshape(nseq, T, N * H)
  for t in range(T):
    mask = OMK.compute_attention_masks(step + t, C, ~in_mask)
    fused = L.gqa_attention(q[:, t:t + 1], k, v, mask, BF16, 'fused').reshape(nseq, -1)
    ref = L.gqa_attention(q[:, t:t + 1], k, v, mask, BF16, 'reference').reshape(nseq, -1)
    # as the one-token kernel: 1 ulp against the f32-internal oracle, bf16 noise against the
    # reference-rounding oracle
    G.assert_bf16_close(got[:, t], fused, ulps=1.0, extra=1e-3, what=f'attention rows, token {t}')
    assert np.abs(got[:, t] - ref).max() < 2e-2, (t, np.abs(got[:, t] - ref).max())


def _head_inputs(M, D, V, seed):
  rng = np.random.default_rng(seed)
  x = bf16_round(rng.standard_normal((M, D)).astype(np.float32))
  w = bf16_round(rng.standard_normal((V, D)).astype(np.float32) * 0.05)
  return x, w


def head_tiles_layout(w):
  """The streaming copy of a head matrix, restated from the C header: tiles of 32 rows x 64 columns, the
  tiles of a row block one after the other; inside a tile the 8 elements w[32 vt + n, 64 kt + 32 h + 8 t : + 8]
  at element (t * 64 + 32 h + n) * 8.  Plain loops over the pieces."""
  V, D = w.shape
  out = np.empty(V * D, w.dtype)
  for vt in range(V // 32):
    for kt in range(D // 64):
      base = (vt * (D // 64) + kt) * 2048
      for t in range(4):
        for h in range(2):
          for n in range(32):
            k0 = 64 * kt + 32 * h + 8 * t
            out[base + (t * 64 + 32 * h + n) * 8: base + (t * 64 + 32 * h + n) * 8 + 8] = w[32 * vt + n, k0:k0 + 8]
  return out


def test_head_tiles_pack_writes_the_documented_layout():
  T = G.Keep()
  V, D = 96, 192
  w = bf16_round(np.random.default_rng(3).standard_normal((V, D)).astype(np.float32))
  tiles = torch.zeros(V * D, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_head_tiles_pack', S(), T.bf(w), G.p(tiles), V, D)
  G.sync()
  np.testing.assert_array_equal(tiles.float().cpu().numpy(), head_tiles_layout(w))
  # shapes the layout does not cover are refused before anything is launched
  lib = _lib.lib()
  assert lib.tmx_head_tiles_pack(S(), T.bf(w), G.p(tiles), 80, 192) != 0
  assert lib.tmx_head_tiles_pack(S(), T.bf(w), G.p(tiles), 96, 96) != 0


HEAD_LAYOUT = 'rows'  # 'tiles': _run_head hands the kernel the streaming copy (tmx_head_sample_tiles)


@pytest.fixture(params=['rows', 'tiles'])
def head_layout(request):
  global HEAD_LAYOUT
  HEAD_LAYOUT = request.param
  yield request.param
  HEAD_LAYOUT = 'rows'


def _run_head(x, w, mode, temperature, key, step, forbidden=(), eos=(-1,), col_len=20):
  T = G.Keep()
  M, D = x.shape
  V = w.shape[0]
  lib = _lib.lib()
  ws = torch.empty(lib.tmx_head_sample_workspace_bytes(M, V), dtype=torch.uint8, device=G.DEV)
  tok = torch.full((M, col_len), -5, dtype=torch.int32, device=G.DEV)
  lp = torch.zeros(M, col_len, dtype=torch.float32, device=G.DEV)
  done = torch.zeros(M, dtype=torch.uint8, device=G.DEV)
  logits = torch.empty(M, V, dtype=torch.float32, device=G.DEV)
  fb = T.i32(list(forbidden)) if forbidden else None
  entry, wd = 'tmx_head_sample', T.bf(w)
  if HEAD_LAYOUT == 'tiles':
    tiles = torch.empty(V * D, dtype=torch.bfloat16, device=G.DEV)
    G.call('tmx_head_tiles_pack', S(), wd, G.p(tiles), V, D)
    entry, wd = 'tmx_head_sample_tiles', G.p(tiles)
  G.call(entry, S(), T.bf(x), wd, M, D, V, mode, temperature, int(key[0]), int(key[1]),
         T.i32([step]), fb, len(forbidden), T.i32(list(eos)), len(eos), G.p(tok), G.p(lp),
         G.p(done), col_len, G.p(logits), G.p(ws))
  G.sync()
  return tok.cpu().numpy(), lp.cpu().numpy(), done.cpu().numpy(), logits.cpu().numpy()


@pytest.mark.parametrize('M,D,V', [(1, 256, 1024), (40, 320, 2080), (64, 4096, 1024)])
def test_head_from_tiles_equals_head_from_rows_bit_for_bit(M, D, V):
  """Both layouts feed the same 16-byte pieces to the same matrix instructions in the same order: logits,
  tokens and log-probs are identical, greedy and sampled."""
  global HEAD_LAYOUT
  x, w = _head_inputs(M, D, V, 3 * M + V)
  for mode, temp, key in ((0, 1.0, (0, 0)), (1, 0.7, prng.prng_key(4))):
    outs = {}
    for HEAD_LAYOUT in ('rows', 'tiles'):
      outs[HEAD_LAYOUT] = _run_head(x, w, mode, temp, key, 2)
    HEAD_LAYOUT = 'rows'
    for a, b in zip(outs['rows'], outs['tiles']):
      np.testing.assert_array_equal(a, b)


@pytest.mark.parametrize('M,D,V', [(1, 256, 1024), (5, 512, 4096), (64, 256, 1056), (100, 128, 2048)])
def test_head_greedy(M, D, V, head_layout):
  T = G.Keep()
  x, w = _head_inputs(M, D, V, M + V)
  step = 3
  tok, lp, done, logits = _run_head(x, w, 0, 1.0, (0, 0), step, eos=(int(0),))
  ref_logits = bf16_round(x @ w.T)
  G.assert_bf16_close(logits, ref_logits, ulps=1.0, min_exact=0.995, what='logits')
  # selection and log-softmax are exact functions of the kernel's own logits
  want_tok, want_lp = OS.sample_best(logits)
  np.testing.assert_array_equal(tok[:, step + 1], want_tok)
  np.testing.assert_allclose(lp[:, step + 1], want_lp, atol=2e-5)
  assert np.all(tok[:, :step + 1] == -5) and np.all(tok[:, step + 2:] == -5)
  np.testing.assert_array_equal(done, (want_tok == 0).astype(np.uint8))
  # against the oracle's logits: same token wherever the top-2 margin exceeds the tolerance
  o_tok, o_lp = OS.sample_best(ref_logits)
  srt = np.sort(ref_logits, axis=-1)
  clear = (srt[:, -1] - srt[:, -2]) > 2e-2
  np.testing.assert_array_equal(tok[clear, step + 1], o_tok[clear])
  assert clear.sum() == 0 or np.abs(lp[clear, step + 1] - o_lp[clear]).max() <= 1e-2


def test_head_scoring_clips_logits_like_the_reference():
  """TMX_SAMPLE_SCORE follows selective_log_softmax (tunix/rl/common.py:217-221): NaN logits count
  as -1e9, the others are clipped to [-1e9, 1e9], so every score is finite.  Row 0 of x is 1e10:
  vocabulary row 7 (+1e30) gives +inf, row 9 -inf, row 11 (alternating signs) inf - inf = NaN, and
  most ordinary logits of that row are beyond the clip."""
  from oracle import scoring
  M, D, V, step, col_len = 4, 256, 1024, 2, 8
  x, w = _head_inputs(M, D, V, 77)
  x[0, :] = 1e10
  w[7, :] = 1e30
  w[9, :] = -1e30
  w[11, :] = np.where(np.arange(D) % 2 == 0, 1e30, -1e30)
  x, w = bf16_round(x), bf16_round(w)
  targets = np.array([[7, 9, 11, 500], [7, 9, 11, 500], [3, 7, 100, 11], [9, 1, 2, 3]], np.int32)
  lib = _lib.lib()
  for col in range(4):
    T = G.Keep()
    ws = torch.empty(lib.tmx_head_sample_workspace_bytes(M, V), dtype=torch.uint8, device=G.DEV)
    tok = torch.full((M, col_len), -5, dtype=torch.int32, device=G.DEV)
    tok[:, step + 1] = torch.from_numpy(targets[:, col]).to(G.DEV)
    lp = torch.zeros(M, col_len, dtype=torch.float32, device=G.DEV)
    done = torch.zeros(M, dtype=torch.uint8, device=G.DEV)
    logits = torch.empty(M, V, dtype=torch.float32, device=G.DEV)
    G.call('tmx_head_sample', S(), T.bf(x), T.bf(w), M, D, V, 2, 0.5, 0, 0, T.i32([step]), None, 0,
           T.i32([-1]), 1, G.p(tok), G.p(lp), G.p(done), col_len, G.p(logits), G.p(ws))
    G.sync()
    lg, got = logits.cpu().numpy(), lp.cpu().numpy()[:, step + 1]
    if col == 0:
      assert lg[0, 7] == np.inf and lg[0, 9] == -np.inf and np.isnan(lg[0, 11])
      rest = np.delete(lg[0], [7, 9, 11])
      assert np.isfinite(rest).all() and (np.abs(rest) > 1e9).mean() > 0.5  # most are beyond the clip
    # exact function of the kernel's own logits
    want = scoring.selective_log_softmax(lg / np.float32(0.5), targets[:, col])
    assert np.isfinite(got).all()
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=2e-5)
    np.testing.assert_array_equal(tok.cpu().numpy()[:, step + 1], targets[:, col])  # scoring chooses nothing
  # row 0: +inf scores 0 against the normaliser 1e9 + log(count), NaN and -inf score -2e9
  # (checked on the last column's neighbours through the closed form of the oracle pin)


def test_head_greedy_ties_pick_first_index_and_forbidden(head_layout):
  T = G.Keep()
  M, D, V = 3, 128, 1024
  x, w = _head_inputs(M, D, V, 5)
  w[700] = w[13]
  w[900] = w[13]
  x[:] = bf16_round(w[13] * 4)[None, :]  # row 13 (and its copies) win by a wide margin
  tok, lp, _, logits = _run_head(x, w, 0, 1.0, (0, 0), 0)
  assert logits[0, 13] == logits[0, 700] == logits[0, 900] == logits[0].max()
  assert np.all(tok[:, 1] == 13)
  tok, _, _, _ = _run_head(x, w, 0, 1.0, (0, 0), 0, forbidden=(13,))
  assert np.all(tok[:, 1] == 700)
  tok, lp, _, _ = _run_head(x, w, 0, 1.0, (0, 0), 0, forbidden=(13, 700, 900, 5))
  assert not np.isin(tok[:, 1], [13, 700, 900, 5]).any() and np.isfinite(lp[:, 1]).all()


@pytest.mark.parametrize('M,D,V,temp', [(4, 256, 1024, 0.9), (64, 128, 4096, 1.0), (33, 256, 2080, 0.7)])
def test_head_temperature_sampling_matches_threefry_oracle(M, D, V, temp, head_layout):
  T = G.Keep()
  x, w = _head_inputs(M, D, V, V + 1)
  seed_key = prng.prng_key(1234)
  step = 6
  tok, lp, _, logits = _run_head(x, w, 1, temp, seed_key, step)
  z = (logits / np.float32(temp)).astype(np.float32)
  key = prng.fold_in(seed_key, step)
  noisy = z + prng.gumbel(key, z.shape)
  want = np.argmax(noisy, axis=-1)
  srt = np.sort(noisy, axis=-1)
  clear = (srt[:, -1] - srt[:, -2]) > 1e-4  # GPU logf differs from numpy by an ulp or two
  assert clear.mean() > 0.9
  np.testing.assert_array_equal(tok[clear, step + 1], want[clear])
  want_lp = OS.log_softmax(z)[np.arange(M), tok[:, step + 1]]
  np.testing.assert_allclose(lp[:, step + 1], want_lp, atol=3e-5)
  # a different step or seed gives a different draw
  tok2, _, _, _ = _run_head(x, w, 1, temp, seed_key, step + 1)
  tok3, _, _, _ = _run_head(x, w, 1, temp, prng.prng_key(99), step)
  if M >= 16:
    assert (tok2[:, step + 2] != tok[:, step + 1]).mean() > 0.5
    assert (tok3[:, step + 1] != tok[:, step + 1]).mean() > 0.5


def _run_nucleus(x, w, temperature, top_p, top_k, key, step, forbidden=(), eos=(-1,), col_len=20):
  T = G.Keep()
  M, D = x.shape
  V = w.shape[0]
  lib = _lib.lib()
  ws = torch.empty(lib.tmx_head_sample_workspace_bytes(M, V), dtype=torch.uint8, device=G.DEV)
  nb = lib.tmx_nucleus_workspace_bytes(M, V)
  assert nb > 0
  nws = torch.empty(nb, dtype=torch.uint8, device=G.DEV)
  tok = torch.full((M, col_len), -5, dtype=torch.int32, device=G.DEV)
  lp = torch.zeros(M, col_len, dtype=torch.float32, device=G.DEV)
  done = torch.zeros(M, dtype=torch.uint8, device=G.DEV)
  fb = T.i32(list(forbidden)) if forbidden else None
  G.call('tmx_head_sample_nucleus', S(), T.bf(x), T.bf(w), M, D, V, temperature, top_p, top_k or 0,
         int(key[0]), int(key[1]), T.i32([step]), fb, len(forbidden), T.i32(list(eos)), len(eos), G.p(tok),
         G.p(lp), G.p(done), col_len, G.p(ws), G.p(nws), nb)
  G.sync()
  return tok.cpu().numpy(), lp.cpu().numpy(), done.cpu().numpy()


def _nucleus_clear_rows(z, key, top_p, top_k):
  """Rows whose outcome cannot flip on f32 rounding: the cut is not within 8e-6 of top_p (the
  running sum is accumulated in another order on the GPU) and the winning noisy key leads by 1e-4."""
  k = z.shape[1] if not top_k else top_k
  order = np.argsort(-z, axis=-1, kind='stable')[:, :k]
  zs = np.take_along_axis(z, order, axis=-1)
  ps = OS.softmax(zs)
  cs = np.cumsum(ps, axis=-1, dtype=np.float32)
  gap = np.abs((cs - ps) - np.float32(top_p)).min(axis=-1)
  keep = ~((cs - ps) > np.float32(top_p))
  noisy = np.where(keep, zs + prng.gumbel(key, zs.shape), -np.inf)
  srt = np.sort(noisy, axis=-1)
  lead = srt[:, -1] - srt[:, -2] if k > 1 else np.full(len(z), np.inf)
  return (gap > 8e-6) & ((lead > 1e-4) | ~np.isfinite(srt[:, -2])), keep.sum(axis=-1)


@pytest.mark.parametrize('M,D,V,temp,top_p,top_k,sharp', [
    (4, 256, 1024, 0.9, 0.9, None, 1.0), (64, 128, 4096, 1.0, 0.5, None, 4.0), (33, 256, 2080, 0.7, 1.0, 50, 1.0),
    (5, 128, 2048, 1.0, 0.8, 100, 2.0), (128, 64, 8192, 1.0, 0.95, None, 1.0), (3, 128, 1024, 1.3, 0.3, 7, 8.0)])
def test_head_nucleus_matches_oracle(M, D, V, temp, top_p, top_k, sharp):
  x, w = _head_inputs(M, D, V, V + M)
  w = bf16_round(w * sharp)
  w[7], w[300] = w[3], w[3]  # equal logits: candidates tie, lower index ranks first
  seed_key = prng.prng_key(77)
  step = 4
  _, _, _, logits = _run_head(x, w, 1, temp, seed_key, step)
  tok, lp, _ = _run_nucleus(x, w, temp, top_p, top_k, seed_key, step)
  key = prng.fold_in(seed_key, step)
  want_tok, want_lp = OS.sample_top_p(logits, key, temp, top_p, top_k)
  z = (logits / np.float32(temp)).astype(np.float32)
  clear, nkeep = _nucleus_clear_rows(z, key, top_p, top_k)
  assert clear.mean() > 0.6
  np.testing.assert_array_equal(tok[clear, step + 1], want_tok[clear])
  np.testing.assert_allclose(lp[clear, step + 1], want_lp[clear], atol=3e-5)
  # every row: the token is a member of the oracle's nucleus (or sits exactly at the cut)
  full_lp = OS.log_softmax(z)
  np.testing.assert_allclose(lp[:, step + 1], full_lp[np.arange(M), tok[:, step + 1]], atol=3e-5)
  for b in range(M):
    if clear[b]:
      members = OS.nucleus_members(z[b], top_p)
      if top_k:
        members &= set(np.argsort(-z[b], kind='stable')[:top_k].tolist())
      assert int(tok[b, step + 1]) in members
  assert np.all(tok[:, :step + 1] == -5) and np.all(tok[:, step + 2:] == -5)


def test_head_nucleus_limits():
  x, w = _head_inputs(16, 128, 1024, 3)
  key = prng.prng_key(5)
  _, _, _, logits = _run_head(x, w, 1, 1.0, key, 2)
  # top_p -> 0 keeps only the best candidate: the draw is the argmax
  tok, lp, _ = _run_nucleus(x, w, 1.0, 0.0, None, key, 2)
  np.testing.assert_array_equal(tok[:, 3], np.argmax(logits, axis=-1))
  # top_k = 1 likewise
  tok1, _, _ = _run_nucleus(x, w, 1.0, 1.0, 1, key, 2)
  np.testing.assert_array_equal(tok1[:, 3], np.argmax(logits, axis=-1))
  # forbidden ids are never drawn and set no eos flag; eos flag follows the token
  banned = tuple(int(t) for t in np.argsort(-logits[0])[:40])
  tokf, lpf, done = _run_nucleus(x, w, 1.0, 0.9, None, key, 2, forbidden=banned, eos=(int(tok[0, 3]),))
  assert not np.isin(tokf[:, 3], banned).any() and np.isfinite(lpf[:, 3]).all()
  np.testing.assert_array_equal(done, (tokf[:, 3] == tok[0, 3]).astype(np.uint8))


def test_head_nucleus_distribution_chi2():
  # one sharp row repeated: empirical frequencies follow softmax(z) renormalised over the nucleus
  M, D, V, top_p = 128, 128, 1024, 0.9
  x, w = _head_inputs(1, D, V, 77)
  w *= 5
  x = np.repeat(x, M, axis=0)
  counts = np.zeros(V)
  _, _, _, logits = _run_head(x, w, 1, 1.0, prng.prng_key(5), 0)
  for s in range(16):
    tok, _, _ = _run_nucleus(x, w, 1.0, top_p, None, prng.prng_key(5), s)
    counts += np.bincount(tok[:, s + 1], minlength=V)
  members = sorted(OS.nucleus_members(logits[0], top_p))
  assert counts.sum() == counts[members].sum()
  pr = OS.softmax(logits[:1])[0].astype(np.float64)
  pr = pr[members] / pr[members].sum()
  assert len(members) > 7
  top = np.argsort(-pr)[:6]
  n = counts.sum()
  obs = np.append(counts[members][top], n - counts[members][top].sum())
  exp = np.append(pr[top], 1 - pr[top].sum()) * n
  assert ((obs - exp) ** 2 / exp).sum() < 24.1  # 6 dof, p = 0.0005


def test_head_sampling_distribution_chi2():
  T = G.Keep()
  # one sharp row repeated: empirical frequencies follow softmax(z)
  M, D, V = 128, 128, 1024
  x, w = _head_inputs(1, D, V, 77)
  w *= 8
  x = np.repeat(x, M, axis=0)
  counts = np.zeros(V)
  for s in range(16):
    tok, _, _, logits = _run_head(x, w, 1, 1.0, prng.prng_key(5), s)
    counts += np.bincount(tok[:, s + 1], minlength=V)
  pr = OS.softmax(logits[:1])[0].astype(np.float64)
  top = np.argsort(-pr)[:8]
  n = counts.sum()
  obs = np.append(counts[top], n - counts[top].sum())
  exp = np.append(pr[top], 1 - pr[top].sum()) * n
  assert ((obs - exp) ** 2 / exp).sum() < 27.9  # 8 dof, p = 0.0005


# ---- routed experts (Qwen3 MoE) ---------------------------------------------------------------

@pytest.mark.parametrize('B,D,E,k', [(8, 256, 16, 4), (32, 512, 128, 8), (3, 256, 8, 1), (32, 2048, 128, 8),
                                     (12, 2304, 160, 16), (5, 128, 32, 32)])
def test_moe_route_matches_oracle(B, D, E, k):
  T = G.Keep()
  rng = np.random.default_rng(B + E)
  x = bf16_round(rng.standard_normal((B, D)).astype(np.float32))
  rw = bf16_round(rng.standard_normal((D, E)).astype(np.float32) * 0.2)
  idx = torch.full((B, k), -1, dtype=torch.int32, device=G.DEV)
  wt = torch.zeros(B, k, dtype=torch.float32, device=G.DEV)
  G.call('tmx_moe_route', S(), T.bf(x), T.bf(rw), B, D, E, k, G.p(idx), G.p(wt))
  G.sync()
  want_w, want_idx = L.moe_route(x, rw, k)
  # expert sets are compared where the k-th / (k+1)-th score margin is clear of bf16 rounding
  scores = np.sort(bf16_round(x @ rw), axis=-1)[:, ::-1]
  clear = np.ones(B, bool) if k == E else (scores[:, k - 1] - scores[:, k]) > 2 * G.ulp_bf16(scores[:, k - 1])
  ordered = np.all(np.diff(scores[:, :k], axis=-1) < -2 * G.ulp_bf16(scores[:, :1]), axis=-1) if k > 1 else clear
  assert clear.mean() > 0.5
  got_idx, got_w = idx.cpu().numpy(), wt.cpu().numpy()
  for b in range(B):
    if clear[b]:
      assert set(got_idx[b]) == set(want_idx[b])
    if clear[b] and ordered[b]:
      np.testing.assert_array_equal(got_idx[b], want_idx[b])
      np.testing.assert_allclose(got_w[b], want_w[b], atol=2 * G.ulp_bf16(want_w[b]).max())
  np.testing.assert_allclose(got_w.sum(-1), 1.0, atol=0.02)
  assert (got_idx >= 0).all() and (got_idx < E).all()
  assert all(len(set(r)) == k for r in got_idx)


@pytest.mark.parametrize('B,D,F,E,k,group', [
    (8, 256, 256, 16, 4, 64), (32, 512, 256, 32, 8, 128), (40, 256, 512, 4, 2, 64),
    # more than 1024 routed pairs (many-rows passes): the block kernel, hundreds of rows per expert
    (600, 256, 256, 6, 2, 64), (300, 512, 256, 9, 4, 128), (300, 256, 256, 40, 4, 64)])
def test_moe_experts_match_oracle(B, D, F, E, k, group):
  T = G.Keep()
  rng = np.random.default_rng(B * 3 + E)
  x = bf16_round(rng.standard_normal((B, D)).astype(np.float32))
  gate = bf16_round(rng.standard_normal((E, D, F)).astype(np.float32) * 0.05)
  up = bf16_round(rng.standard_normal((E, D, F)).astype(np.float32) * 0.05)
  down = bf16_round(rng.standard_normal((E, F, D)).astype(np.float32) * 0.05)
  # routing table: every token picks k distinct experts; expert E - 1 is never used; when the
  # batch allows it one expert receives more than 32 rows (second row chunk)
  idx = np.stack([rng.permutation(E - 1)[:k] for _ in range(B)]).astype(np.int32)
  if B > 32:
    idx[:, 0] = 0
  gu = np.stack([gate, up], axis=2).transpose(1, 0, 2, 3).reshape(D, E * 2 * F)
  dn = down.transpose(1, 0, 2).reshape(F, E * D)
  pgu, pdn = _packed(gu, group), _packed(dn, group)
  P = B * k
  idx_t = T.i32(idx.reshape(-1))
  act = torch.full((P, F), 7.0, dtype=torch.bfloat16, device=G.DEV)
  y = torch.full((P, D), 7.0, dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_moe_experts', S(), T.bf(x), D, G.p(pgu.qweight), G.p(pgu.scales), idx_t, P, k, E, D, 2 * F,
         group, 0, G.p(act), F)
  G.call('tmx_moe_experts', S(), G.p(act), F, G.p(pdn.qweight), G.p(pdn.scales), idx_t, P, k, E, F, D,
         group, 1, G.p(y), D)
  G.sync()
  got_act, got_y = G.host(act), G.host(y)
  lin = lambda w: L.Linear(q=int4.quantize(w, group)[0], scale=int4.quantize(w, group)[1], group=group)
  for e in range(E - 1):
    rows = np.nonzero(idx.reshape(-1) == e)[0]
    if rows.size == 0:
      continue
    xe = x[rows // k]
    g, u = lin(gate[e])(xe, BF16), lin(up[e])(xe, BF16)
    want_act = bf16_round(L.silu(g, BF16) * u)
    # a one-ulp flip of g or u (f32 accumulation order) moves the product by about one ulp of it
    few = 2 if rows.size > 128 else 0  # hundreds of thousands of outputs: sums that cancel to far below their terms
    G.assert_bf16_close(got_act[rows], want_act, ulps=2.0, extra=1e-6, min_exact=0.98, what=f'act e{e}', stragglers=few)
    ld = lin(down[e])
    want_y = ld(got_act[rows], BF16)  # the kernel's own activations: isolates the down product
    # sums that cancel to far below their terms carry the f32 accumulation error itself (eps32 x sum |x w|)
    acc_err = 2.0 ** -23 * (np.abs(got_act[rows]) @ np.abs(ld.weight()))
    G.assert_bf16_close(got_y[rows], want_y, ulps=1.0, extra=acc_err, min_exact=0.995, what=f'down e{e}', stragglers=few)
  assert not np.isin(idx, E - 1).any()


# ---- LoRA delta finished by the projection's own launch ----------------------------------------------

@pytest.mark.parametrize('M,K,widths,group,r,nsplit', [
    (64, 14336, (4096,), 64, 16, 7),        # the 8B down projection
    (8, 8192, (2048,), 64, 8, 4),           # rank 8: half of the 16-wide rank step is masked
    (32, 8192, (4096,), 128, 12, 2),        # rank not a multiple of 8: the element-wise fragment path
    (128, 12288, (4096,), 128, 32, 4),      # 128 rows, two rank steps
    (16, 8192, (2048, 512, 512), 64, 16, 2),  # three fused matrices (q | k | v): t columns by segment
])
def test_projection_writes_the_lora_delta(M, K, widths, group, r, nsplit):
  """tmx_qlora_linear_planes_delta: the y planes add up to x . W as before, and delta equals
  bf16(bf16(t . B) * s) with t = bf16(x . A) per fused matrix (tunix's qwix-wrapped Einsum, tunix/models/llama3/model.py:216-218:
  (x . A) . B * alpha / rank), twice in a row on one workspace (its counters must be back at zero)."""
  T = G.Keep()
  lib = _lib.lib()
  rng = np.random.default_rng(M + K + r)
  N = sum(widths)
  x = bf16_round(rng.standard_normal((M, K)).astype(np.float32))
  ws = [bf16_round(rng.standard_normal((K, n)).astype(np.float32) * 0.02) for n in widths]
  As = [bf16_round(rng.standard_normal((K, r)).astype(np.float32) * 0.05) for _ in widths]
  Bs = [bf16_round(rng.standard_normal((r, n)).astype(np.float32) * 0.05) for n in widths]
  ls = 2.0
  pl = quant.PackedLinear.from_dense([torch.from_numpy(w) for w in ws], group, G.DEV,
                                     [(torch.from_numpy(a), torch.from_numpy(b)) for a, b in zip(As, Bs)], ls)
  nb = lib.tmx_qlora_linear_delta_workspace_bytes(M, K, N, r, pl.r_pad, nsplit)
  assert nb > 0
  nls = lib.tmx_qlora_linear_num_lora_splits(K, N)
  wsb = torch.empty(nb, dtype=torch.uint8, device=G.DEV)
  yp = torch.full((nsplit, M, N), float('nan'), dtype=torch.float32, device=G.DEV)
  tp = torch.full((nls, M, 128), float('nan'), dtype=torch.float32, device=G.DEV)
  ends = list(np.cumsum(widths))
  e0, e1 = (ends[0], ends[1]) if len(widths) == 3 else (N, N)
  outs = []
  for _ in range(2):
    d = torch.full((M, N), float('nan'), dtype=torch.bfloat16, device=G.DEV)
    G.call('tmx_qlora_linear_planes_delta', S(), T.bf(x), G.p(pl.qweight), G.p(pl.scales), G.p(pl.lora_a_t), G.p(pl.lora_b),
           G.p(yp), G.p(tp), G.p(d), G.p(wsb), M, K, N, group, r, pl.r_pad, ls, int(e0), int(e1), nsplit)
    G.sync()
    outs.append(G.host(d))
  np.testing.assert_array_equal(outs[0], outs[1])
  assert int(wsb[:16].view(torch.int32).abs().sum().item()) == 0
  assert lib.tmx_handover_status(S(), G.p(wsb)) == 0   # no LoRA block's wait ran out
  got = outs[1]
  want = np.concatenate([bf16_round(bf16_round(bf16_round(x @ a) @ b) * ls) for a, b in zip(As, Bs)], axis=1)
  # a last-bit flip of a t element (f32 summation order of x . A) moves the product by ulp(t) |B|
  tt = [bf16_round(x @ a) for a in As]
  slack = np.concatenate([(G.ulp_bf16(t) @ np.abs(b)) * ls for t, b in zip(tt, Bs)], axis=1)
  G.assert_bf16_close(got, want, ulps=1.0, extra=slack + 2.0 ** -22 * np.abs(want), min_exact=0.9, what=f'delta {M}x{K}x{N} r{r}')
  # the planes still add up to the base product
  qs = [int4.quantize(w, group) for w in ws]
  base = np.concatenate([x @ L.Linear(q=q, scale=sc, group=group).weight() for q, sc in qs], axis=1)
  ysum = yp.sum(0).cpu().numpy()
  np.testing.assert_allclose(ysum, base, rtol=2e-3, atol=2e-3 * np.abs(base).max())


def test_projection_delta_only_where_it_hides():
  lib = _lib.lib()
  assert lib.tmx_qlora_linear_delta_workspace_bytes(64, 14336, 4096, 16, 32, 7) > 0
  assert lib.tmx_qlora_linear_delta_workspace_bytes(64, 4096, 4096, 16, 32, 4) == 0   # 4-step slices: the stage would stick out
  assert lib.tmx_qlora_linear_delta_workspace_bytes(64, 4096, 28672, 16, 32, 1) == 0  # too many column tiles per LoRA wave
  assert lib.tmx_qlora_linear_delta_workspace_bytes(256, 14336, 4096, 16, 32, 7) == 0  # more than 128 rows


# ---- single-sequence regime: norm | projection | LoRA | residual / SwiGLU in one launch -----------

@pytest.mark.parametrize('M,K,N,group,r,mode', [
    (1, 2048, 3072, 64, 16, 'norm'), (1, 2048, 2048, 64, 16, 'residual'), (1, 2048, 1024, 64, 16, 'swiglu'),
    (1, 8192, 2048, 64, 16, 'residual'), (4, 256, 96, 64, 8, 'norm'), (3, 512, 256, 128, 0, 'plain'),
    (2, 1024, 256, 64, 32, 'residual'), (4, 512, 128, 64, 4, 'swiglu'), (1, 320, 64, 64, 0, 'swiglu'),
    (1, 2048, 3072, 64, 0, 'norm_qwen'), (1, 2048, 16384, 64, 16, 'swiglu'), (4, 2048, 16384, 64, 16, 'swiglu')])
def test_small_linear_matches_oracle(M, K, N, group, r, mode):
  T = G.Keep()
  rng = np.random.default_rng(M * 13 + K + N)
  w = bf16_round(rng.standard_normal((K, N)).astype(np.float32) * 0.02)
  x = bf16_round(rng.standard_normal((M, K)).astype(np.float32))
  res = bf16_round(rng.standard_normal((M, N)).astype(np.float32))
  nw = bf16_round(1.0 + 0.1 * rng.standard_normal(K).astype(np.float32))
  swiglu = mode == 'swiglu'
  a = b = None
  loras = None
  if r:
    a = bf16_round(rng.standard_normal((K, r)).astype(np.float32) * 0.02)
    b = bf16_round(rng.standard_normal((r, N)).astype(np.float32) * 0.02)
  if swiglu:
    F = N // 2
    ws = [w[:, :F], w[:, F:]]
    # gate and up carry their own A (the same values here) and their own B columns
    pl = quant.PackedLinear.from_dense([torch.from_numpy(np.ascontiguousarray(v)) for v in ws], group, G.DEV,
                                       [(torch.from_numpy(a), torch.from_numpy(np.ascontiguousarray(b[:, :F]))),
                                        (torch.from_numpy(a), torch.from_numpy(np.ascontiguousarray(b[:, F:])))] if r else None, 2.0)
  else:
    pl = _packed(w, group, (a, b) if r else None, 2.0)
  qo, so = int4.quantize(w, group)
  lin = L.Linear(q=qo, scale=so, group=group, a=a, b=b, lora_scale=2.0)
  family = 1 if mode == 'norm_qwen' else 0
  use_norm = mode in ('norm', 'norm_qwen', 'swiglu')
  xin = x
  if use_norm:
    xin = (L.rmsnorm_qwen3 if family else L.rmsnorm_llama3)(x, nw, 1e-5, BF16)
  out = lin(xin, BF16)
  base = bf16_round(xin @ lin.weight())
  if swiglu:
    F = N // 2
    want = bf16_round(L.silu(out[:, :F], BF16) * out[:, F:])
  elif mode == 'residual':
    want = bf16_round(out + res)
  else:
    want = out
  y = torch.full(want.shape, float('nan'), dtype=torch.bfloat16, device=G.DEV)
  G.call('tmx_small_linear', S(), T.bf(x), T.bf(nw) if use_norm else None, 1e-5, family, G.p(pl.qweight), G.p(pl.scales),
         G.p(pl.lora_a_t), G.p(pl.lora_b), T.bf(res) if mode == 'residual' else None, G.p(y), M, K, N, group, r,
         pl.r_pad, 2.0, 1 if swiglu else 0)
  G.sync()
  got = G.host(y)
  if swiglu:
    # a last-bit flip of gate or up (f32 summation order) moves the product by about an ulp of it
    # (gate and up both flipping on one element is rare: a couple of elements in 32768 may reach three bounds)
    G.assert_bf16_close(got, want, ulps=2.0, extra=1e-6 + 2.0 * G.ulp_bf16(want), min_exact=0.97, what=f'small swiglu {K}x{N}',
                        stragglers=2 if want.size > 8192 else 0)
  else:
    extra = (G.ulp_bf16(base) + G.ulp_bf16(out)) if (r or mode == 'residual') else 0.0
    if r:
      extra = extra + 2.0 * G.ulp_bf16(out - base)
    extra = extra + 2.0 ** -23 * (np.abs(xin) @ np.abs(lin.weight()))
    G.assert_bf16_close(got, want, ulps=1.0, extra=extra, min_exact=0.99, what=f'small {mode} {M}x{K}x{N}')


def test_small_linear_rejects_what_it_cannot_take():
  lib = _lib.lib()
  one = torch.zeros(64, dtype=torch.uint8, device=G.DEV)
  p = G.p(one)
  assert lib.tmx_small_linear(S(), p, None, 1e-5, 0, p, p, None, None, None, p, 5, 256, 64, 64, 0, 0, 0.0, 0) == -2   # 5 rows
  assert lib.tmx_small_linear(S(), p, p, 1e-5, 0, p, p, None, None, None, p, 4, 8192, 64, 64, 0, 0, 0.0, 0) == -2  # M K too large for the norm
  assert lib.tmx_small_linear(S(), p, None, 1e-5, 0, p, p, None, None, None, p, 1, 256, 64, 64, 0, 0, 0.0, 1) == -4  # SwiGLU needs the norm prologue
  assert lib.tmx_small_linear(S(), None, None, 1e-5, 0, p, p, None, None, None, p, 1, 256, 64, 64, 0, 0, 0.0, 0) == -1
