"""Child process of test_host_abi.py::test_host_code_under_address_and_undefined_sanitizers.

Runs the host-side code of the C ABI that needs no GPU (argument checks, K-slice and LoRA-slice
planning, workspace carving, shape gates of every launch form) over the shapes of the five benchmark
configurations, inside a library whose host code was compiled with AddressSanitizer and
UndefinedBehaviorSanitizer (tunix_amd.build.build(host_sanitizers=True)); TMX_LIB selects it and the
parent preloads the sanitizer runtime.  A sanitizer report aborts the process.  Nothing is launched:
every call either computes a size or fails its argument checks before the first launch.
"""
import ctypes
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from tunix_amd import _lib
from tunix_amd.model import DecodeState, LayerDesc, ModelDesc, QLinearDesc

FAKE = 0x1000  # a non-null "device pointer": never dereferenced on the host

# family, layers, vocab, D, F, heads, kv heads, head_dim, experts, experts per token, group, rank, LoRA on the MLP
CONFIGS = {
    'toy': (0, 2, 1024, 256, 1024, 4, 4, 64, 0, 0, 64, 8, False),
    'llama3.2-1b': (0, 16, 128256, 2048, 8192, 32, 8, 64, 0, 0, 64, 16, True),
    'llama3.1-8b': (0, 32, 128256, 4096, 14336, 32, 8, 128, 0, 0, 64, 16, True),
    'qwen3-8b': (1, 36, 151936, 4096, 12288, 32, 8, 128, 0, 0, 128, 32, True),
    'qwen3-30b-a3b': (1, 48, 151936, 2048, 768, 32, 4, 128, 128, 8, 64, 8, False),
}


def qdesc(k, n, group, rank, fused):
  d = QLinearDesc()
  d.qweight, d.scales = FAKE, FAKE
  if rank:
    d.lora_a_t, d.lora_b = FAKE, FAKE
    d.rank, d.r_pad, d.lora_scale = rank, (rank * fused + 31) // 32 * 32, 2.0
  d.K, d.N, d.G = k, n, group
  return d


def model_desc(family, layers, vocab, dm, f, n, kh, h, experts, per_tok, group, rank, mlp_lora):
  arr = (LayerDesc * layers)()
  for i in range(layers):
    arr[i].norm1_w = arr[i].norm2_w = FAKE
    if family == 1:
      arr[i].q_norm_w = arr[i].k_norm_w = FAKE
    arr[i].qkv = qdesc(dm, (n + 2 * kh) * h, group, rank, 3)
    arr[i].o = qdesc(n * h, dm, group, rank, 1)
    arr[i].gate_up = qdesc(dm, 2 * f, group, rank if mlp_lora else 0, 2)
    arr[i].down = qdesc(f, dm, group, rank if mlp_lora else 0, 1)
    if experts:
      arr[i].router_w = FAKE
  d = ModelDesc()
  d.family, d.num_layers, d.vocab_size, d.embed_dim, d.hidden_dim = family, layers, vocab, dm, f
  d.num_heads, d.num_kv_heads, d.head_dim, d.num_experts, d.experts_per_tok = n, kh, h, experts, per_tok
  d.rope_theta, d.norm_eps = 1e6, 1e-6
  d.embed = d.final_norm_w = d.head = FAKE
  d.layers = ctypes.cast(arr, ctypes.POINTER(LayerDesc))
  return d, arr


def main():
  lib = _lib.lib()
  assert os.path.basename(_lib.LIB_PATH) == 'libtmx_hostsan.so', _lib.LIB_PATH
  assert lib.tmx_abi_version() >= 7
  sizes = []
  for name, c in CONFIGS.items():
    d, keep = model_desc(*c)
    for batch in (1, 3, 4, 5, 32, 33, 64, 65, 128, 129, 512, 4096):
      for cache in (64, 768, 1536):
        nb = lib.tmx_decode_workspace_bytes(ctypes.byref(d), batch, cache)
        assert nb > 0
        sizes.append(nb)
        st = DecodeState()
        st.batch, st.buf_len, st.cache_size = batch, cache, cache
        st.token_buffer = st.positions = st.input_mask = st.done = st.step = st.kv_cache = st.workspace = FAKE
        # every argument is checked and the whole launch plan is made before the first launch: a workspace one
        # byte short fails after the planning code has run (nothing is launched)
        st.workspace_bytes = nb - 1
        rc = lib.tmx_decode_steps(ctypes.byref(d), ctypes.byref(st), None, 1, 1)
        assert rc == -2, (name, batch, cache, rc)
        st.workspace = None
        assert lib.tmx_decode_steps(ctypes.byref(d), ctypes.byref(st), None, 1, 1) == -1
    n, kh, h, dm, f, group, rank = c[5], c[6], c[7], c[3], c[4], c[10], c[11]
    for m in (1, 4, 32, 64, 128, 1024):
      for k, nn in ((dm, (n + 2 * kh) * h), (n * h, dm), (dm, 2 * f), (f, dm)):
        ns = lib.tmx_qlora_linear_num_splits(m, k, nn)
        assert 1 <= ns <= 16
        assert 1 <= lib.tmx_qlora_linear_num_lora_splits(k, nn) <= 32
        assert lib.tmx_qlora_linear_workspace_bytes(m, k, nn) > 0
        lib.tmx_qlora_linear_delta_workspace_bytes(m, k, nn, rank, (rank + 31) // 32 * 32, ns)
        lib.tmx_qlora_gate_up_swiglu_handover_bytes(m, k, nn // 2, rank)
        # null operands: refused by the argument checks of every launch form
        assert lib.tmx_qlora_linear_planes(None, None, None, None, None, None, None, m, k, nn, group, 0, ns) == -1
        assert lib.tmx_qlora_linear(None, FAKE, FAKE, FAKE, None, None, None, None, None, m, k, nn, group, 0, 0, 0.0) == -1
    for b in (1, 64, 128):
      lib.tmx_gqa_decode_workspace_bytes(b, n, kh, h, 1536)
      lib.tmx_head_sample_workspace_bytes(b, c[2])
      lib.tmx_nucleus_workspace_bytes(b, c[2])
  assert lib.tmx_int4_dequant(None, None, None, None, 64, 32, 64) == -1
  assert lib.tmx_int4_dequant(None, FAKE, FAKE, FAKE, 65, 32, 64) == -2
  assert lib.tmx_qlora_linear_planes(None, FAKE, FAKE, FAKE, None, FAKE, None, 4, 100, 32, 64, 0, 1) == -2
  assert lib.tmx_qlora_linear_noalloc(None, FAKE, FAKE, FAKE, None, None, None, FAKE, 4096, 14336, 4096, 64, 0, 0, 0.0) == -5
  assert lib.tmx_handover_status(None, None) == -1
  assert lib.tmx_decode_steps(None, None, None, 1, 1) == -1
  assert lib.tmx_decode_status(None, None, None) == -1
  for code in range(-8, 2):
    assert len(lib.tmx_status_string(code)) > 1
  print(f'host sanitizer run ok: {len(sizes)} workspace plans')


if __name__ == '__main__':
  main()
