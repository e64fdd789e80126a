"""ctypes binding of libtmx.so (the C ABI declared in include/tmx.h).

There is no CPU fallback: if the library is missing every operator raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get('TMX_LIB', os.path.join(_HERE, 'libtmx.so'))

_lib = None
ABI_VERSION = 7  # TMX_ABI_VERSION of include/tmx.h

vp, ci, cf, cu32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_uint32

# name -> argtypes (restype is int unless noted)
SIGNATURES = {
    'tmx_abi_version': [],
    'tmx_int4_dequant': [vp, vp, vp, vp, ci, ci, ci],
    'tmx_qlora_linear': [vp, vp, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, cf],
    'tmx_qlora_linear_noalloc': [vp, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, cf],
    'tmx_qlora_linear_planes_delta': [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, cf, ci, ci, ci],
    'tmx_small_linear': [vp, vp, vp, cf, ci, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, cf, ci],
    'tmx_qlora_linear_num_splits': [ci, ci, ci],
    'tmx_qlora_linear_num_lora_splits': [ci, ci],
    'tmx_qlora_linear_planes': [vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci],
    'tmx_rmsnorm': [vp, vp, vp, vp, ci, ci, cf, ci],
    'tmx_lora_residual_rmsnorm': [vp, vp, vp, ci, vp, ci, ci, vp, ci, cf, vp, vp, vp, vp, ci, ci, cf, ci],
    'tmx_rope_kv_write': [vp, vp, vp, ci, vp, ci, ci, vp, ci, cf, vp, vp, vp, vp, ci, vp, vp, vp, ci, ci,
                          ci, ci, ci, cf, cf, ci],
    'tmx_swiglu': [vp, vp, vp, ci, vp, ci, ci, vp, ci, cf, vp, ci, ci],
    'tmx_qlora_gate_up_swiglu': [vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, cf],
    'tmx_qlora_gate_up_swiglu_handover': [vp, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, cf],
    'tmx_handover_status': [vp, vp],
    'tmx_gqa_decode_attention': [vp, vp, vp, vp, vp, vp, ci, vp, vp, ci, ci, ci, ci, ci],
    'tmx_gqa_decode_attention_shared': [vp, vp, vp, vp, vp, vp, ci, vp, vp, ci, ci, ci, ci, ci, ci, ci],
    'tmx_gqa_attention_rows': [vp, vp, vp, vp, vp, vp, ci, vp, vp, ci, ci, ci, ci, ci, ci],
    'tmx_head_sample': [vp, vp, vp, ci, ci, ci, ci, cf, cu32, cu32, vp, vp, ci, vp, ci, vp, vp, vp, ci,
                        vp, vp],
    'tmx_head_sample_tiles': [vp, vp, vp, ci, ci, ci, ci, cf, cu32, cu32, vp, vp, ci, vp, ci, vp, vp, vp, ci,
                              vp, vp],
    'tmx_head_tiles_pack': [vp, vp, vp, ci, ci],
    'tmx_head_sample_nucleus': [vp, vp, vp, ci, ci, ci, cf, cf, ci, cu32, cu32, vp, vp, ci, vp, ci, vp, vp,
                                vp, ci, vp, vp, ctypes.c_size_t],
    'tmx_moe_route': [vp, vp, vp, ci, ci, ci, ci, vp, vp],
    'tmx_moe_experts': [vp, vp, ci, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, vp, ci],
    'tmx_decode_steps': [vp, vp, vp, ci, ci],
    'tmx_decode_steps_graph': [vp, vp, vp, ci, ci],
    'tmx_decode_steps_profiled': [vp, vp, vp, ci, ci, vp, vp],
    'tmx_decode_status': [vp, vp, vp],
}
# entry points that return size_t
SIZE_FUNCS = {
    'tmx_gqa_decode_workspace_bytes': [ci, ci, ci, ci, ci],
    'tmx_gqa_decode_shared_workspace_bytes': [ci, ci, ci, ci, ci],
    'tmx_qlora_linear_workspace_bytes': [ci, ci, ci],
    'tmx_qlora_linear_noalloc_max_bytes': [],
    'tmx_head_sample_workspace_bytes': [ci, ci],
    'tmx_nucleus_workspace_bytes': [ci, ci],
    'tmx_qlora_linear_delta_workspace_bytes': [ci, ci, ci, ci, ci, ci],
    'tmx_decode_workspace_bytes': [vp, ci, ci],
    'tmx_qlora_gate_up_swiglu_handover_bytes': [ci, ci, ci, ci],
}


class TmxError(RuntimeError):
  pass


def lib():
  """Loads the library once; raises if it has not been built."""
  global _lib
  if _lib is None:
    if not os.path.exists(LIB_PATH):
      raise TmxError(
          f'{LIB_PATH} is missing: build it with `python -m tunix_amd.build` '
          '(there is no CPU fallback for the decode path).')
    l = ctypes.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
      fn = getattr(l, name)
      fn.argtypes = args
      fn.restype = ci
    for name, args in SIZE_FUNCS.items():
      fn = getattr(l, name)
      fn.argtypes = args
      fn.restype = ctypes.c_size_t
    l.tmx_status_string.argtypes = [ci]
    l.tmx_status_string.restype = ctypes.c_char_p
    # the ctypes structs of model.py mirror the header of ABI_VERSION: a library built from another header
    # would read them with the wrong layout
    if l.tmx_abi_version() != ABI_VERSION:
      raise TmxError(f'{LIB_PATH} has ABI version {l.tmx_abi_version()}, this package expects {ABI_VERSION}: '
                     'rebuild it with `python -m tunix_amd.build`.')
    _lib = l
  return _lib


def check(status, what):
  if status != 0:
    raise TmxError(f'{what}: {lib().tmx_status_string(status).decode()} (status {status})')


def ptr(t):
  """Device pointer of a torch tensor (None -> NULL)."""
  return None if t is None else t.data_ptr()


def stream():
  import torch
  return torch.cuda.current_stream().cuda_stream
