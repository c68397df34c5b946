"""ctypes binding of libmoe_mi355x.so (declared in include/moe_mi355x.h).

There is no fallback: if the library has not been built, or a call reports an error, a
RuntimeError is raised.  torch is used only for device memory and the current stream.
"""

from __future__ import annotations

import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
# MOE_MI355X_LIB points the loader at another build of the same library (a tuning variant, an installed copy)
LIB_PATH = os.environ.get("MOE_MI355X_LIB") or os.path.join(_PKG, "lib", "libmoe_mi355x.so")

# enums of include/moe_mi355x.h
MOE_BF16, MOE_INT8, MOE_FP8_E4M3, MOE_INT4, MOE_F32, MOE_MXFP4, MOE_FP8_E5M2 = 0, 1, 2, 3, 4, 5, 6
MOE_ROUTE_SOFTMAX_TOPK, MOE_ROUTE_DEEPSEEK, MOE_ROUTE_TOPK_RAW, MOE_ROUTE_SOFTMAX_ALL = 0, 1, 2, 3
ROUTE_BY_NAME = {"softmax_topk": 0, "deepseek": 1, "topk_raw": 2, "softmax_all": 3}
MOE_ACT_NONE, MOE_ACT_SILU, MOE_ACT_SWIGLUOAI, MOE_ACT_SILU_CLIP = 0, 1, 2, 3
MOE_GMM_KEEP_OTHER_ROWS = 1
MOE_GMM_RHS_KN = 2
MOE_GMM_RHS_SCALE_KMAJOR = 4
MOE_GMM_RHS_SCALE_SHARED = 8
MOE_GMM_SAME_GROUPS = 16
MOE_SCALE_PER_TENSOR = -1
GMM_KERNEL_BY_NAME = {None: 0, "auto": 0, "stream": 1, "tiled": 2, "big": 3, "dl64": 4, "stream_nosplit": 5}
MOE_QUANT_RINT_DIV, MOE_QUANT_V2 = 0, 1
QUANT_RULE_BY_NAME = {"rint_div": MOE_QUANT_RINT_DIV, "v2": MOE_QUANT_V2}

ACT_BY_NAME = {None: MOE_ACT_NONE, "silu": MOE_ACT_SILU, "swigluoai": MOE_ACT_SWIGLUOAI, "silu_clip": MOE_ACT_SILU_CLIP}

c_void_p, c_int, c_float, c_size_t = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t


class GmmArgs(ctypes.Structure):
  """moe_gmm_args."""

  _fields_ = [
      ("struct_size", c_size_t),
      ("lhs", c_void_p),
      ("lhs_scale", c_void_p),
      ("rhs", c_void_p),
      ("rhs_scale", c_void_p),
      ("rhs_up", c_void_p),
      ("rhs_up_scale", c_void_p),
      ("group_sizes", c_void_p),
      ("out", c_void_p),
      ("workspace", c_void_p),
      ("workspace_bytes", c_size_t),
      ("M", ctypes.c_int32),
      ("K", ctypes.c_int32),
      ("N", ctypes.c_int32),
      ("num_groups_total", ctypes.c_int32),
      ("num_groups_local", ctypes.c_int32),
      ("group_offset", ctypes.c_int32),
      ("lhs_dtype", ctypes.c_int32),
      ("rhs_dtype", ctypes.c_int32),
      ("lhs_scale_block_k", ctypes.c_int32),
      ("rhs_scale_block_n", ctypes.c_int32),
      ("rhs_scale_block_k", ctypes.c_int32),
      ("act", ctypes.c_int32),
      ("act_limit", c_float),
      ("out_dtype", ctypes.c_int32),
      ("lhs_row_idx_div", ctypes.c_int32),
      ("lhs_rows", ctypes.c_int32),
      ("reserved", ctypes.c_int32),
      ("rhs_bias", c_void_p),
      ("rhs_up_bias", c_void_p),
      ("partial_sum", c_void_p),
      ("partial_sum_up", c_void_p),
      ("flags", ctypes.c_int32),
      ("pad_", ctypes.c_int32),
      ("lhs_row_idx", c_void_p),
      ("out_row_scale", c_void_p),
      ("group_offset_dev", c_void_p),
  ]


SIGNATURES = {
    "moe_last_error": (ctypes.c_char_p, []),
    "moe_abi_version": (c_int, []),
    "moe_route_topk": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "moe_gate_route_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "moe_gate_route": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float,
                               c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "moe_sort_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "moe_sort_by_expert": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "moe_sort_by_expert_rolled": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "moe_sort_by_expert_mapped": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                          c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "moe_route_sort_mapped": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p,
                                      c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_void_p, c_size_t,
                                      c_void_p]),
    "moe_gather_rows": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                c_void_p]),
    "moe_gmm_workspace_bytes": (c_size_t, [c_int, c_int]),
    "moe_gmm_rhs_kn_supported": (c_int, [c_int, c_int, c_int, c_int]),
    "moe_gmm_lhs_e5m2_supported": (c_int, [c_int, c_int, c_int, c_int]),
    "moe_gmm_fp8_rhs_kn_supported": (c_int, [c_int, c_int, c_int, c_int]),
    "moe_gmm_stream_kernel_takes": (c_int, [c_int, c_int, c_int, c_int, ctypes.c_longlong]),
    "moe_gmm": (c_int, [ctypes.POINTER(GmmArgs), c_void_p]),
    "moe_gmm_tuned": (c_int, [ctypes.POINTER(GmmArgs), c_int, c_int, c_void_p]),
    "moe_gmm_static_ws": (c_int, [ctypes.POINTER(GmmArgs), c_void_p]),
    "moe_gmm_static_ws_capacity": (c_size_t, []),
    "moe_init": (c_int, []),
    "moe_tgmm": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "moe_tgmm_scaled": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "moe_tgmm_fp8_supported": (c_int, [c_int, c_int, c_int, c_int, c_int]),
    "moe_tgmm_fp8": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "moe_transpose_rhs": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "moe_unpermute_combine": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
    "moe_glu_act": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_float, c_void_p, c_void_p]),
    "moe_glu_act_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_float, c_void_p, c_void_p, c_void_p]),
    "moe_bwd_scale_grad": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "moe_tensor_scale": (c_int, [c_void_p, ctypes.c_longlong, c_int, c_float, c_void_p, c_void_p]),
    "moe_sort_by_expert_rolled_dev": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "moe_quantize_rhs": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "moe_add_group_bias": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    "moe_unpermute_combine_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "moe_local_expert_keys_workspace_bytes": (c_size_t, [c_int, c_int]),
    "moe_local_expert_keys": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "moe_ring_ragged_indices": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "moe_all_to_all_params": (c_int, [c_void_p, c_int, c_int, c_int, ctypes.c_longlong, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "moe_local_expert_keys_dev": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "moe_ring_ragged_indices_dev": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "moe_all_to_all_params_dev": (c_int, [c_void_p, c_int, c_void_p, c_int, ctypes.c_longlong, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
}

_lib = None


def load():
  """Loads the shared library once; raises if it has not been built."""
  global _lib
  if _lib is not None:
    return _lib
  if not os.path.exists(LIB_PATH):
    raise RuntimeError(
        f"{LIB_PATH} is missing: build it with `python -m maxtext_amd.build` "
        "(there is no non-HIP fallback for the MoE expert path)"
    )
  lib = ctypes.CDLL(LIB_PATH)
  for name, (res, args) in SIGNATURES.items():
    fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
    fn.restype = res
    fn.argtypes = args
  _lib = lib
  return lib


def check(status: int, what: str):
  if status != 0:
    msg = load().moe_last_error().decode("utf-8", "replace")
    raise RuntimeError(f"{what} failed with status {status}: {msg}")


def ptr(t):
  """Device pointer of a torch tensor (None -> NULL)."""
  return None if t is None else ctypes.c_void_p(t.data_ptr())


def current_stream():
  import torch

  return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
