"""Loads librg_lru.so (the gfx950 HIP kernels behind a C ABI) with ctypes.

There is no CPU or eager-torch fallback: if the library is missing or a kernel
call fails, the caller gets an exception.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "librg_lru.so")
CSRC = os.path.join(_HERE, "csrc")

RG_OK = 0
RG_DTYPE_F32 = 0
RG_DTYPE_BF16 = 1
RG_STEP_STATIC_SCRATCH_BYTES = 8 << 20
ABI_VERSION = 1

_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64
_sz = ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/rg_lru.h declaration by declaration
SIGNATURES = {
    "rg_abi_version": (_i, []),
    "rg_clock_probe": (_i, [_vp, _i, _vp]),
    "rg_prefill_clock_probe": (_i, [_vp]),
    "rg_last_error": (ctypes.c_char_p, []),
    "rg_conv1d_prefill": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i,
                               _i, _vp]),
    "rg_conv1d_step": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "rg_block_diag_linear": (_i, [_vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp]),
    "rg_gates_weight_grads_workspace_bytes": (_sz, [_i64, _i, _i]),
    "rg_gates_weight_grads": (_i, [_vp] * 8 + [_sz, _i64, _i, _i, _i, _vp]),
    "rg_gates_gemm": (_i, [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                           _vp, _i, _i, _i, _i, _i, _vp]),
    "rg_lru_scan_fused": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp,
                               _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "rg_recurrent_prefill": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp,
                                  _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i,
                                  _i, _vp]),
    "rg_recurrent_prefill_split_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "rg_recurrent_prefill_split": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp,
                                        _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                        _sz, _i, _i, _i, _i, _i, _vp]),
    "rg_recurrent_prefill_gelu_mul": (_i, [_vp, _vp, _vp, _i] + [_vp] * 13 +
                                      [_sz, _i, _i, _i, _i, _i, _vp]),
    "rg_recurrent_core_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "rg_recurrent_core": (_i, [_vp, _vp, _vp, _i] + [_vp] * 13 +
                          [_sz, _i, _i, _i, _i, _i, _vp]),
    "rg_linear_scan": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "rg_linear_scan_backward": (_i, [_vp] * 9 + [_i, _i, _i, _i, _vp]),
    "rg_conv1d_backward_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "rg_conv1d_backward": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _vp, _sz, _i, _i,
                                _i, _i, _i, _vp]),
    "rg_attention_prefill": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i,
                                  ctypes.c_float, _i, _vp]),
    "rg_rglru_backward": (_i, [_vp] * 14 + [_i, _i, _i, _i, _vp]),
    "rg_scan_split_workspace_bytes": (_sz, [_i, _i, _i]),
    "rg_lru_scan_fused_split": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i,
                                     _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i,
                                     _i, _vp]),
    "rg_linear_scan_split": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i,
                                  _i, _i, _i, _vp]),
    "rg_recurrent_step_workspace_bytes": (_sz, [_i, _i, _i]),
    "rg_recurrent_step_static": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp,
                                      _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i,
                                      _i, _vp]),
    "rg_gelu_mul": (_i, [_vp, _vp, _vp, ctypes.c_int64, _i, _vp]),
    "rg_gelu_mul_backward": (_i, [_vp] * 5 + [ctypes.c_int64, _i, _vp]),
    "rg_rms_norm": (_i, [_vp, _vp, _vp, ctypes.c_int64, _i, ctypes.c_float, _i,
                         _vp]),
    "rg_linear_packed_bytes": (ctypes.c_size_t, [_i, _i, _i]),
    "rg_linear_pack": (_i, [_vp, _i, _i, _i, _vp, _i, _i, _vp]),
    "rg_linear_rows_workspace_bytes": (ctypes.c_size_t, [_i, _i, _i]),
    "rg_linear_rows": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_size_t, _i,
                            _i, _i, _i, _i, _vp]),
    "rg_rope_pair": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _vp, ctypes.c_int64, _i,
                          _i, _i, _i, _vp]),
    "rg_soft_cap": (_i, [_vp, _vp, ctypes.c_int64, ctypes.c_float, _i, _vp]),
    "rg_argmax_rows": (_i, [_vp, _vp, _i, _i, _i, _vp]),
    "rg_linear_rows_partial": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "rg_add_rms_norm_partial": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i,
                                     ctypes.c_float, _i, _vp]),
    "rg_add_rms_norm": (_i, [_vp, _vp, _vp, _vp, _vp, ctypes.c_int64, _i,
                             ctypes.c_float, _i, _vp]),
    "rg_rope": (_i, [_vp, _vp, _i, _vp, _vp, ctypes.c_int64, _i, _i, _i, _vp]),
    "rg_attention_decode_probs": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i,
                                       ctypes.c_float, _i, _vp]),
    "rg_attention_decode_finish": (_i, [_vp] * 8 + [_i] * 6 + [_vp]),
    "rg_attention_decode_fused_workspace_bytes": (_sz, [_i, _i, _i]),
    "rg_attention_decode_fused": (_i, [_vp, ctypes.c_int64, _vp, ctypes.c_int64,
                                       _vp, ctypes.c_int64, _vp, _i, _vp, _vp,
                                       _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i,
                                       ctypes.c_float, _i, _i, _vp]),
    "rg_packed_gate_weights_bytes": (_sz, [_i, _i, _i]),
    "rg_pack_gate_weights": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "rg_recurrent_step_packed": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp,
                                      _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i,
                                      _i, _vp]),
    "rg_recurrent_step_gelu_mul": (_i, [_vp, _vp, _vp, _i] + [_vp] * 11 +
                                   [_i, _i, _i, _i, _vp]),
    "rg_recurrent_step": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                               _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i,
                               _vp]),
}

_lib = None


class KernelError(RuntimeError):
  """A C-ABI call returned a non-zero status."""


def build(force: bool = True) -> str:
  """Compiles the HIP sources for gfx950 into librg_lru.so (in-tree)."""
  cmd = ["make", "-C", CSRC, "-j4"]
  if force:
    cmd.append("-B")
  subprocess.check_call(cmd)
  # The prefill kernel numbers its weight registers by hand: a build in which
  # the register allocator wanted one of them for itself must not be used.
  subprocess.check_call(["make", "-C", CSRC, "check-registers"])
  return LIB_PATH


def lib() -> ctypes.CDLL:
  global _lib
  if _lib is None:
    if not os.path.exists(LIB_PATH):
      raise RuntimeError(
          f"{LIB_PATH} is missing: build it with `make -C {CSRC}` "
          "(or __graft_entry__.build()). recurrentgemma_amd has no fallback "
          "path without its HIP library.")
    handle = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
      fn = getattr(handle, name)
      fn.restype = res
      fn.argtypes = args
    got = handle.rg_abi_version()
    if got != ABI_VERSION:
      raise RuntimeError(f"librg_lru.so has ABI {got}, expected {ABI_VERSION}")
    _lib = handle
  return _lib


def check(status: int) -> None:
  if status != RG_OK:
    msg = lib().rg_last_error().decode("utf-8", "replace")
    raise KernelError(f"librg_lru status {status}: {msg}")
