"""ctypes front-end of the plain-C oracle (oracle/rglru_ref.c).

TEST INFRASTRUCTURE ONLY.  Numpy in, numpy out; dtype float32 or float64 picks
the `_f32` / `_f64` symbol.  Build with `make -C oracle` (also done by
`__graft_entry__.build()`).
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "librglru_ref.so")
_lib = None


def build(force: bool = False) -> str:
  if force or not os.path.exists(_SO):
    subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
  return _SO


def lib():
  global _lib
  if _lib is None:
    _lib = ctypes.CDLL(build())
  return _lib


def _fn(name, dtype):
  suffix = {np.dtype(np.float32): "_f32", np.dtype(np.float64): "_f64"}[
      np.dtype(dtype)]
  f = getattr(lib(), name + suffix)
  f.restype = None
  return f


def _p(a):
  return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
  return np.ascontiguousarray(a, dtype=dtype)


def conv1d_prefill(x, segpos, w, b, want_cache=True):
  dt = x.dtype
  B, T, W = x.shape
  K = w.shape[0]
  x, w, b = _c(x, dt), _c(w, dt), _c(b, dt)
  sp = _c(segpos, np.int64)
  out = np.empty((B, T, W), dt)
  cache = np.empty((B, K - 1, W), dt) if want_cache else None
  _fn("ref_conv1d_prefill", dt)(_p(x), _p(sp), _p(w), _p(b), B, T, W, K,
                                _p(out), _p(cache))
  return out, cache


def conv1d_step(x, cache, w, b):
  dt = x.dtype
  B, W = x.shape[0], x.shape[-1]
  K = w.shape[0]
  x, cache, w, b = _c(x, dt), _c(cache, dt), _c(w, dt), _c(b, dt)
  out = np.empty((B, 1, W), dt)
  new_cache = np.empty((B, K - 1, W), dt)
  _fn("ref_conv1d_step", dt)(_p(x), _p(cache), _p(w), _p(b), B, W, K, _p(out),
                             _p(new_cache))
  return out, new_cache


def block_diag_linear(x, w, b):
  dt = x.dtype
  H, bw, _ = w.shape
  M = x.size // (H * bw)
  x, w, b = _c(x, dt), _c(w, dt), _c(b, dt)
  y = np.empty(x.shape, dt)
  _fn("ref_block_diag_linear", dt)(_p(x), _p(w), _p(b), M, H, bw, _p(y))
  return y


def rglru(x, segpos, a_param, w_x, b_x, w_a, b_a, h0=None):
  """Full RGLRU.forward on the conv output x [B,T,W] -> (y, h_last)."""
  dt = x.dtype
  B, T, W = x.shape
  x = _c(x, dt)
  gx = block_diag_linear(x, w_x, b_x)
  ga = block_diag_linear(x, w_a, b_a)
  sp = _c(segpos, np.int64)
  ap = _c(a_param, dt)
  h0 = None if h0 is None else _c(h0, dt)
  y = np.empty((B, T, W), dt)
  h = np.empty((B, W), dt)
  _fn("ref_rglru_scan", dt)(_p(x), _p(gx), _p(ga), _p(sp), _p(ap), _p(h0), B,
                            T, W, _p(y), _p(h))
  return y, h
