"""Writes tests/golden/hotpath_golden.npz from the REAL reference implementation.

Run once, in the build container only (the reference does not exist on the GPU
box):  python tests/golden/make_golden.py

The reference's `recurrentgemma/torch/layers.py` is loaded by file path.  Its
package `__init__` imports JAX and `array_typing.py` imports `jaxtyping`, neither
of which is installed, so `sys.modules` is pre-seeded with a minimal stand-in for
the `jaxtyping` annotation classes and with empty parent packages; no reference
file is modified, copied or written.

Vectors are written for the three things that closed forms and brute force do
not pin (everything else in the oracle is pinned without the reference):
  * Conv1D.forward: the returned cache when a document boundary lies in the
    last positions, and the in-place modification of the input;
  * RGLRU.forward (and through it BlockDiagonalLinear / rnn_scan): the exact
    sequence of roundings in bfloat16;
  * rnn_param_init: the draws for a given torch seed.
bfloat16 tensors are stored as their int16 bit patterns.
"""

import importlib.util
import os
import sys
import types

import numpy as np
import torch

REF = "/root/reference/recurrentgemma/torch"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)),
                   "hotpath_golden.npz")


def load_reference_layers():
  class _Ann:
    def __class_getitem__(cls, item):
      return cls

  jt = types.ModuleType("jaxtyping")
  for name in ("Float", "Integer", "Bool", "Int", "Array"):
    setattr(jt, name, type(name, (_Ann,), {}))
  sys.modules["jaxtyping"] = jt
  for pkg in ("recurrentgemma", "recurrentgemma.torch"):
    m = types.ModuleType(pkg)
    m.__path__ = []
    sys.modules[pkg] = m

  def load(name, path):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod

  at = load("recurrentgemma.torch.array_typing",
            os.path.join(REF, "array_typing.py"))
  sys.modules["recurrentgemma.torch"].array_typing = at
  return load("recurrentgemma.torch.layers", os.path.join(REF, "layers.py"))


def f32(t):
  """float32 as is; bfloat16 as its int16 bit pattern (half the bytes)."""
  t = t.detach()
  if t.dtype == torch.bfloat16:
    return t.contiguous().view(torch.int16).numpy().copy()
  return t.to(torch.float32).numpy().copy()


def segment_patterns(T):
  """name -> [2, T] int64 positions (row 0 and row 1 differ)."""
  ar = torch.arange(T)
  pats = {"arange": torch.stack([ar, ar])}
  half = torch.arange(max(T // 2, 1))
  two = torch.cat([half, half])[:T]
  if two.shape[0] < T:
    two = torch.cat([two, torch.arange(T - two.shape[0])])
  pats["halves"] = torch.stack([two, ar])
  # boundaries in the last two positions / at the very end
  tail1 = ar.clone()
  tail1[-1] = 0
  tail2 = ar.clone()
  if T >= 2:
    tail2[-2] = 0
    tail2[-1] = 1
  pats["tail"] = torch.stack([tail1, tail2])
  # sampler-style left padding: pad positions are -1, first real token is 0
  npad = T // 3
  padded = torch.cat([torch.full((npad,), -1), torch.arange(T - npad)])
  dense = ar.clone()
  dense[::2] = 0  # a boundary every other token
  pats["pad_dense"] = torch.stack([padded, dense])
  return pats


def main():
  layers = load_reference_layers()
  torch.manual_seed(20240607)
  out = {}
  index = []

  # ---- Conv1D ----------------------------------------------------------
  W = 32
  for dtype in (torch.float32, torch.bfloat16):
    for K in (4, 8):
      conv = layers.Conv1D(width=W, temporal_width=K, dtype=dtype)
      with torch.no_grad():
        conv.b.normal_(0.0, 0.1)
      for T in (1, 2, 3, 5, 32):
        for pname, seg in segment_patterns(T).items():
          key = f"conv/{str(dtype)[6:]}/K{K}/T{T}/{pname}"
          x = torch.randn(2, T, W).to(dtype)
          x_in = x.clone()
          with torch.no_grad():
            y, cache = conv(x, seg)
            y_nc, none_cache = conv(x_in.clone(), seg, return_cache=False)
          assert none_cache is None and torch.equal(y, y_nc)
          out[key + "/x"] = f32(x_in)
          out[key + "/x_after"] = f32(x)  # mutated by the reference
          out[key + "/seg"] = seg.numpy()
          out[key + "/w"] = f32(conv.w)
          out[key + "/b"] = f32(conv.b)
          out[key + "/y"] = f32(y)
          out[key + "/cache"] = f32(cache)
          # two decode steps from that cache (decode ignores segment_pos)
          xs = torch.randn(2, 2, W).to(dtype)
          out[key + "/step_x"] = f32(xs)
          for i in range(2):
            with torch.no_grad():
              ys, cache = conv(xs[:, i:i + 1].clone(), seg[:, -1:] + 1 + i,
                               cache)
            out[key + f"/step{i}_y"] = f32(ys)
            out[key + f"/step{i}_cache"] = f32(cache)
          index.append(key)

  # ---- RGLRU -----------------------------------------------------------
  for (W, H, dtypes) in ((128, 1, (torch.float32,)),
                         (128, 16, (torch.float32, torch.bfloat16)),
                         (256, 1, (torch.bfloat16,))):
    for dtype in dtypes:
      lru = layers.RGLRU(width=W, num_heads=H, dtype=dtype)
      with torch.no_grad():
        lru.input_gate.b.normal_(0.0, 0.3)
        lru.a_gate.b.normal_(0.0, 0.3)
      pkey = f"rglru/{str(dtype)[6:]}/W{W}H{H}"
      out[pkey + "/a_param"] = f32(lru.a_param)
      out[pkey + "/w_x"] = f32(lru.input_gate.w)
      out[pkey + "/b_x"] = f32(lru.input_gate.b)
      out[pkey + "/w_a"] = f32(lru.a_gate.w)
      out[pkey + "/b_a"] = f32(lru.a_gate.b)
      for T in (1, 5, 32):
        for pname, seg in segment_patterns(T).items():
          if T == 32 and pname in ("arange", "tail"):
            continue
          for with_h0 in (False, True):
            if T == 32 and with_h0 != (pname == "pad_dense"):
              continue
            key = f"{pkey}/T{T}/{pname}/h0{int(with_h0)}"
            x = torch.randn(2, T, W).to(dtype)
            h0 = torch.randn(2, W) if with_h0 else None
            with torch.no_grad():
              y, h = lru(x, seg, h0)
            out[key + "/x"] = f32(x)
            out[key + "/seg"] = seg.numpy()
            if with_h0:
              out[key + "/h0"] = f32(h0)
            out[key + "/y"] = f32(y)
            out[key + "/h"] = f32(h)
            xs = torch.randn(2, 2, W).to(dtype)
            out[key + "/step_x"] = f32(xs)
            for i in range(2):
              with torch.no_grad():
                ys, h = lru(xs[:, i:i + 1], seg[:, -1:] + 1 + i, h)
              out[key + f"/step{i}_y"] = f32(ys)
              out[key + f"/step{i}_h"] = f32(h)
            index.append(key)

  # ---- rnn_param_init --------------------------------------------------
  for seed in (0, 1, 2):
    torch.manual_seed(seed)
    t = torch.empty(64)
    layers.rnn_param_init(t, min_rad=0.9, max_rad=0.999)
    out[f"init/seed{seed}"] = f32(t)
    index.append(f"init/seed{seed}")

  out["index"] = np.array(index)
  np.savez_compressed(OUT, **out)
  print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(index), "cases")


if __name__ == "__main__":
  main()
