"""Writes tests/golden/grad_golden.npz: gradients of the REAL reference's
RecurrentBlock (recurrentgemma/torch/modules.py:496-680) by torch autograd
through its own Python loop over time, float32, tiny shapes.

Run once, in the build container only:  python tests/golden/make_grad_golden.py
(the reference is loaded by file path as in make_griffin_golden.py).

Nothing else pins the backward pass: the clipped derivative of
sqrt(1 - a^2), the treatment of document starts (a = 0, unit input scale, conv
history cut) and the carried-in state in the gradients.
Cases: a left-padded / multi-document batch, and an initial state h0 given to
the RG-LRU alone (the block itself does not take one in prefill).
"""

import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import make_griffin_golden as loader  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)),
                   "grad_golden.npz")


def main():
  loader.load_reference()
  modules = sys.modules["recurrentgemma.torch.modules"]
  layers = sys.modules["recurrentgemma.torch.layers"]
  out = {}
  torch.manual_seed(99)
  gen = torch.Generator().manual_seed(5)

  # ---- the whole block ----------------------------------------------------
  blk = modules.RecurrentBlock(width=32, num_heads=2, lru_width=64,
                               dtype=torch.float32)
  with torch.no_grad():
    for name, p in blk.named_parameters():
      if name.endswith((".b", ".bias")):
        p.normal_(0.0, 0.2)
  B, T = 2, 13
  x = torch.randn(B, T, 32, generator=gen, requires_grad=True)
  seg = torch.stack([torch.tensor([-1, -1, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10]),
                     torch.tensor([0, 1, 2, 3, 0, 1, 0, 0, 1, 2, 3, 4, 5])])
  r = torch.randn(B, T, 32, generator=gen)
  rh = torch.randn(B, 64, generator=gen)
  y, cache = blk(x, seg)
  loss = (y * r).sum() + (cache.rg_lru_state * rh).sum()
  loss.backward()
  out["blk/x"], out["blk/seg"] = x.detach().numpy().copy(), seg.numpy()
  out["blk/r"], out["blk/rh"] = r.numpy(), rh.numpy()
  out["blk/y"] = y.detach().numpy().copy()
  out["blk/h"] = cache.rg_lru_state.detach().numpy().copy()
  out["blk/loss"] = np.array(loss.item())
  out["blk/grad/x"] = x.grad.numpy().copy()
  for name, p in blk.named_parameters():
    out[f"blk/param/{name}"] = p.detach().numpy().copy()
    out[f"blk/grad/{name}"] = p.grad.numpy().copy()

  # ---- the RG-LRU alone, with a carried-in state ----------------------------
  lru = layers.RGLRU(width=64, num_heads=2, dtype=torch.float32)
  with torch.no_grad():
    lru.input_gate.b.normal_(0.0, 0.2)
    lru.a_gate.b.normal_(0.0, 0.2)
  T = 7
  x = torch.randn(B, T, 64, generator=gen, requires_grad=True)
  h0 = torch.randn(B, 64, generator=gen, requires_grad=True)
  seg = torch.stack([torch.arange(5, 5 + T),
                     torch.tensor([9, 10, 0, 1, 2, 0, 1])])
  r = torch.randn(B, T, 64, generator=gen)
  rh = torch.randn(B, 64, generator=gen)
  y, h = lru(x, seg, h0)
  loss = (y * r).sum() + (h * rh).sum()
  loss.backward()
  out["lru/x"], out["lru/seg"] = x.detach().numpy().copy(), seg.numpy()
  out["lru/h0"] = h0.detach().numpy().copy()
  out["lru/r"], out["lru/rh"] = r.numpy(), rh.numpy()
  out["lru/y"], out["lru/h"] = y.detach().numpy().copy(), h.detach().numpy().copy()
  out["lru/grad/x"], out["lru/grad/h0"] = x.grad.numpy().copy(), h0.grad.numpy().copy()
  for name, p in lru.named_parameters():
    out[f"lru/param/{name}"] = p.detach().numpy().copy()
    out[f"lru/grad/{name}"] = p.grad.numpy().copy()

  np.savez_compressed(OUT, **out)
  print("wrote", OUT, len(out), "arrays,", os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
  main()
