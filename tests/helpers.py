"""Shared input builders and fixture loading for the tests."""

from __future__ import annotations

import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                      "hotpath_golden.npz")


class Golden:
  """tests/golden/hotpath_golden.npz: int16 arrays are bfloat16 bit patterns."""

  def __init__(self, path=GOLDEN):
    self._z = np.load(path, allow_pickle=False)
    self.index = [str(s) for s in self._z["index"]]

  def has(self, key):
    return key in self._z.files

  def get(self, key):
    a = self._z[key]
    t = torch.from_numpy(a.copy())
    if a.dtype == np.int16:
      return t.view(torch.bfloat16)
    return t

  def cases(self, prefix):
    return [k for k in self.index if k.startswith(prefix)]


def load_golden():
  return Golden()


def document_positions(batch, length, mean_len, seed, first_is_zero=True):
  """[B,T] int64 position-within-document; document lengths ~ Geometric."""
  rng = np.random.default_rng(seed)
  out = np.zeros((batch, length), np.int64)
  for b in range(batch):
    t = 0
    while t < length:
      n = int(rng.geometric(1.0 / mean_len))
      n = min(n, length - t)
      out[b, t:t + n] = np.arange(n)
      t += n
    if not first_is_zero:
      out[b, 0] = 7
  return torch.from_numpy(out)


def max_rel(got, want):
  """max|got-want| / max|want| over the whole tensor (both widened to fp64)."""
  got = got.detach().double().cpu()
  want = want.detach().double().cpu()
  denom = want.abs().max().item()
  return (got - want).abs().max().item() / max(denom, 1e-30)
