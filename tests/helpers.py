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


def assert_close_elementwise(got, want, rtol=1e-2, atol_of_max=2e-3, what=""):
  """Element by element: |got - want| <= rtol |want| + atol_of_max max|want|
  (the reference's tests compare with rtol/atol per element,
  torch/layers_test.py:131; the absolute term is scaled to the tensor so that
  it stays a small fraction of typical magnitudes).  max_rel() alone would let
  small elements be wrong by many of their own ulps."""
  got = got.detach().double().cpu()
  want = want.detach().double().cpu()
  bound = rtol * want.abs() + atol_of_max * want.abs().max()
  excess = (got - want).abs() - bound
  worst = excess.max().item()
  assert worst <= 0, (
      f"{what}: {int((excess > 0).sum())} of {excess.numel()} elements outside "
      f"rtol={rtol} atol={atol_of_max}*max; worst excess {worst:.3e}")


def seeded_state_dict(shapes, seed, dtype=torch.bfloat16):
  """A state dict that a seed fixes: {name: shape} -> {name: tensor}, every
  value rounded to `dtype` and returned in it.  The golden vectors of the bf16
  residual stack were written by the reference model holding exactly these
  parameters (tests/golden/make_griffin_golden.py), so that a few MB of
  weights need not be stored; `param_checksum` in the fixture guards the
  regeneration.  Matrices ~ N(0, 1/fan_in), biases and norm scales ~ N(0, 0.1),
  a_param such that the base decay is uniform in [0.9, 0.999]."""
  out = {}
  for i, name in enumerate(sorted(shapes)):
    shape = tuple(shapes[name])
    g = torch.Generator().manual_seed(seed * 1000 + i)
    if name.endswith("a_param"):
      u = torch.rand(shape, generator=g) * 0.099 + 0.9
      t = torch.log(torch.expm1(-0.5 * torch.log(u)))
    elif name.endswith((".b", ".bias", ".scale")) or len(shape) < 2:
      t = torch.randn(shape, generator=g) * 0.1
    else:
      # nn.Linear and the embedding table are [out, in]; the block-diagonal,
      # einsum and conv weights [..., in, out]
      fan_in = (shape[-1] if name.endswith((".weight", "input_embedding"))
                else shape[-2])
      t = torch.randn(shape, generator=g) / fan_in ** 0.5
    out[name] = t.to(dtype)
  return out


def state_dict_checksum(sd):
  """Sum of |value| * (1 + position mod 7) over all tensors in name order, in
  float64: moves if any value, shape or order differs."""
  total = 0.0
  for name in sorted(sd):
    v = sd[name].detach().double().flatten().abs()
    w = (torch.arange(v.numel(), dtype=torch.float64) % 7) + 1.0
    total += float((v * w).sum())
  return total
