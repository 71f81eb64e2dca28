"""Drop-in modules for the reference's recurrent-block layers, on HIP kernels.

Same constructor arguments, parameter names/shapes (so reference state-dicts
load unchanged), forward signatures and cache conventions as
recurrentgemma/torch/layers.py:
  BlockDiagonalLinear  layers.py:76-137
  rnn_scan             layers.py:140-191
  rnn_param_init       layers.py:194-213
  RGLRU                layers.py:233-376
  Conv1D               layers.py:379-650
The kernels are forward only; inside `training.differentiable()` the modules
run the reference's op sequence under autograd with the recurrence on the scan
kernel in both directions (see training.py).

Differences from the reference, on purpose:
  * Conv1D.forward does not modify its input (the reference multiplies slices
    of `x` by the document mask in place); the returned cache is the same
    masked tail the reference returns.
  * In bfloat16 the kernels compute in float32 and round once per module output
    (gate pre-activations are also held in bfloat16), where the reference rounds
    after every elementwise op.
  * Tensors must live on a GPU; there is no CPU path.
"""

from __future__ import annotations

import math

import torch
from torch import nn

from recurrentgemma_amd import ops
from recurrentgemma_amd import training


def _normal_(w: torch.Tensor, variance: float) -> None:
  torch.nn.init.normal_(w, mean=0.0, std=math.sqrt(variance))


def _new_param(shape, device, dtype) -> nn.Parameter:
  return nn.Parameter(torch.empty(tuple(shape), device=device, dtype=dtype))


class BlockDiagonalLinear(nn.Module):
  """Block-diagonal linear layer: y[..., h, :] = x[..., h, :] @ w[h] + b[h]."""

  def __init__(self, width, num_blocks, w_init_variance_scale=1.0, device=None,
               dtype=None):
    nn.Module.__init__(self)
    bw = width // num_blocks
    self.width, self.num_blocks, self.block_width = width, num_blocks, bw
    self.w_init_variance_scale = w_init_variance_scale
    self.w = _new_param((num_blocks, bw, bw), device, dtype)  # [H, in, out]
    self.b = _new_param((num_blocks, bw), device, dtype)
    self.reset_parameters()

  def reset_parameters(self) -> None:
    self.w_init_(self.w)
    with torch.no_grad():
      self.b.zero_()

  def w_init_(self, w: torch.Tensor) -> None:
    _normal_(w, self.w_init_variance_scale / self.block_width)

  def forward(self, x: torch.Tensor) -> torch.Tensor:
    if training.is_enabled():
      return training.block_diag_linear(x, self.w, self.b)
    with torch.no_grad():
      return ops.block_diag_linear(x, self.w, self.b)


def rnn_scan(x, a, reset, h0, acc_dtype=torch.float32):
  """h_t = a_t h_{t-1} + x_t with a zeroed at resets; float32 state."""
  if x.ndim != 3 or a.shape != x.shape[-a.ndim:]:
    raise AssertionError(f"x {tuple(x.shape)} / a {tuple(a.shape)}")
  if a.dtype != x.dtype or type(a) is not type(x):
    raise AssertionError("x and a must have one dtype")
  if h0 is not None and h0.dtype != acc_dtype:
    raise AssertionError(f"h0 must be {acc_dtype}")
  if acc_dtype != torch.float32:
    raise NotImplementedError("the scan kernel keeps its state in float32")
  if training.is_enabled():
    return training.rnn_scan(x, a, reset, h0)
  if a.shape != x.shape:
    a = a.expand_as(x)
  with torch.no_grad():
    return ops.linear_scan(x, a, reset, h0)


def rnn_param_init(tensor, min_rad, max_rad, transform="softplus", eps=1e-8):
  """Initialises Lambda so that exp(-softplus(Lambda)) lies on a ring."""
  if transform != "softplus":
    raise NotImplementedError(transform)
  lo, hi = min_rad * min_rad + eps, max_rad * max_rad + eps
  with torch.no_grad():
    # u ~ U[lo, hi];  Lambda = log(u^(-1/2) - 1), step by step in place so that
    # the values are those of the reference for the same generator state
    for op, arg in (("uniform_", (lo, hi)), ("log_", ()), ("mul_", (0.5,)),
                    ("neg_", ()), ("exp_", ()), ("sub_", (1.0,)), ("log_", ())):
      getattr(tensor, op)(*arg)
  return tensor


class RGLRU(nn.Module):
  """Real-Gated Linear Recurrent Unit."""

  def __init__(self, width, num_heads, w_init_variance_scale=1.0, device=None,
               dtype=None):
    nn.Module.__init__(self)
    self.width, self.num_heads = width, num_heads
    self.w_init_variance_scale = w_init_variance_scale
    self.a_param = _new_param((width,), device, dtype)
    gate = dict(width=width, num_blocks=num_heads,
                w_init_variance_scale=w_init_variance_scale, device=device,
                dtype=dtype)
    self.input_gate, self.a_gate = (BlockDiagonalLinear(**gate),
                                    BlockDiagonalLinear(**gate))
    self.reset_parameters()

  def reset_parameters(self) -> None:
    for gate in (self.input_gate, self.a_gate):
      gate.reset_parameters()
    self.a_param_init(self.a_param)

  def a_param_init(self, w: torch.Tensor) -> torch.Tensor:
    return rnn_param_init(w, min_rad=0.9, max_rad=0.999)

  def forward(self, x, segment_pos, cache=None, return_cache=True):
    """x [B,T,W] (the conv output), cache: previous state [B,W] float32."""
    if tuple(segment_pos.shape) != tuple(x.shape[:2]):
      raise AssertionError(f"segment_pos {tuple(segment_pos.shape)} does not "
                           f"match x {tuple(x.shape)}")
    if training.is_enabled():
      y, last_h = training.rg_lru(
          x, segment_pos, self.a_param, self.input_gate.w, self.input_gate.b,
          self.a_gate.w, self.a_gate.b, h0=cache)
      return y, (last_h if return_cache else None)
    with torch.no_grad():
      return self._forward_kernels(x, segment_pos, cache, return_cache)

  def _forward_kernels(self, x, segment_pos, cache, return_cache):
    # one call without conv weights: the library picks the single prefill
    # kernel or gate GEMM + scan as it does for the whole block
    y, last_h, _ = ops.recurrent_core(
        x, segment_pos, None, None, self.input_gate.w, self.input_gate.b,
        self.a_gate.w, self.a_gate.b, self.a_param, h0=cache,
        return_h=return_cache, return_conv_cache=False)
    if not return_cache:
      return y, None
    return y, last_h

  @classmethod
  def init_cache(cls, batch_size, width, device=None):
    # The RG-LRU state is always float32.
    return torch.zeros((batch_size, width), dtype=torch.float32, device=device)


class Conv1D(nn.Module):
  """Causal depthwise temporal convolution with document masking."""

  def __init__(self, width, temporal_width, w_init_variance_scale=0.01,
               device=None, dtype=None):
    nn.Module.__init__(self)
    self.width, self.temporal_width = width, temporal_width
    self.w_init_variance_scale = w_init_variance_scale
    self.w = _new_param((temporal_width, width), device, dtype)
    self.b = _new_param((width,), device, dtype)
    self.reset_parameters()

  def reset_parameters(self) -> None:
    self.w_init_(self.w)
    with torch.no_grad():
      self.b.zero_()

  def w_init_(self, w: torch.Tensor) -> None:
    _normal_(w, self.w_init_variance_scale / self.temporal_width)

  def forward(self, x, segment_pos, cache=None, return_cache=True):
    """cache None: prefill over [B,T,W]; cache [B,K-1,W]: one decode token."""
    if training.is_enabled():
      if cache is not None:
        raise NotImplementedError("the differentiable path is prefill only")
      out = training.conv1d(x, segment_pos, self.w, self.b)
      new_cache = None
      if return_cache:  # the masked tail the kernels return, outside autograd
        with torch.no_grad():
          new_cache = ops.conv1d_prefill(x.detach(), segment_pos, self.w,
                                         self.b, True)[1]
      return out, new_cache
    with torch.no_grad():
      return self._forward_kernels(x, segment_pos, cache, return_cache)

  def _forward_kernels(self, x, segment_pos, cache, return_cache):
    if cache is not None:
      b, num_tokens, d = x.shape
      assert cache.shape == (b, self.temporal_width - 1, d)
      assert num_tokens == 1
      return ops.conv1d_step(x, cache, self.w, self.b, return_cache)
    return ops.conv1d_prefill(x, segment_pos, self.w, self.b, return_cache)

  @classmethod
  def init_cache(cls, *, batch_size, width, dtype, conv1d_temporal_width=4,
                 device=None):
    shape = (batch_size, conv1d_temporal_width - 1, width)
    return torch.zeros(shape, dtype=dtype, device=device)
