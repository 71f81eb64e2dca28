"""The caller of the hot path: Griffin's recurrent block, on the fused kernels.

RecurrentBlock / RecurrentBlockCache mirror
recurrentgemma/torch/modules.py:32-37 and :496-680 (same constructor,
parameter names, forward signature and cache tuple).  linear_x / linear_y /
linear_out stay torch.nn.Linear (hipBLASLt); conv_1d -> rg_lru runs as
  prefill: rg_recurrent_core (the single prefill kernel, or rg_gates_gemm with
           the conv on load + rg_lru_scan_fused: the library picks)
  decode : rg_recurrent_step
unless the conv width is not 4, where the stand-alone conv kernel is used.
"""

from __future__ import annotations

import math
from typing import NamedTuple

import torch
from torch import nn

from recurrentgemma_amd import compiled
from recurrentgemma_amd import layers
from recurrentgemma_amd import ops
from recurrentgemma_amd import training


class RecurrentBlockCache(NamedTuple):
  rg_lru_state: torch.Tensor  # [B, lru_width] float32
  conv1d_state: torch.Tensor  # [B, temporal_width-1, lru_width]


def gelu(x: torch.Tensor) -> torch.Tensor:
  return nn.functional.gelu(x, approximate="tanh")


@torch.no_grad()
def recurrent_core(conv_1d: layers.Conv1D, rg_lru: layers.RGLRU, x,
                   segment_pos, cache: RecurrentBlockCache | None = None,
                   return_cache: bool = True, in_place: bool = False,
                   gate_branch=None):
  """conv_1d -> rg_lru exactly as RecurrentBlock.forward chains them
  (modules.py:632-643), fused.  Returns (y, RecurrentBlockCache | None).
  in_place (decode only): the step overwrites the tensors of `cache` and
  returns them, for callers that replay a captured step on fixed buffers; the
  default returns new tensors like the reference.
  gate_branch: the block's linear_y output; the result is then the join
  y * gelu(gate_branch) of modules.py:627-628, 644 -- inside the prefill
  kernel where that runs, as a pass of its own (ops.gelu_mul) elsewhere."""
  bs, l, _ = x.shape
  assert segment_pos.shape == (bs, l)
  fused = conv_1d.temporal_width == 4
  if cache is not None:
    b, num_tokens, d = x.shape
    assert cache.conv1d_state.shape == (b, conv_1d.temporal_width - 1, d)
    assert num_tokens == 1
    if fused:
      if compiled.tracing() and not in_place:
        # (a traced program holds the step as one operator node)
        y, h, conv_state = torch.ops.recurrentgemma_amd.recurrent_step(
            x, segment_pos, cache.conv1d_state, cache.rg_lru_state, conv_1d.w,
            conv_1d.b, rg_lru.input_gate.w, rg_lru.input_gate.b,
            rg_lru.a_gate.w, rg_lru.a_gate.b, rg_lru.a_param, gate_branch)
      else:
        y, h, conv_state = ops.recurrent_step(
            x, segment_pos, cache.conv1d_state, cache.rg_lru_state, conv_1d.w,
            conv_1d.b, rg_lru.input_gate.w, rg_lru.input_gate.b,
            rg_lru.a_gate.w, rg_lru.a_gate.b, rg_lru.a_param,
            in_place=in_place, gate_branch=gate_branch)
      if not return_cache:
        return y, None
      return y, RecurrentBlockCache(rg_lru_state=h, conv1d_state=conv_state)
  if not fused or cache is not None:
    if in_place:
      raise ValueError("in-place decode needs the fused step (conv width 4)")
    xc, conv_state = conv_1d(x, segment_pos,
                             None if cache is None else cache.conv1d_state,
                             return_cache)
    y, h = rg_lru(xc, segment_pos,
                  None if cache is None else cache.rg_lru_state, return_cache)
  else:
    # One call; the library picks the kernels (rg_recurrent_core): for bf16
    # and 256-wide heads the single-launch kernel, one workgroup per (row,
    # head) or -- rows of few pairs -- per chunk of one (many rows of a few
    # tokens and every other dtype or head width: gate GEMM + scan; float32
    # with 256-wide heads and few pairs: a one-launch float32 kernel), and
    # the join with the gate branch inside those kernels (after the two-kernel
    # form it is a pass of its own).
    if compiled.tracing():
      y, h, conv_state = torch.ops.recurrentgemma_amd.recurrent_core(
          x, segment_pos, conv_1d.w, conv_1d.b, rg_lru.input_gate.w,
          rg_lru.input_gate.b, rg_lru.a_gate.w, rg_lru.a_gate.b,
          rg_lru.a_param, None, gate_branch)
    else:
      y, h, conv_state = ops.recurrent_core(
          x, segment_pos, conv_1d.w, conv_1d.b, rg_lru.input_gate.w,
          rg_lru.input_gate.b, rg_lru.a_gate.w, rg_lru.a_gate.b,
          rg_lru.a_param, h0=None, return_h=return_cache,
          return_conv_cache=return_cache, gate_branch=gate_branch)
    gate_branch = None
  if gate_branch is not None:
    y = ops.gelu_mul(y, gate_branch)
  if not return_cache:
    return y, None
  return y, RecurrentBlockCache(rg_lru_state=h, conv1d_state=conv_state)


class RecurrentBlock(nn.Module):
  """Griffin and Hawk's recurrent block."""

  def __init__(self, width, num_heads, lru_width=None, conv1d_temporal_width=4,
               final_w_init_variance_scale=1.0, device=None, dtype=None):
    super().__init__()
    self.width = width
    self.num_heads = num_heads
    self.lru_width = lru_width or width
    self.conv1d_temporal_width = conv1d_temporal_width
    self.final_w_init_variance_scale = final_w_init_variance_scale
    self.linear_y = nn.Linear(self.width, self.lru_width, device=device,
                              dtype=dtype)
    self.linear_x = nn.Linear(self.width, self.lru_width, device=device,
                              dtype=dtype)
    self.linear_out = nn.Linear(self.lru_width, self.width, device=device,
                                dtype=dtype)
    self.conv_1d = layers.Conv1D(width=self.lru_width,
                                 temporal_width=self.conv1d_temporal_width,
                                 device=device, dtype=dtype)
    self.rg_lru = layers.RGLRU(width=self.lru_width, num_heads=self.num_heads,
                               device=device, dtype=dtype)
    # True: a cached single-token call updates the cache tensors it is given
    # instead of returning new ones (set by callers that replay a captured
    # decode step on fixed buffers)
    self.decode_in_place = False
    # the linear layers for at most 64 rows (a decode step): linear_y and
    # linear_x as one pass over both weight matrices, linear_out as another
    self._rows_yx = ops.PackedLinear()
    self._rows_out = ops.PackedLinear()
    self.reset_parameters()

  def reset_parameters(self) -> None:
    self.w_init_(self.linear_x.weight)
    torch.nn.init.zeros_(self.linear_x.bias)
    self.w_init_(self.linear_y.weight)
    torch.nn.init.zeros_(self.linear_y.bias)
    self.out_w_init_(self.linear_out.weight)
    torch.nn.init.zeros_(self.linear_out.bias)
    self.conv_1d.reset_parameters()
    self.rg_lru.reset_parameters()

  def w_init_(self, w: torch.Tensor) -> None:
    torch.nn.init.normal_(w, mean=0.0, std=math.sqrt(1.0 / self.width))

  def out_w_init_(self, w: torch.Tensor) -> None:
    std = math.sqrt(self.final_w_init_variance_scale / self.lru_width)
    torch.nn.init.normal_(w, mean=0.0, std=std)

  def forward(self, x, segment_pos, cache=None, return_cache=True,
              defer_out=False):
    """defer_out: the caller adds the result to a residual and normalises it
    next (ops.add_rms_norm) and accepts it as ops.PartialSums, which is what
    it gets where that saves a pass (a few rows, bf16)."""
    if training.is_enabled():
      return self._forward_differentiable(x, segment_pos, cache, return_cache)
    with torch.no_grad():
      # (a traced program keeps torch's own linear layers: the few-row
      # kernels are reached through ctypes, which a tracer cannot follow)
      few_rows = (
          not compiled.tracing() and
          ops.PackedLinear.usable(x, self.width, self.lru_width) and
          ops.PackedLinear.usable(x, self.lru_width, self.width))
      if few_rows:
        y, x = self._rows_yx(x, (self.linear_y.weight, self.linear_x.weight),
                             (self.linear_y.bias, self.linear_x.bias))
      else:
        y = self.linear_y(x)
        x = self.linear_x(x)
      # x * gelu(y) (modules.py:627-628, 644) is part of the core call: inside
      # the prefill kernel where that runs, one pass after it elsewhere
      x, new_cache = recurrent_core(
          self.conv_1d, self.rg_lru, x, segment_pos, cache, return_cache,
          in_place=self.decode_in_place and cache is not None and return_cache,
          gate_branch=y)
      if few_rows and defer_out and ops.PackedLinear.partial_slices(
          x, self.lru_width, self.width):
        x = self._rows_out.partial(x, (self.linear_out.weight,),
                                   (self.linear_out.bias,))
      elif few_rows:
        x = self._rows_out(x, (self.linear_out.weight,),
                           (self.linear_out.bias,))
      else:
        x = self.linear_out(x)
    if not return_cache:
      return x, None
    return x, new_cache

  def _forward_differentiable(self, x, segment_pos, cache, return_cache):
    """The reference's op sequence (modules.py:605-655) under autograd."""
    if cache is not None:
      raise NotImplementedError("the differentiable path is prefill only")
    y = self.linear_y(x)
    x = self.linear_x(x)
    x, conv_state = self.conv_1d(x, segment_pos, None, return_cache)
    x, h = self.rg_lru(x, segment_pos, None, return_cache)
    x = self.linear_out(training.gelu_mul(x, y))  # x * gelu(y)
    if not return_cache:
      return x, None
    return x, RecurrentBlockCache(rg_lru_state=h, conv1d_state=conv_state)

  @classmethod
  def init_cache(cls, batch_size, lru_width, dtype, conv1d_temporal_width=4,
                 device=None):
    return RecurrentBlockCache(
        rg_lru_state=layers.RGLRU.init_cache(batch_size=batch_size,
                                             width=lru_width, device=device),
        conv1d_state=layers.Conv1D.init_cache(
            batch_size=batch_size, width=lru_width, dtype=dtype,
            conv1d_temporal_width=conv1d_temporal_width, device=device),
    )
