"""The hot-path calls as torch custom operators, so that a traced program
(torch.compile, torch.export) can hold them: each is an opaque node with a
shape function, no graph break, no tracing into the ctypes layer.

  torch.ops.recurrentgemma_amd.recurrent_core   conv -> RG-LRU of a prefill
                                                (ops.recurrent_core)
  torch.ops.recurrentgemma_amd.recurrent_step   one decode step, new cache
                                                tensors (ops.recurrent_step)

modules.recurrent_core goes through them while a program is being traced and
calls ops.* directly otherwise (the dispatcher costs about ten microseconds a
call, which a decode step launched from Python does not have to spare).  The
reference has no counterpart: its modules are plain tensor ops, which the
tracer follows by itself.  Inference only (no autograd formula is registered;
inside training.differentiable() the modules take the differentiable path).
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from recurrentgemma_amd import ops

Tensor = torch.Tensor


@torch.library.custom_op("recurrentgemma_amd::recurrent_core", mutates_args=())
def recurrent_core(x: Tensor, segment_pos: Tensor, conv_w: Tensor,
                   conv_b: Tensor, w_x: Tensor, b_x: Tensor, w_a: Tensor,
                   b_a: Tensor, a_param: Tensor, h0: Optional[Tensor],
                   gate_branch: Optional[Tensor]
                   ) -> Tuple[Tensor, Tensor, Tensor]:
  y, h, cache = ops.recurrent_core(x, segment_pos, conv_w, conv_b, w_x, b_x,
                                   w_a, b_a, a_param, h0=h0,
                                   gate_branch=gate_branch)
  return y, h, cache


@recurrent_core.register_fake
def _(x, segment_pos, conv_w, conv_b, w_x, b_x, w_a, b_a, a_param, h0,
      gate_branch):
  B, T, W = x.shape
  return (torch.empty_like(x),
          x.new_empty((B, W), dtype=torch.float32),
          x.new_empty((B, 3, W)))


@torch.library.custom_op("recurrentgemma_amd::recurrent_step", mutates_args=())
def recurrent_step(x: Tensor, segment_pos: Tensor, conv_cache: Tensor,
                   h: Tensor, conv_w: Tensor, conv_b: Tensor, w_x: Tensor,
                   b_x: Tensor, w_a: Tensor, b_a: Tensor, a_param: Tensor,
                   gate_branch: Optional[Tensor]
                   ) -> Tuple[Tensor, Tensor, Tensor]:
  y, h_new, cache = ops.recurrent_step(x, segment_pos, conv_cache, h, conv_w,
                                       conv_b, w_x, b_x, w_a, b_a, a_param,
                                       gate_branch=gate_branch)
  return y, h_new, cache


@recurrent_step.register_fake
def _(x, segment_pos, conv_cache, h, conv_w, conv_b, w_x, b_x, w_a, b_a,
      a_param, gate_branch):
  return torch.empty_like(x), torch.empty_like(h), torch.empty_like(conv_cache)


def tracing() -> bool:
  """Whether the caller runs under a tracer that needs operator nodes."""
  return torch.compiler.is_compiling()
