"""Differentiable forward of the recurrent block, for fine-tuning.

The inference kernels fuse conv, gates and recurrence and keep nothing for a
backward pass.  Inside `with training.differentiable():` the drop-in modules
(Conv1D, BlockDiagonalLinear, RGLRU, RecurrentBlock) instead run the
reference's sequence of tensor ops (recurrentgemma/torch/layers.py:127-137,
313-365, 447-529) on the GPU under autograd, except for the one part that is
a Python loop over time there: the linear recurrence (layers.py:140-191),
which is the scan kernel in both directions (and, for the RG-LRU, the gating
around it: one forward and one backward kernel from the gate pre-activations
on, rg_rglru_backward; the block's x * gelu(y) join likewise, rg_gelu_mul and
rg_gelu_mul_backward) --

  forward   h_t = a_t h_{t-1} + x_t
  backward  g_t = dy_t + a_{t+1} g_{t+1}     (the same recurrence, time
            dx_t = g_t                        reversed, coefficients shifted by
            da_t = g_t h_{t-1}                one step)
            dh_0 = a_0 g_0

with a_t zeroed at document starts.  sqrt(1 - a^2) keeps the reference's
clipped derivative (layers.py:216-230).  Prefill only (no decode cache).
"""

from __future__ import annotations

import contextlib

import torch

from recurrentgemma_amd import ops

_MAX_SQRT_GRADIENT = 1000.0
_enabled = False


def is_enabled() -> bool:
  return _enabled


@contextlib.contextmanager
def differentiable():
  """Within this context the modules of this package build an autograd
  graph (and are correspondingly slower and hungrier for memory)."""
  global _enabled
  old, _enabled = _enabled, True
  try:
    yield
  finally:
    _enabled = old


class _LinearScan(torch.autograd.Function):
  """y_t = h_t = a'_t h_{t-1} + x_t in float32, a' = a with zeros at resets;
  returns (y rounded to the activation dtype, h_last float32)."""

  @staticmethod
  def forward(ctx, x, a, reset, h0):
    y, h_last = ops.linear_scan(x, a, reset, h0)
    ctx.save_for_backward(a, reset, y, h0)
    return y, h_last

  @staticmethod
  def backward(ctx, dy, dh_last):
    a, reset, y, h0 = ctx.saved_tensors
    dh = None if dh_last is None else dh_last.float().contiguous()
    dy = torch.zeros_like(y) if dy is None else dy.contiguous()
    g, da, dh0 = ops.linear_scan_backward(dy, a, reset, y, h0, dh)
    return g, da, None, dh0


class _BoundedSqrt(torch.autograd.Function):
  """sqrt with the derivative clipped at _MAX_SQRT_GRADIENT."""

  @staticmethod
  def forward(ctx, x):
    ctx.save_for_backward(x)
    return torch.sqrt(x)

  @staticmethod
  def backward(ctx, grad):
    (x,) = ctx.saved_tensors
    return grad / torch.sqrt(torch.clip(4.0 * x,
                                        min=1 / (_MAX_SQRT_GRADIENT ** 2)))


def rnn_scan(x, a, reset, h0=None):
  if a.shape != x.shape:
    a = a.expand_as(x)
  return _LinearScan.apply(x.contiguous(), a.contiguous(), reset, h0)


def block_diag_linear_tensor_ops(x, w, b):
  """y[..., h, :] = x[..., h, :] @ w[h] + b[h]  (layers.py:127-137), the
  reference's own two tensor ops (the form the kernels are tested against)."""
  h, bw, _ = w.shape
  xs = x.reshape(*x.shape[:-1], h, bw)
  y = torch.einsum("...hi,hij->...hj", xs, w) + b
  return y.reshape(x.shape)


def _projection_grads(x, w, dy, need):
  """Gradients of y = block_diag_linear(x, w, b) for need = (x, w, b).
    dx[m, h, i] = sum_j dy[m, h, j] w[h, i, j]: the forward kernel on the
                  transposed blocks
    dw[h, i, j] = sum_m x[m, h, i] dy[m, h, j]: one batched product over
                  strided views of the [M, W] tensors (no copies)
    db[h, j]    = sum_m dy[m, h, j]"""
  heads, bw, _ = w.shape
  dx = dw = db = None
  if need[0]:
    dx = ops.block_diag_linear(dy, w.transpose(1, 2).contiguous(),
                               w.new_zeros((heads, bw)))
  if need[1] or need[2]:
    dy_h = dy.reshape(-1, heads, bw).transpose(0, 1)          # [H, M, bw]
    if need[1]:
      x_h = x.reshape(-1, heads, bw).permute(1, 2, 0)         # [H, bw, M]
      dw = torch.bmm(x_h, dy_h)
    if need[2]:
      db = dy.reshape(-1, heads, bw).sum(0)
  return dx, dw, db


class _BlockDiagLinear(torch.autograd.Function):
  """BlockDiagonalLinear.forward (layers.py:127-137) on rg_block_diag_linear
  in both directions."""

  @staticmethod
  def forward(ctx, x, w, b):
    x = x.contiguous()
    ctx.save_for_backward(x, w)
    return ops.block_diag_linear(x, w, b)

  @staticmethod
  def backward(ctx, dy):
    x, w = ctx.saved_tensors
    return _projection_grads(x, w, dy.contiguous(), ctx.needs_input_grad)


def _projections_on_kernels(x):
  """bf16: the kernels (one pass over x for both gates, no permuted copies);
  float32 keeps the library's batched products, which are ahead of the
  true-float32 matrix kernel at the row counts of a training step (B4 T2048
  W2560, whole block forward + backward: 9.4 ms against 10.3 ms; bf16 2.6
  against 2.4 ms)."""
  return x.dtype == torch.bfloat16


def block_diag_linear(x, w, b):
  """y[..., h, :] = x[..., h, :] @ w[h] + b[h]  (layers.py:127-137)."""
  if _projections_on_kernels(x):
    return _BlockDiagLinear.apply(x, w, b)
  return block_diag_linear_tensor_ops(x, w, b)


class _GateProjections(torch.autograd.Function):
  """Both gate projections of RGLRU.forward (layers.py:338-339, before the
  sigmoids): one pass over x forwards (rg_gates_gemm), the transposed blocks
  on the same kernels backwards."""

  @staticmethod
  def forward(ctx, x, w_x, b_x, w_a, b_a):
    x = x.contiguous()
    ctx.save_for_backward(x, w_x, w_a)
    return ops.gates_gemm(x, w_x, b_x, w_a, b_a)

  @staticmethod
  def backward(ctx, dgx, dga):
    x, w_x, w_a = ctx.saved_tensors
    need = ctx.needs_input_grad
    dgx, dga = dgx.contiguous(), dga.contiguous()
    if (need[1] and need[3] and need[2] == need[4] and
        ops.gates_weight_grads_supported(x, w_x.shape[0])):
      # weight and bias gradients of both projections in one pass over x and
      # the two output gradients (rg_gates_weight_grads)
      dwx, dwa, dbx, dba = ops.gates_weight_grads(x, dgx, dga, w_x.shape[0],
                                                  with_bias=need[2])
      dx1 = _projection_grads(x, w_x, dgx, (need[0], False, False))[0]
      dx2 = _projection_grads(x, w_a, dga, (need[0], False, False))[0]
      dx = dx1.add_(dx2) if need[0] else None
      return dx, dwx, dbx, dwa, dba
    dx1, dwx, dbx = _projection_grads(x, w_x, dgx, (need[0], need[1], need[2]))
    dx2, dwa, dba = _projection_grads(x, w_a, dga, (need[0], need[3], need[4]))
    # (the sum autograd would form of the two layers' input gradients)
    dx = dx1.add_(dx2) if need[0] else None
    return dx, dwx, dbx, dwa, dba


class _Conv1d(torch.autograd.Function):
  """Conv1D.forward without a cache (layers.py:447-529): the conv kernel
  forwards, rg_conv1d_backward backwards."""

  @staticmethod
  def forward(ctx, x, segment_pos, w, b):
    x = x.contiguous()
    out, _ = ops.conv1d_prefill(x, segment_pos, w, b, return_cache=False)
    ctx.save_for_backward(x, segment_pos, w)
    return out

  @staticmethod
  def backward(ctx, dout):
    x, segment_pos, w = ctx.saved_tensors
    dx, dw, db = ops.conv1d_backward(dout.contiguous(), x, segment_pos, w)
    return dx, None, dw, db


def conv1d(x, segment_pos, w, b):
  """Conv1D.forward without a cache, on the kernels in both directions."""
  return _Conv1d.apply(x, segment_pos, w, b)


def conv1d_tensor_ops(x, segment_pos, w, b):
  """Conv1D.forward without a cache (layers.py:447-529), functional: tap s of
  token t is x[t - s] unless a document starts at one of t-s+1 .. t.  (The
  form conv1d is tested against.)"""
  K = w.shape[0]
  T = x.shape[1]
  not_start = (segment_pos != 0).to(x.dtype)  # [B, T]
  keep = torch.ones_like(not_start)
  out = None
  for s in range(min(K, T)):
    if s > 0:
      # keep_s[t] = prod_{j < s} not_start[t - j]
      shifted = torch.nn.functional.pad(not_start, (s - 1, 0), value=1.0)[:, :T]
      keep = keep * shifted
    xs = torch.nn.functional.pad(x, (0, 0, s, 0))[:, :T]
    term = xs * keep[..., None] * w[K - 1 - s]
    out = term if out is None else out + term
  return out + b


class _GeluMul(torch.autograd.Function):
  """a * gelu_tanh(g), the join of RecurrentBlock.forward's two branches
  (modules.py:627-628, :644): one kernel each way, keeping the two inputs
  and not the activation."""

  @staticmethod
  def forward(ctx, a, g):
    a, g = a.contiguous(), g.contiguous()
    ctx.save_for_backward(a, g)
    return ops.gelu_mul(a, g)

  @staticmethod
  def backward(ctx, dout):
    a, g = ctx.saved_tensors
    return ops.gelu_mul_backward(dout.contiguous(), a, g)


def gelu_mul(a, g):
  """a * gelu_tanh(g) on kernels in both directions."""
  return _GeluMul.apply(a, g)


class _GatedScan(torch.autograd.Function):
  """RGLRU.forward from the gate pre-activations on (layers.py:338-360): the
  inference kernel forwards, one kernel backwards (the reversed recurrence
  with the derivatives of both sigmoids, of exp and of the clipped sqrt
  inside it); only y and the inputs are kept."""

  @staticmethod
  def forward(ctx, x, gx_pre, ga_pre, a_param, segment_pos, h0):
    x, gx_pre, ga_pre = x.contiguous(), gx_pre.contiguous(), ga_pre.contiguous()
    y, h_last, _ = ops.lru_scan_fused(x, gx_pre, ga_pre, a_param, segment_pos,
                                      h0=h0)
    ctx.save_for_backward(x, gx_pre, ga_pre, a_param, segment_pos == 0, y, h0)
    return y, h_last

  @staticmethod
  def backward(ctx, dy, dh_last):
    x, gx_pre, ga_pre, a_param, reset, y, h0 = ctx.saved_tensors
    dh = None if dh_last is None else dh_last.float().contiguous()
    dy = torch.zeros_like(y) if dy is None else dy.contiguous()
    dx, dgx, dga, dlam, dh0 = ops.rglru_backward(
        dy, x, gx_pre, ga_pre, a_param, reset, y, h0, dh)
    return dx, dgx, dga, dlam, None, dh0


def rg_lru(x, segment_pos, a_param, w_x, b_x, w_a, b_a, h0=None):
  """RGLRU.forward (layers.py:313-365) on kernels in both directions: the two
  gate projections (bf16; float32: batched products of the library), then
  everything after them.  Returns (y, h_last)."""
  if x.dim() == 3 and _projections_on_kernels(x):
    gx_pre, ga_pre = _GateProjections.apply(x, w_x, b_x, w_a, b_a)
  else:
    gx_pre = block_diag_linear(x, w_x, b_x)
    ga_pre = block_diag_linear(x, w_a, b_a)
  return _GatedScan.apply(x, gx_pre, ga_pre, a_param, segment_pos, h0)


def rg_lru_tensor_ops(x, segment_pos, a_param, w_x, b_x, w_a, b_a, h0=None):
  """The same as the reference's sequence of tensor ops under autograd, with
  only the recurrence on the scan kernel (the form rg_lru is tested against).
  Returns (y, h_last)."""
  reset = segment_pos == 0
  gate_x = torch.sigmoid(block_diag_linear_tensor_ops(x, w_x, b_x))
  gate_a = torch.sigmoid(block_diag_linear_tensor_ops(x, w_a, b_a))
  log_a = -8.0 * gate_a * torch.nn.functional.softplus(a_param)
  a = torch.exp(log_a)
  a_square = torch.exp(2 * log_a)
  gated_x = x * gate_x
  multiplier = _BoundedSqrt.apply(1 - a_square)
  multiplier = reset[..., None] + ~reset[..., None] * multiplier
  normalized_x = gated_x * multiplier.type(x.dtype)
  return rnn_scan(normalized_x, a, reset, h0)
