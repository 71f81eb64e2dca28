"""CPU oracle for the recurrent-block hot path (Conv1D + RG-LRU), in eager torch.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the smoke
check and the benchmark's CPU-baseline leg may import it; the shipped modules in
`recurrentgemma_amd/` never do and raise if the HIP library is missing.

Each function restates, op for op and in the same order, one function of the
reference's torch path so that in a low-precision activation dtype every
intermediate is rounded at the same point as in the reference:

  conv1d_forward         recurrentgemma/torch/layers.py:447-529 (+ helpers 531-636)
  block_diagonal_linear  recurrentgemma/torch/layers.py:127-137
  rnn_scan               recurrentgemma/torch/layers.py:140-191
  rglru_forward          recurrentgemma/torch/layers.py:313-365
  rnn_param_init         recurrentgemma/torch/layers.py:194-213
  conv1d_init_cache      recurrentgemma/torch/layers.py:638-650
  rglru_init_cache       recurrentgemma/torch/layers.py:367-376
  recurrent_core         the conv -> rg_lru part of
                         recurrentgemma/torch/modules.py:632-643

Three ways of evaluating them are used by the tests:
  * native: tensors in the activation dtype (fp32 or bf16) -- the reference's own
    arithmetic, rounding after every op;
  * widened ("oracle A"): bf16-valued inputs and parameters converted to fp32,
    every op in fp32, module outputs rounded back to bf16 (`widened_*` helpers);
  * truth: the same functions on fp64 tensors.

Pinning status (what fixes each function besides this restatement itself):
  conv1d_forward         F.conv1d special case, brute-force formula, per-document
                         invariance, golden vectors written from the reference
                         (tests/golden) incl. resets in the last two positions.
  block_diagonal_linear  torch.block_diag dense product, fp64 brute force, golden.
  rnn_scan               closed forms (geometric series, a=0, a=1), fp64 loop,
                         chunk associativity, golden.
  rglru_forward          zero-gate closed form, reset identity, prefill == prefill
                         o step, golden vectors (fp32 and the bf16 rounding order).
  rnn_param_init         algebraic identity + range, golden draws for fixed seeds.
"""

from __future__ import annotations

import math
from typing import NamedTuple

import torch
import torch.nn.functional as F


class CoreCache(NamedTuple):
  """Same field order as RecurrentBlockCache (torch/modules.py:32-37)."""

  rg_lru_state: torch.Tensor  # [B, W] float32
  conv1d_state: torch.Tensor  # [B, K-1, W] activation dtype


# --------------------------------------------------------------------------
# Conv1D
# --------------------------------------------------------------------------


def conv1d_init_cache(batch_size, width, dtype, temporal_width=4, device=None):
  return torch.zeros((batch_size, temporal_width - 1, width), dtype=dtype,
                     device=device)


def _left_pad_time(v: torch.Tensor, length: int) -> torch.Tensor:
  missing = length - v.shape[1]
  fill = torch.zeros((v.shape[0], missing, v.shape[2]), dtype=v.dtype,
                     device=v.device)
  return torch.cat([fill, v], dim=1)


def conv1d_forward(x, segment_pos, w, b, cache=None, return_cache=True,
                   mutate_input=False):
  """Causal depthwise temporal convolution with document masking.

  x [B,T,W], segment_pos [B,T] int, w [K,W], b [W], cache [B,K-1,W] or None.
  Returns (out [B,T,W], new_cache [B,K-1,W] | None).

  In prefill mode the reference multiplies slices of its input by the 0/1
  document mask IN PLACE (layers.py:497,508) and afterwards cuts the new cache
  out of that same tensor (layers.py:526), so the returned cache is masked.
  That is reproduced here; the caller's `x` is only touched when
  `mutate_input=True` (then it ends up modified exactly like the reference's).
  """
  k_width = w.shape[0]
  n_out = x.shape[1]
  if cache is not None:
    assert cache.shape == (x.shape[0], k_width - 1, x.shape[2])
    assert n_out == 1
    seq = torch.cat([cache.type(x.dtype), x], dim=1)
    n_before = k_width - 1
    cache_dtype = cache.dtype
  else:
    seq = x if mutate_input else x.clone()
    n_before = 0
    cache_dtype = x.dtype

  acc = 0.0
  for back in range(min(k_width, n_before + n_out)):
    lo = max(n_before - back, 0)
    hi = n_before + n_out - back
    piece = seq[:, lo:hi]
    if cache is None:
      inside_doc = (segment_pos != 0).type(torch.int32)
      keep = torch.ones((segment_pos.shape[0], hi - lo),
                        device=segment_pos.device)
      for ahead in range(1, back + 1):
        keep *= inside_doc[:, lo + ahead:hi + ahead]
      piece *= keep[:, :, None].type(x.dtype).to(device=x.device)  # in place
    piece = _left_pad_time(piece, n_out)
    acc += piece * w[k_width - back - 1][None, None, :]
  acc += b[None, None]

  if not return_cache:
    return acc, None
  tail = seq[:, 1 - k_width:].type(cache_dtype)
  return acc, _left_pad_time(tail, k_width - 1)


# --------------------------------------------------------------------------
# Block-diagonal linear
# --------------------------------------------------------------------------


def block_diagonal_linear(x, w, b):
  """x [..., H*bw], w [H,bw,bw] laid out [head, in, out], b [H,bw]."""
  heads, bw, _ = w.shape
  xs = x.reshape(*x.shape[:-1], heads, bw)
  ys = torch.einsum("... h i, h i j -> ... h j", xs, w) + b
  return ys.reshape(*x.shape[:-1], heads * bw)


# --------------------------------------------------------------------------
# Linear recurrence
# --------------------------------------------------------------------------


def rnn_scan(x, a, reset, h0, acc_dtype=torch.float32):
  """h_t = a_t h_{t-1} + x_t with fp32 state; a is zeroed at resets."""
  assert x.ndim == 3
  assert a.shape == x.shape[-a.ndim:]
  assert a.dtype == x.dtype
  assert h0 is None or h0.dtype == acc_dtype

  a = a * ~reset[..., None]

  if x.shape[1] == 1:
    if h0 is None:
      return x, x[:, 0].type(acc_dtype)
    y = a.type(acc_dtype) * h0[:, None] + x.type(acc_dtype)
    return y.type(x.dtype), y[:, -1]

  if h0 is not None:
    h = h0
  else:
    h = torch.zeros(x[:, 0].shape, dtype=acc_dtype, device=x.device)
  y = torch.zeros_like(x)
  for t in range(x.shape[1]):
    h = a[:, t].type(acc_dtype) * h + x[:, t].type(acc_dtype)
    y[:, t] = h.type(x.dtype)
  return y, h


def rnn_param_init(tensor, min_rad, max_rad, eps=1e-8):
  """Lambda such that exp(-softplus(Lambda)) is spread on a ring (in place)."""
  with torch.no_grad():
    tensor.uniform_(min_rad ** 2 + eps, max_rad ** 2 + eps)
    tensor.log_().mul_(0.5)
    return tensor.neg_().exp_().sub_(1.0).log_()


# --------------------------------------------------------------------------
# RG-LRU
# --------------------------------------------------------------------------


def rglru_init_cache(batch_size, width, device=None):
  return torch.zeros((batch_size, width), dtype=torch.float32, device=device)


def rglru_forward(x, segment_pos, a_param, w_x, b_x, w_a, b_a, cache=None,
                  return_cache=True, acc_dtype=torch.float32):
  """x [B,T,W] (the conv output), cache [B,W] acc_dtype or None.

  w_x/b_x: input gate, w_a/b_a: recurrence gate.  Returns (y, h_last | None).
  `acc_dtype` is float32 in the reference; the fp64 "truth" evaluation passes
  float64 so that the state is not narrowed.
  """
  bs, length, _ = x.shape
  assert segment_pos.shape == (bs, length)
  reset = segment_pos == 0

  gate_x = torch.sigmoid(block_diagonal_linear(x, w_x, b_x))
  gate_a = torch.sigmoid(block_diagonal_linear(x, w_a, b_a))

  log_a = -8.0 * gate_a * F.softplus(a_param)
  a = torch.exp(log_a)
  a_square = torch.exp(2 * log_a)

  gated_x = x * gate_x

  multiplier = torch.sqrt(1 - a_square)
  multiplier = reset[..., None] + ~reset[..., None] * multiplier
  normalized_x = gated_x * multiplier.type(x.dtype)

  y, last_h = rnn_scan(normalized_x, a, reset, cache, acc_dtype=acc_dtype)
  if not return_cache:
    return y, None
  return y, last_h


# --------------------------------------------------------------------------
# conv -> rg_lru, as RecurrentBlock.forward chains them (modules.py:632-643)
# --------------------------------------------------------------------------


def recurrent_core(x, segment_pos, params, cache: CoreCache | None = None,
                   return_cache=True):
  """params: dict with conv_w, conv_b, a_param, w_x, b_x, w_a, b_a."""
  xc, conv_state = conv1d_forward(
      x, segment_pos, params["conv_w"], params["conv_b"],
      cache=None if cache is None else cache.conv1d_state,
      return_cache=return_cache)
  y, h = rglru_forward(
      xc, segment_pos, params["a_param"], params["w_x"], params["b_x"],
      params["w_a"], params["b_a"],
      cache=None if cache is None else cache.rg_lru_state,
      return_cache=return_cache)
  if not return_cache:
    return y, None
  return y, CoreCache(rg_lru_state=h, conv1d_state=conv_state)


# --------------------------------------------------------------------------
# Widened evaluation ("oracle A"): low-precision values, fp32 arithmetic
# --------------------------------------------------------------------------


def _wide(t):
  return None if t is None else t.to(torch.float32)


def widened_conv1d_forward(x, segment_pos, w, b, cache=None, return_cache=True):
  out, new_cache = conv1d_forward(_wide(x), segment_pos, _wide(w), _wide(b),
                                  _wide(cache), return_cache)
  cache_dtype = x.dtype if cache is None else cache.dtype
  return out.to(x.dtype), (None if new_cache is None
                           else new_cache.to(cache_dtype))


def widened_rglru_forward(x, segment_pos, a_param, w_x, b_x, w_a, b_a,
                          cache=None, return_cache=True):
  y, h = rglru_forward(_wide(x), segment_pos, _wide(a_param), _wide(w_x),
                       _wide(b_x), _wide(w_a), _wide(b_a), cache, return_cache)
  return y.to(x.dtype), h


def widened_recurrent_core(x, segment_pos, params, cache=None,
                           return_cache=True):
  """Module boundaries (conv output, y) are rounded to the activation dtype."""
  xc, conv_state = widened_conv1d_forward(
      x, segment_pos, params["conv_w"], params["conv_b"],
      None if cache is None else cache.conv1d_state, return_cache)
  y, h = widened_rglru_forward(
      xc, segment_pos, params["a_param"], params["w_x"], params["b_x"],
      params["w_a"], params["b_a"],
      None if cache is None else cache.rg_lru_state, return_cache)
  if not return_cache:
    return y, None
  return y, CoreCache(rg_lru_state=h, conv1d_state=conv_state)


# --------------------------------------------------------------------------
# Parameter construction shared by tests and the benchmark
# --------------------------------------------------------------------------


def make_params(width, num_heads, dtype, seed, temporal_width=4,
                gate_bias_std=0.0):
  """Random parameters with the reference's initial distributions.

  conv w ~ N(0, 0.01/K) (layers.py:422-425), gate w ~ N(0, 1/bw)
  (layers.py:122-125), biases zero (optionally perturbed so that tests see a
  non-trivial bias), Lambda from rnn_param_init(0.9, 0.999) (layers.py:289-291).
  Drawn in fp32 from one seeded generator, then cast.
  """
  g = torch.Generator().manual_seed(seed)
  bw = width // num_heads
  p = {}
  p["conv_w"] = torch.randn(temporal_width, width, generator=g) * math.sqrt(
      0.01 / temporal_width)
  p["conv_b"] = torch.randn(width, generator=g) * gate_bias_std
  p["w_x"] = torch.randn(num_heads, bw, bw, generator=g) / math.sqrt(bw)
  p["b_x"] = torch.randn(num_heads, bw, generator=g) * gate_bias_std
  p["w_a"] = torch.randn(num_heads, bw, bw, generator=g) / math.sqrt(bw)
  p["b_a"] = torch.randn(num_heads, bw, generator=g) * gate_bias_std
  u = torch.rand(width, generator=g) * (0.999 ** 2 - 0.9 ** 2) + 0.9 ** 2 + 1e-8
  p["a_param"] = torch.log(torch.exp(-0.5 * torch.log(u)) - 1.0)
  return {k: v.to(dtype) for k, v in p.items()}
