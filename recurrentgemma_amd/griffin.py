"""The callers around the recurrent block: Griffin's residual stack.

Mirrors the module surface of recurrentgemma/torch/modules.py (attention
block :294-493, MLP block :683-760, residual block :763-932, embedder
:935-1003), recurrentgemma/torch/griffin.py:27-209 (model, cache dictionary
keyed "blocks.{i}") and the config types of recurrentgemma/common.py:22-190:
same constructor arguments, parameter names (reference state dicts load
unchanged), forward signatures and cache tuples.  On this package's kernels:
the recurrent block, RMSNorm (with the residual sums in front of it), the two
gelu(a) * b joins, the rotary embedding, the prompt attention and the decode
step of the attention block (bf16, head_dim 256), the linear layers of a
decode step of at most 64 rows, the logits' soft cap and the greedy pick.
Library calls: linear layers with more rows and the logits projection
(hipBLASLt), attention in other dtypes and head sizes
(scaled_dot_product_attention / batched products).  It exists so that the
recurrent path can be exercised and measured inside the model it belongs to.
Inference only (no autograd through the kernels).
"""

from __future__ import annotations

import enum
import itertools
import math
import functools
import weakref
from typing import Any, NamedTuple

import torch
from torch import nn

from recurrentgemma_amd import modules
from recurrentgemma_amd import ops

_MAX_WAVELENGTH = 10_000


@enum.unique
class TemporalBlockType(enum.Enum):
  ATTENTION = enum.auto()
  RECURRENT = enum.auto()


@enum.unique
class Preset(enum.Enum):
  """The published shapes (common.py:47-112)."""
  GRIFFIN_PAPER_7B = enum.auto()
  HAWK_PAPER_7B = enum.auto()
  RECURRENT_GEMMA_2B_V1 = enum.auto()
  RECURRENT_GEMMA_9B_V1 = enum.auto()

  @property
  def config_dict(self) -> dict[str, Any]:
    r, a = TemporalBlockType.RECURRENT, TemporalBlockType.ATTENTION

    def pattern(n):  # recurrent, recurrent, attention, ...
      return tuple(itertools.islice(itertools.cycle((r, r, a)), n))

    paper = dict(width=4096, mlp_expanded_width=3 * 4096, num_heads=32,
                 lru_width=5632, embeddings_scale_by_sqrt_dim=False,
                 attention_window_size=1024, logits_soft_cap=0.0)
    gemma = dict(embeddings_scale_by_sqrt_dim=True, attention_window_size=2048,
                 logits_soft_cap=30.0)
    if self is Preset.GRIFFIN_PAPER_7B:
      return dict(paper, block_types=pattern(32))
    if self is Preset.HAWK_PAPER_7B:
      return dict(paper, block_types=(r,) * 32)
    if self is Preset.RECURRENT_GEMMA_2B_V1:
      return dict(gemma, width=2560, mlp_expanded_width=3 * 2560, num_heads=10,
                  lru_width=2560, block_types=pattern(26))
    return dict(gemma, width=4096, mlp_expanded_width=3 * 4096, num_heads=16,
                lru_width=4096, block_types=pattern(38))


class GriffinConfig(NamedTuple):
  """common.py:115-190 without the Flax-only scan_type field."""
  vocab_size: int
  width: int
  mlp_expanded_width: int
  num_heads: int
  block_types: tuple[TemporalBlockType, ...]
  embeddings_scale_by_sqrt_dim: bool
  attention_window_size: int
  logits_soft_cap: float
  lru_width: int | None = None

  @property
  def max_cache_length(self) -> int:
    return self.attention_window_size

  @property
  def num_layers(self) -> int:
    return len(self.block_types)

  @classmethod
  def from_preset(cls, preset: Preset, vocab_size: int = 256_000,
                  max_sequence_length: int | None = None) -> "GriffinConfig":
    kw = preset.config_dict
    if max_sequence_length is not None:
      kw["attention_window_size"] = min(kw["attention_window_size"],
                                        max_sequence_length)
    return cls(vocab_size=vocab_size, **kw)


class AttentionBlockCache(NamedTuple):
  keys: torch.Tensor        # [B, window, 1, head_dim], ring buffer
  values: torch.Tensor      # [B, window, 1, head_dim]
  num_tokens: torch.Tensor  # [B] int32, tokens seen so far


ResidualBlockCache = modules.RecurrentBlockCache | AttentionBlockCache
Cache = dict[str, ResidualBlockCache]


class RMSNorm(nn.Module):
  """x / rms(x) * (1 + scale)  (layers.py:30-73); scale starts at zero."""

  def __init__(self, width, eps=1e-6, device=None, dtype=None):
    super().__init__()
    self.width = width
    self.eps = eps
    self.scale = nn.Parameter(torch.empty([width], device=device, dtype=dtype))
    self.reset_parameters()

  def reset_parameters(self) -> None:
    torch.nn.init.zeros_(self.scale)

  def forward(self, x):
    # one kernel; every step rounded to the activation dtype like the
    # reference's chain of tensor ops
    return ops.rms_norm(x, self.scale, self.eps)

  def add_then_norm(self, x, addend):
    """(x + addend, forward(x + addend)) in one kernel.  x may be an
    ops.PartialSums (a layer output not added up yet; addend may then be None
    or ride in x)."""
    return ops.add_rms_norm(x, addend, self.scale, self.eps)


class _StackedLinear(nn.Module):
  """Two width -> expanded projections with stacked parameters `w`
  [2, width, expanded] and `b` [2, 1, 1, expanded]: the parameters of the
  reference's `Einsum("...td,cdD->c...tD")` (layers.py:653-703) under the same
  names."""

  def __init__(self, width, expanded, device=None, dtype=None):
    super().__init__()
    self.w_shape = (2, width, expanded)
    self.w = nn.Parameter(torch.empty(self.w_shape, device=device, dtype=dtype))
    self.b = nn.Parameter(
        torch.empty((2, 1, 1, expanded), device=device, dtype=dtype))
    self.reset_parameters()

  def reset_parameters(self) -> None:
    torch.nn.init.normal_(self.w, mean=0.0,
                          std=math.sqrt(1.0 / self.w_shape[1]))
    torch.nn.init.zeros_(self.b)

  def forward(self, x):
    lead = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1])
    if x2.shape[0] <= 1024:
      # few rows (decode): both projections as one batched product on the
      # stacked parameters, half the launches
      out = torch.baddbmm(self.b.reshape(2, 1, -1),
                          x2[None].expand(2, -1, -1), self.w)
      gate, up = out[0], out[1]
    else:
      gate = torch.addmm(self.b[0].reshape(-1), x2, self.w[0])
      up = torch.addmm(self.b[1].reshape(-1), x2, self.w[1])
    return gate.reshape(*lead, -1), up.reshape(*lead, -1)


class MLPBlock(nn.Module):
  """gelu(x W0 + b0) * (x W1 + b1) -> ffw_down  (modules.py:683-760)."""

  def __init__(self, width, expanded_width, final_w_init_variance_scale=1.0,
               device=None, dtype=None):
    super().__init__()
    self.width = width
    self.expanded_width = expanded_width
    self.final_w_init_variance_scale = final_w_init_variance_scale
    self.ffw_up = _StackedLinear(width, expanded_width, device=device,
                                 dtype=dtype)
    self.ffw_down = nn.Linear(expanded_width, width, device=device, dtype=dtype)
    # for at most 64 rows (a decode step): up-projections, gelu and product in
    # one pass over the stacked weight; down-projection with the residual add
    self._rows_up = ops.PackedLinear(layout=1, gelu_pair=True)
    self._rows_down = ops.PackedLinear()
    self.reset_parameters()

  def reset_parameters(self) -> None:
    self.ffw_up.reset_parameters()
    std = math.sqrt(self.final_w_init_variance_scale / self.expanded_width)
    torch.nn.init.normal_(self.ffw_down.weight, mean=0.0, std=std)
    torch.nn.init.zeros_(self.ffw_down.bias)

  def forward(self, x, residual=None, defer_out=False):
    """residual: added to the result (the block's skip connection,
    modules.py:897-898).  defer_out: the caller normalises the result next and
    accepts it as ops.PartialSums or ops.PendingSum (returned where that saves
    a pass)."""
    if (ops.PackedLinear.usable(x, self.width, 2 * self.expanded_width, True)
        and ops.PackedLinear.usable(x, self.expanded_width, self.width)):
      hidden = self._rows_up(x, (self.ffw_up.w,), (self.ffw_up.b,))
      if defer_out and ops.PackedLinear.partial_slices(
          hidden, self.expanded_width, self.width):
        return self._rows_down.partial(hidden, (self.ffw_down.weight,),
                                       (self.ffw_down.bias,), addend=residual)
      return self._rows_down(hidden, (self.ffw_down.weight,),
                             (self.ffw_down.bias,), residual=residual)
    gate, up = self.ffw_up(x)
    out = self.ffw_down(ops.gelu_mul(up, gate))  # gelu(gate) * up, one pass
    if residual is None:
      return out
    # (many rows: the norm that reads the sum next adds the two in its pass)
    return ops.PendingSum(out, residual) if defer_out else out + residual


def _inv_frequencies(head_dim, device, max_wavelength=_MAX_WAVELENGTH):
  """1 / max_wavelength^(2i / half) for the i-th rotated pair, with the
  reference's own tensor expression (modules.py:70-73) so that the table has
  its float32 values."""
  half = head_dim // 2
  freq = torch.arange(half // 2, device=device)
  return 1.0 / (max_wavelength ** (2 * freq / half))


def _visible(q_pos, k_pos, window, q_doc=None, k_doc=None):
  """[B, Tq, Tk] mask (modules.py:86-127): keys not after the query, at most
  `window` positions back, in the same document (or, without document ids, at
  a real position >= 0)."""
  q, k = q_pos[..., :, None], k_pos[..., None, :]
  mask = (q >= k) & (q <= k + window)
  if q_doc is not None:
    return mask & (q_doc[..., :, None] == k_doc[..., None, :])
  return mask & (k >= 0)


def _inference_only(forward):
  """The residual stack around the recurrent block runs without an autograd
  graph (its few-row linear layers, attention and normalisation kernels have
  no backward pass).  Called the way the reference's own tests call it --
  constructed, not switched to eval(), gradients enabled
  (recurrentgemma/torch/griffin_test.py, modules_test.py) -- it simply
  computes, under no_grad.  A caller that asks for gradients through it --
  inside training.differentiable(), or with an input tensor that requires
  grad -- gets an error instead of silently detached tensors."""

  @functools.wraps(forward)
  def wrapper(self, *args, **kwargs):
    from recurrentgemma_amd import training
    wants_grad = training.is_enabled() or (
        torch.is_grad_enabled() and any(
            isinstance(a, torch.Tensor) and a.requires_grad
            for a in itertools.chain(args, kwargs.values())))
    if wants_grad:
      raise NotImplementedError(
          f"{type(self).__name__} is forward only: no gradient flows through "
          "it (only RecurrentBlock, Conv1D and RGLRU have a differentiable "
          "path, inside training.differentiable())")
    with torch.no_grad():
      return forward(self, *args, **kwargs)

  return wrapper


_first_key = [None, None, None, None]  # tensor (weak), version, window, answer


def _first_visible_key(segment_pos, window):
  """[B, T] int32: the first key each query of a prompt sees -- the later of
  the first token of its document (the latest position with segment_pos == 0,
  else the start of the row) and `window` tokens back: what the mask of
  modules.py:86-127 amounts to for a prompt.  Kept for the tensor object it
  was computed for (the attention blocks of a model all ask for the same)."""
  ref, version, w, answer = _first_key
  now = None if segment_pos.is_inference() else segment_pos._version
  if (ref is not None and ref() is segment_pos and now is not None and
      version == now and w == window):
    return answer
  b, t = segment_pos.shape
  pos = torch.arange(t, device=segment_pos.device)[None].expand(b, t)
  start = torch.cummax(
      torch.where(segment_pos == 0, pos, torch.zeros_like(pos)), dim=-1).values
  answer = torch.maximum(start, pos - window).to(torch.int32).contiguous()
  _first_key[:] = [weakref.ref(segment_pos), now, window, answer]
  return answer


_one_document = [None, None, False]  # tensor (weak), its version, answer


def _rows_are_one_document(segment_pos) -> bool:
  """True if no row starts a document after its first token: every row is then
  one document (or the tail of one) and its mask is the plain causal one.
  Asking costs a host synchronisation, so the answer is kept for the tensor
  object it was given for (the blocks of a model all ask about the same one)."""
  ref, version, answer = _one_document
  # (inference-mode tensors keep no version counter: asked again every time)
  now = None if segment_pos.is_inference() else segment_pos._version
  if (ref is not None and ref() is segment_pos and now is not None and
      version == now):
    return answer
  answer = bool((segment_pos[:, 1:] != 0).all())
  _one_document[:] = [weakref.ref(segment_pos), now, answer]
  return answer


class LocalAttentionBlock(nn.Module):
  """Sliding-window multi-query attention with a ring KV cache
  (modules.py:294-493)."""

  def __init__(self, width, num_heads, window_size,
               final_w_init_variance_scale=1.0, device=None, dtype=None):
    super().__init__()
    self.width = width
    self.num_heads = num_heads
    self.window_size = window_size
    self.final_w_init_variance_scale = final_w_init_variance_scale
    kw = dict(device=device, dtype=dtype)
    self.proj_q = nn.Linear(width, width, bias=False, **kw)
    self.proj_k = nn.Linear(width, self.head_dim, bias=False, **kw)
    self.proj_v = nn.Linear(width, self.head_dim, bias=False, **kw)
    self.proj_final = nn.Linear(width, width, bias=True, **kw)
    # the projections for at most 64 rows (a decode step)
    self._rows_q = ops.PackedLinear()
    self._rows_kv = ops.PackedLinear()
    self._rows_qkv = ops.PackedLinear()  # a decode step: one launch for all
    self._rows_final = ops.PackedLinear()
    self._inv_freq = None
    self.reset_parameters()

  @property
  def head_dim(self) -> int:
    return self.width // self.num_heads

  def reset_parameters(self) -> None:
    for proj in (self.proj_q, self.proj_k, self.proj_v):
      torch.nn.init.normal_(proj.weight, mean=0.0,
                            std=math.sqrt(1.0 / self.width))
    std = math.sqrt(self.final_w_init_variance_scale / self.width)
    torch.nn.init.normal_(self.proj_final.weight, mean=0.0, std=std)
    torch.nn.init.zeros_(self.proj_final.bias)

  @staticmethod
  def _cache_from_prompt(keys, values, segment_pos, window):
    """Ring buffer filled from a prompt (modules.py:253-283): the last
    min(window, T) tokens, token with position p in slot p % window when the
    prompt fills the window."""
    w = min(window, keys.shape[1])
    # int32 like init_cache (the reference keeps the dtype of segment_pos)
    num_tokens = (segment_pos[:, -1] + 1).to(torch.int32)
    shift = (num_tokens % window)[:, None]
    src = (torch.arange(w, device=keys.device)[None] - shift) % w  # [B, w]

    def place(x):
      tail = x[:, -w:]
      idx = src[:, :, None, None].expand(-1, -1, *tail.shape[2:])
      out = torch.gather(tail, 1, idx)
      if w < window:
        pad = out.new_zeros(out.shape[0], window - w, *out.shape[2:])
        out = torch.cat([out, pad], dim=1)
      return out

    return AttentionBlockCache(keys=place(keys), values=place(values),
                               num_tokens=num_tokens)

  @_inference_only
  def forward(self, x, segment_pos, cache=None, return_cache=True,
              defer_out=False):
    """defer_out: as for RecurrentBlock.forward."""
    b, t, _ = x.shape
    assert segment_pos.shape == (b, t), segment_pos.shape
    if self._inv_freq is None or self._inv_freq.device != x.device:
      self._inv_freq = _inv_frequencies(self.head_dim, x.device)
    if (cache is not None and t == 1 and
        ops.PackedLinear.usable(x, self.width,
                                self.width + 2 * self.head_dim) and
        ops.attention_decode_fused_supported(
            x, self.num_heads, self.head_dim, self.window_size)):
      return self._decode_step_fused(x, segment_pos, cache, return_cache,
                                     defer_out)
    few_rows = (ops.PackedLinear.usable(x, self.width, self.width) and
                ops.PackedLinear.usable(x, self.width, 2 * self.head_dim))
    if few_rows:
      q = self._rows_q(x, (self.proj_q.weight,))
      k, v = self._rows_kv(x, (self.proj_k.weight, self.proj_v.weight))
    else:
      q, k, v = self.proj_q(x), self.proj_k(x), self.proj_v(x)
    q = q.reshape(b, t, self.num_heads, self.head_dim)
    k = k.reshape(b, t, 1, self.head_dim)
    v = v.reshape(b, t, 1, self.head_dim)
    # rotary embedding of queries and keys (modules.py:431-432), one kernel
    q, k = ops.rope_pair(q, k, segment_pos, self._inv_freq)

    if cache is not None and t == 1:
      return self._decode_step(x, q, k, v, cache, return_cache, defer_out)

    new_cache = None
    if cache is not None:
      w = self.window_size
      k_pos, q_pos = self._ring_positions(cache.num_tokens, t)
      mask = _visible(q_pos, torch.cat([k_pos, q_pos], dim=-1), w)
      k_all = torch.cat([cache.keys, k], dim=1)
      v_all = torch.cat([cache.values, v], dim=1)
      if return_cache:
        if t >= w:
          new_cache = self._cache_from_prompt(k, v, segment_pos, w)
        else:
          raise NotImplementedError(
              "a cached call takes one token or at least a window of them")
    else:
      k_all, v_all = k, v
      if return_cache:
        new_cache = self._cache_from_prompt(k, v, segment_pos,
                                            self.window_size)
      if ops.attention_prefill_supported(q):
        # bf16, head_dim 256: scores, mask, softmax and values in one kernel
        # (the mask of modules.py:86-127 for a prompt is a band: a query sees
        # from the start of its document, or the window's width back, up to
        # itself)
        out = ops.attention_prefill(
            q, k, v, _first_visible_key(segment_pos, self.window_size),
            self.head_dim ** -0.5)
        return self._project_out(out.reshape(b, t, self.width),
                                 defer_out), new_cache
      if (x.is_cuda and 1 < t <= self.window_size + 1 and
          _rows_are_one_document(segment_pos)):
        # one document per row, all of it inside the window: the mask of
        # modules.py:86-127 is the causal one, which the library's attention
        # kernel applies by itself (4 ms instead of 17 ms per block at
        # 64 x 2047 tokens, where the mask is 268 MB to build and to read)
        out = nn.functional.scaled_dot_product_attention(
            q.transpose(1, 2),
            k.transpose(1, 2).expand(-1, self.num_heads, -1, -1),
            v.transpose(1, 2).expand(-1, self.num_heads, -1, -1),
            is_causal=True)
        out = out.transpose(1, 2).reshape(b, t, self.width)
        return self._project_out(out, defer_out), new_cache
      doc = torch.cumsum(segment_pos == 0, dim=-1)
      pos = torch.arange(t, device=x.device)[None].expand(b, t)
      mask = _visible(pos, pos, self.window_size, doc, doc)

    # [B, heads, T, head_dim] against one shared key/value head
    out = nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2),
        k_all.transpose(1, 2).expand(-1, self.num_heads, -1, -1),
        v_all.transpose(1, 2).expand(-1, self.num_heads, -1, -1),
        attn_mask=mask[:, None])
    out = out.transpose(1, 2).reshape(b, t, self.width)
    return self._project_out(out, defer_out), new_cache

  def _project_out(self, x, defer_out=False):
    weights, biases = (self.proj_final.weight,), (self.proj_final.bias,)
    if defer_out and ops.PackedLinear.partial_slices(x, self.width, self.width):
      return self._rows_final.partial(x, weights, biases)
    if ops.PackedLinear.usable(x, self.width, self.width):
      return self._rows_final(x, weights, biases)
    return self.proj_final(x)

  def _ring_positions(self, num_tokens, t):
    """Positions held by the ring (slot j keeps the largest position congruent
    to j that is below num_tokens; negative = never written) and positions of
    the t new tokens (modules.py:152-183)."""
    w = self.window_size
    n = num_tokens[:, None]
    now = torch.arange(w, device=n.device)[None] + (n // w) * w
    k_pos = torch.where(now < n, now, now - w)
    q_pos = torch.arange(t, device=n.device)[None] + n
    return k_pos, q_pos

  def _decode_step_fused(self, x, segment_pos, cache, return_cache,
                         defer_out=False):
    """One new token (bf16, head_dim 256) in three launches: the three
    projections as one pass over their weights, then rotary embedding, scores
    against the ring as it lies, mask, softmax, values, the new token's own
    share, ring update and token count as one call that reads the ring once
    (rg_attention_decode_fused), then proj_final.  Roundings as in
    _decode_step, except that the probabilities enter the second product
    unnormalised."""
    b = x.shape[0]
    if cache.num_tokens.dtype != torch.int32:
      raise TypeError("AttentionBlockCache.num_tokens must be int32")
    qkv = self._rows_qkv(
        x, (self.proj_q.weight, self.proj_k.weight, self.proj_v.weight))
    qkv = qkv.reshape(b, self.width + 2 * self.head_dim)
    out = ops.attention_decode_fused(
        qkv[:, :self.width], qkv[:, self.width:self.width + self.head_dim],
        qkv[:, self.width + self.head_dim:], segment_pos, self._inv_freq,
        cache.keys, cache.values, cache.num_tokens, self.head_dim ** -0.5,
        update_cache=return_cache)
    out = self._project_out(out.reshape(b, 1, self.width), defer_out)
    return out, (cache if return_cache else None)

  def _decode_step(self, x, q, k, v, cache, return_cache, defer_out=False):
    """One new token against the ring and itself, without concatenating or
    expanding the cached keys and values: all heads share them, so the scores
    are one batched [heads, head_dim] x [head_dim, window] product per row on
    the cache as it lies.  Scaling, mask, softmax and the new token's own
    score are one kernel; the new token's share of the output, the ring update
    and the token count another.  Same order of roundings as the reference:
    scores in the activation dtype, scaled, masked, softmax in float32,
    probabilities back in the activation dtype (modules.py:462-474)."""
    b = x.shape[0]
    w = self.window_size
    if cache.num_tokens.dtype != torch.int32:
      raise TypeError("AttentionBlockCache.num_tokens must be int32")
    qh = q[:, 0]                                           # [B, heads, hd]
    ring_k, ring_v = cache.keys[:, :, 0], cache.values[:, :, 0]  # [B, w, hd]
    scores = torch.bmm(qh, ring_k.transpose(1, 2))         # [B, heads, w]
    probs = ops.attention_decode_probs(scores, qh, k[:, 0, 0],
                                       cache.num_tokens, self.head_dim ** -0.5)
    from_ring = torch.bmm(probs[..., :w], ring_v)
    out = ops.attention_decode_finish(
        from_ring, probs, k[:, 0, 0], v[:, 0, 0], cache.keys, cache.values,
        cache.num_tokens, update_cache=return_cache)
    out = self._project_out(out.reshape(b, 1, self.width), defer_out)
    return out, (cache if return_cache else None)

  @classmethod
  def init_cache(cls, batch_size, window_size, heads_dim, dtype, device=None):
    shape = (batch_size, window_size, 1, heads_dim)
    return AttentionBlockCache(
        keys=torch.zeros(shape, device=device, dtype=dtype),
        values=torch.zeros(shape, device=device, dtype=dtype),
        num_tokens=torch.zeros([batch_size], dtype=torch.int32, device=device))


class ResidualBlock(nn.Module):
  """norm -> temporal block -> +x -> norm -> MLP -> +  (modules.py:763-932)."""

  def __init__(self, width, mlp_expanded_width, num_heads,
               attention_window_size, temporal_block_type, lru_width=None,
               conv1d_temporal_width=4, final_w_init_variance_scale=1.0,
               device=None, dtype=None):
    super().__init__()
    self.width = width
    self.mlp_expanded_width = mlp_expanded_width
    self.num_heads = num_heads
    self.attention_window_size = attention_window_size
    self.temporal_block_type = temporal_block_type
    self.lru_width = lru_width
    self.conv1d_temporal_width = conv1d_temporal_width
    self.final_w_init_variance_scale = final_w_init_variance_scale
    kw = dict(device=device, dtype=dtype)
    self.temporal_pre_norm = RMSNorm(width, **kw)
    if temporal_block_type is TemporalBlockType.RECURRENT:
      self.recurrent_block = modules.RecurrentBlock(
          width=width, num_heads=num_heads, lru_width=lru_width,
          conv1d_temporal_width=conv1d_temporal_width,
          final_w_init_variance_scale=final_w_init_variance_scale, **kw)
    else:
      self.attention_block = LocalAttentionBlock(
          width=width, num_heads=num_heads, window_size=attention_window_size,
          final_w_init_variance_scale=final_w_init_variance_scale, **kw)
    self.channel_pre_norm = RMSNorm(width, **kw)
    self.mlp_block = MLPBlock(
        width=width, expanded_width=mlp_expanded_width,
        final_w_init_variance_scale=final_w_init_variance_scale, **kw)

  @property
  def temporal_block(self) -> nn.Module:
    if self.temporal_block_type is TemporalBlockType.RECURRENT:
      return self.recurrent_block
    return self.attention_block

  def reset_parameters(self) -> None:
    self.temporal_pre_norm.reset_parameters()
    self.temporal_block.reset_parameters()
    self.channel_pre_norm.reset_parameters()
    self.mlp_block.reset_parameters()

  @_inference_only
  def forward(self, x, segment_pos, cache=None, return_cache=True,
              defer_out=False):
    """x and, with defer_out, the result may be ops.PartialSums: the output of
    the previous block's last layer before its slices of K are added, which
    the norm kernel that reads it next does (Griffin.forward chains the blocks
    that way for a decode step) -- or, with many rows, ops.PendingSum: that
    output and the skip connection before they are added."""
    if isinstance(x, ops.PartialSums):
      x, normed = self.temporal_pre_norm.add_then_norm(x, None)
    elif isinstance(x, ops.PendingSum):
      x, normed = self.temporal_pre_norm.add_then_norm(x.a, x.b)
    else:
      normed = self.temporal_pre_norm(x)
    mixed, new_cache = self.temporal_block(normed, segment_pos, cache,
                                           return_cache=return_cache,
                                           defer_out=True)
    residual, normed = self.channel_pre_norm.add_then_norm(mixed, x)
    return (self.mlp_block(normed, residual=residual, defer_out=defer_out),
            new_cache)

  @classmethod
  def init_cache(cls, batch_size, width, num_heads, attention_window_size,
                 temporal_block_type, dtype, lru_width=None,
                 conv1d_temporal_width=4, device=None):
    if temporal_block_type is TemporalBlockType.RECURRENT:
      return modules.RecurrentBlock.init_cache(
          batch_size=batch_size, lru_width=lru_width or width, dtype=dtype,
          conv1d_temporal_width=conv1d_temporal_width, device=device)
    return LocalAttentionBlock.init_cache(
        batch_size=batch_size, window_size=attention_window_size,
        heads_dim=width // num_heads, dtype=dtype, device=device)


class Embedder(nn.Module):
  """Token table used for both the input embedding and the output logits
  (modules.py:935-1003)."""

  def __init__(self, vocab_size, embed_dim, scale_by_sqrt_dim, device=None,
               dtype=None):
    super().__init__()
    self.vocab_size = vocab_size
    self.embed_dim = embed_dim
    self.scale_by_sqrt_dim = scale_by_sqrt_dim
    self.input_embedding = nn.Parameter(
        torch.empty([vocab_size, embed_dim], device=device, dtype=dtype))
    self.reset_parameters()

  def reset_parameters(self) -> None:
    torch.nn.init.normal_(self.input_embedding, mean=0.0,
                          std=math.sqrt(1.0 / self.embed_dim))

  def encode(self, tokens):
    x = self.input_embedding[(tokens,)]
    if self.scale_by_sqrt_dim:
      # the factor is rounded to bfloat16 whatever the model dtype
      x = x * torch.tensor(math.sqrt(self.embed_dim)).type(torch.bfloat16)
    return x

  def decode(self, x):
    return x @ self.input_embedding.T


class Griffin(nn.Module):
  """Embedder -> residual blocks -> final norm -> logits (soft-capped)
  (griffin.py:27-209)."""

  def __init__(self, config: GriffinConfig, gradient_checkpointing=True,
               device=None, dtype=None):
    super().__init__()
    self.config = config
    # accepted for signature compatibility; this build is inference only and
    # never checkpoints
    self.gradient_checkpointing = gradient_checkpointing
    self.embedder = Embedder(
        vocab_size=config.vocab_size, embed_dim=config.width,
        scale_by_sqrt_dim=config.embeddings_scale_by_sqrt_dim, device=device,
        dtype=dtype)
    self.blocks = nn.ModuleList([
        ResidualBlock(
            width=config.width, mlp_expanded_width=config.mlp_expanded_width,
            num_heads=config.num_heads,
            attention_window_size=config.attention_window_size,
            temporal_block_type=kind, lru_width=config.lru_width,
            final_w_init_variance_scale=2.0 / config.num_layers, device=device,
            dtype=dtype) for kind in config.block_types])
    self.final_norm = RMSNorm(config.width, device=device, dtype=dtype)

  def reset_parameters(self) -> None:
    self.embedder.reset_parameters()
    for block in self.blocks:
      block.reset_parameters()
    self.final_norm.reset_parameters()

  @_inference_only
  def forward(self, tokens, segment_pos, cache: Cache | None = None,
              return_logits=True, return_cache=True):
    if not return_logits and not return_cache:
      return None, None
    x = self.embedder.encode(tokens)
    new_cache = {}
    for i, block in enumerate(self.blocks):
      name = f"blocks.{i}"
      x, new_cache[name] = block(x, segment_pos,
                                 None if cache is None else cache[name],
                                 return_cache=return_cache,
                                 defer_out=return_logits or
                                 i + 1 < len(self.blocks))
    if not return_logits:
      return None, new_cache
    if isinstance(x, ops.PartialSums):
      x = self.final_norm.add_then_norm(x, None)[1]
    elif isinstance(x, ops.PendingSum):
      x = self.final_norm.add_then_norm(x.a, x.b)[1]
    else:
      x = self.final_norm(x)
    logits = self.embedder.decode(x)
    cap = self.config.logits_soft_cap
    if cap:
      logits = ops.soft_cap(logits, cap)
    return logits, (new_cache if return_cache else None)

  def init_cache(self, batch_size, dtype, device=None) -> Cache:
    c = self.config
    if device is None:
      device = self.embedder.input_embedding.device
    return {
        f"blocks.{i}": ResidualBlock.init_cache(
            batch_size=batch_size, width=c.width, num_heads=c.num_heads,
            attention_window_size=c.attention_window_size,
            temporal_block_type=kind, dtype=dtype, lru_width=c.lru_width,
            device=device) for i, kind in enumerate(c.block_types)}
