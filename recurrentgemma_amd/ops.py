"""Functional front-end of the C ABI on torch tensors (device memory + stream).

Every function checks shapes/dtypes/devices on the host, allocates the outputs
with torch's caching allocator, and enqueues the kernels on torch's current
HIP stream.  Nothing here computes on the CPU.
"""

from __future__ import annotations

import torch

from recurrentgemma_amd import _lib

_DTYPES = {torch.float32: _lib.RG_DTYPE_F32, torch.bfloat16: _lib.RG_DTYPE_BF16}


def _dtype_code(t: torch.Tensor) -> int:
  if t.dtype not in _DTYPES:
    raise TypeError(
        f"recurrentgemma_amd kernels support float32 and bfloat16, got {t.dtype}")
  return _DTYPES[t.dtype]


def _dev(t: torch.Tensor, name: str, in_place: bool = False) -> torch.Tensor:
  """Contiguous, 16-byte aligned, on a GPU; raises instead of computing on CPU.

  A tensor that is not contiguous or not aligned is copied -- unless the call
  updates it in place (in_place): the kernel would then write to the copy and
  the caller's tensor would go stale, so that case raises."""
  if not t.is_cuda:
    raise RuntimeError(
        f"{name} is on {t.device}: recurrentgemma_amd runs on the GPU only "
        "(there is no CPU fallback)")
  if in_place:
    if not t.is_contiguous() or t.data_ptr() % 16:
      raise ValueError(f"{name} must be a contiguous, 16-byte aligned GPU "
                       "tensor (it is updated in place)")
    return t
  t = t.contiguous()
  if t.data_ptr() % 16:
    t = t.clone(memory_format=torch.contiguous_format)
  return t


def _same(dtype, device, **tensors):
  for name, t in tensors.items():
    if t is None:
      continue
    if t.dtype != dtype:
      raise TypeError(f"{name} has dtype {t.dtype}, expected {dtype} "
                      "(parameters and activations must share one dtype)")
    if t.device != device:
      raise RuntimeError(f"{name} is on {t.device}, expected {device}")


def _segpos(segment_pos: torch.Tensor, B: int, T: int):
  assert segment_pos.shape == (B, T), (
      f"segment_pos has shape {tuple(segment_pos.shape)}, expected {(B, T)}")
  if segment_pos.dtype not in (torch.int32, torch.int64):
    if segment_pos.dtype.is_floating_point or segment_pos.dtype == torch.bool:
      raise TypeError(f"segment_pos must be an integer tensor, got "
                      f"{segment_pos.dtype}")
    segment_pos = segment_pos.to(torch.int64)
  return _dev(segment_pos, "segment_pos"), int(segment_pos.dtype == torch.int64)


def _stream(t: torch.Tensor) -> int:
  # (the raw handle: current_stream() builds a Stream object per call, which
  # is a microsecond of a decode step's host time)
  return torch._C._cuda_getCurrentRawStream(t.device.index)


class _NoGuard:
  def __enter__(self):
    return None

  def __exit__(self, *exc):
    return False


_NO_GUARD = _NoGuard()


def _on(device):
  """Context that makes `device` the current one for a launch; free when it
  already is (entering torch.cuda.device costs more than the rest of the
  argument handling of a small call)."""
  if torch.cuda.current_device() == device.index:
    return _NO_GUARD
  return torch.cuda.device(device)


def _p(t):
  return None if t is None else t.data_ptr()


def _empty_prefill(x, h0, return_h, return_conv_cache, taps=3):
  """What the reference returns for no tokens (or no rows): nothing to
  compute, the state stays what it was (layers.py:181-189 with an empty loop,
  :526-527 a conv state padded with zeros)."""
  B, _, W = x.shape
  h = None
  if return_h:
    h = (h0.clone() if h0 is not None else
         torch.zeros((B, W), dtype=torch.float32, device=x.device))
  cache = x.new_zeros((B, taps, W)) if return_conv_cache else None
  return torch.empty_like(x), h, cache


def conv1d_prefill(x, segment_pos, w, b, return_cache=True):
  assert x.ndim == 3, f"x must be [B,T,W], got {tuple(x.shape)}"
  B, T, W = x.shape
  K = w.shape[0]
  assert w.shape == (K, W) and b.shape == (W,)
  x = _dev(x, "x")
  _same(x.dtype, x.device, w=w, b=b)
  if x.numel() == 0:
    out, _, cache = _empty_prefill(x, None, False, return_cache, K - 1)
    return out, cache
  w, b = _dev(w, "w"), _dev(b, "b")
  seg, is64 = _segpos(segment_pos, B, T)
  out = torch.empty_like(x)
  cache = x.new_empty((B, K - 1, W)) if return_cache else None
  with _on(x.device):
    _lib.check(_lib.lib().rg_conv1d_prefill(
        _p(x), _p(seg), is64, _p(w), _p(b), _p(out), _p(cache), B, T, W, K,
        _dtype_code(x), _stream(x)))
  return out, cache


def conv1d_backward(dout, x, segment_pos, w):
  """Gradients of conv1d_prefill: (dx, dw, db) from the gradient of its
  output; one kernel and a sum over its per-chunk partial sums."""
  B, T, W = x.shape
  K = w.shape[0]
  assert w.shape == (K, W) and dout.shape == x.shape
  x = _dev(x, "x")
  _same(x.dtype, x.device, dout=dout, w=w)
  dout, w = _dev(dout, "dout"), _dev(w, "w")
  seg, is64 = _segpos(segment_pos, B, T)
  lib = _lib.lib()
  need = lib.rg_conv1d_backward_workspace_bytes(B, T, W, K)
  partial = torch.empty(need // 4, dtype=torch.float32, device=x.device)
  dx = torch.empty_like(x)
  with _on(x.device):
    _lib.check(lib.rg_conv1d_backward(
        _p(dout), _p(x), _p(seg), is64, _p(w), _p(dx), _p(partial), need, B, T,
        W, K, _dtype_code(x), _stream(x)))
  sums = partial.view(-1, K + 1, W).sum(0)
  return dx, sums[:K].to(w.dtype), sums[K].to(w.dtype)


def conv1d_step(x, cache, w, b, return_cache=True):
  B, n_tok, W = x.shape
  K = w.shape[0]
  assert cache.shape == (B, K - 1, W)
  assert n_tok == 1
  x = _dev(x, "x")
  _same(x.dtype, x.device, w=w, b=b)
  w, b = _dev(w, "w"), _dev(b, "b")
  cache_in = _dev(cache.to(x.dtype), "cache")
  out = torch.empty_like(x)
  new_cache = torch.empty_like(cache_in) if return_cache else None
  with _on(x.device):
    _lib.check(_lib.lib().rg_conv1d_step(
        _p(x), _p(cache_in), _p(w), _p(b), _p(out), _p(new_cache), B, W, K,
        _dtype_code(x), _stream(x)))
  if new_cache is not None and new_cache.dtype != cache.dtype:
    new_cache = new_cache.to(cache.dtype)
  return out, new_cache


def block_diag_linear(x, w, b):
  H, bw, bw2 = w.shape
  assert bw == bw2 and b.shape == (H, bw)
  assert x.shape[-1] == H * bw, (
      f"last dim {x.shape[-1]} != num_blocks*block_width {H * bw}")
  x = _dev(x, "x")
  _same(x.dtype, x.device, w=w, b=b)
  w, b = _dev(w, "w"), _dev(b, "b")
  y = torch.empty_like(x)
  M = x.numel() // (H * bw)
  if M == 0:
    return y
  with _on(x.device):
    _lib.check(_lib.lib().rg_block_diag_linear(
        _p(x), _p(w), _p(b), _p(y), M, H, bw, _dtype_code(x), _stream(x)))
  return y


def gates_gemm(x, w_x, b_x, w_a, b_a, conv=None):
  """conv = None or (segment_pos, conv_w, conv_b) for conv-on-load."""
  B, T, W = x.shape
  H, bw, _ = w_x.shape
  assert H * bw == W and w_a.shape == w_x.shape
  assert b_x.shape == (H, bw) and b_a.shape == (H, bw)
  x = _dev(x, "x")
  _same(x.dtype, x.device, w_x=w_x, b_x=b_x, w_a=w_a, b_a=b_a)
  w_x, b_x, w_a, b_a = (_dev(w_x, "w_x"), _dev(b_x, "b_x"), _dev(w_a, "w_a"),
                        _dev(b_a, "b_a"))
  seg = cw = cb = None
  is64 = 0
  if conv is not None:
    segment_pos, cw, cb = conv
    assert cw.shape == (4, W) and cb.shape == (W,)
    _same(x.dtype, x.device, conv_w=cw, conv_b=cb)
    cw, cb = _dev(cw, "conv_w"), _dev(cb, "conv_b")
    seg, is64 = _segpos(segment_pos, B, T)
  gx = torch.empty_like(x)
  ga = torch.empty_like(x)
  if x.numel() == 0:
    return gx, ga
  with _on(x.device):
    _lib.check(_lib.lib().rg_gates_gemm(
        _p(x), int(conv is not None), _p(seg), is64, _p(cw), _p(cb), _p(w_x),
        _p(b_x), _p(w_a), _p(b_a), _p(gx), _p(ga), B, T, W, H, _dtype_code(x),
        _stream(x)))
  return gx, ga


def gates_weight_grads_supported(x, num_heads) -> bool:
  """bf16 with 256-wide heads: what rg_gates_weight_grads takes."""
  return (x.dtype == torch.bfloat16 and x.shape[-1] == 256 * num_heads)


def gates_weight_grads(x, dgx, dga, num_heads, with_bias=True):
  """(dw_x, dw_a, db_x, db_a) of the two gate projections on x from the
  gradients of their outputs (autograd of layers.py:134-136 with respect to
  w and b): dw [H,256,256], db [H,256] or None; bf16, 256-wide heads."""
  W = x.shape[-1]
  assert dgx.shape == x.shape and dga.shape == x.shape
  x = _dev(x, "x")
  _same(x.dtype, x.device, dgx=dgx, dga=dga)
  dgx, dga = _dev(dgx, "dgx"), _dev(dga, "dga")
  M = x.numel() // W
  H = num_heads
  lib = _lib.lib()
  need = lib.rg_gates_weight_grads_workspace_bytes(M, W, H)
  if need == 0:
    raise ValueError("gates_weight_grads: bf16 with 256-wide heads only")
  ws = torch.empty(need, dtype=torch.uint8, device=x.device)
  dwx = torch.empty(H, 256, 256, dtype=x.dtype, device=x.device)
  dwa = torch.empty_like(dwx)
  dbx = torch.empty(H, 256, dtype=x.dtype, device=x.device) if with_bias else None
  dba = torch.empty_like(dbx) if with_bias else None
  with _on(x.device):
    _lib.check(lib.rg_gates_weight_grads(
        _p(x), _p(dgx), _p(dga), _p(dwx), _p(dwa),
        None if dbx is None else _p(dbx), None if dba is None else _p(dba),
        _p(ws), need, M, W, H, _dtype_code(x), _stream(x)))
  return dwx, dwa, dbx, dba


def _scan_workspace(B, T, W, device, split):
  """Workspace for a scan whose sequences are cut into chunks that run side
  by side (few rows and channels, long sequences), or None for the one-pass
  form (split=False forces that one)."""
  need = _lib.lib().rg_scan_split_workspace_bytes(B, T, W) if split else 0
  return torch.empty(need, dtype=torch.uint8, device=device) if need else None


def lru_scan_fused(x, gx_pre, ga_pre, a_param, segment_pos, h0=None, conv=None,
                   return_h=True, return_conv_cache=False, split=True):
  """conv = None or (conv_w, conv_b): apply the width-4 conv to x first."""
  B, T, W = x.shape
  assert gx_pre.shape == x.shape and ga_pre.shape == x.shape
  assert a_param.shape == (W,)
  x = _dev(x, "x")
  _same(x.dtype, x.device, gx_pre=gx_pre, ga_pre=ga_pre, a_param=a_param)
  gx_pre, ga_pre, a_param = (_dev(gx_pre, "gx_pre"), _dev(ga_pre, "ga_pre"),
                             _dev(a_param, "a_param"))
  seg, is64 = _segpos(segment_pos, B, T)
  if h0 is not None:
    assert h0.dtype == torch.float32, "the RG-LRU state is always float32"
    assert h0.shape == (B, W)
    h0 = _dev(h0, "h0")
  cw = cb = None
  if conv is not None:
    cw, cb = conv
    assert cw.shape == (4, W) and cb.shape == (W,)
    _same(x.dtype, x.device, conv_w=cw, conv_b=cb)
    cw, cb = _dev(cw, "conv_w"), _dev(cb, "conv_b")
  if x.numel() == 0:
    return _empty_prefill(x, h0, return_h, return_conv_cache)
  y = torch.empty_like(x)
  h_last = (torch.empty((B, W), dtype=torch.float32, device=x.device)
            if return_h else None)
  cache = None
  if return_conv_cache:
    assert conv is not None
    cache = x.new_empty((B, 3, W))
  ws = _scan_workspace(B, T, W, x.device, split)
  with _on(x.device):
    if ws is None:
      _lib.check(_lib.lib().rg_lru_scan_fused(
          _p(x), int(conv is not None), _p(cw), _p(cb), _p(gx_pre), _p(ga_pre),
          _p(a_param), _p(seg), is64, _p(h0), _p(y), _p(h_last), _p(cache), B,
          T, W, _dtype_code(x), _stream(x)))
    else:
      _lib.check(_lib.lib().rg_lru_scan_fused_split(
          _p(x), int(conv is not None), _p(cw), _p(cb), _p(gx_pre), _p(ga_pre),
          _p(a_param), _p(seg), is64, _p(h0), _p(y), _p(h_last), _p(cache),
          _p(ws), ws.numel(), B, T, W, _dtype_code(x), _stream(x)))
  return y, h_last, cache


def recurrent_prefill_supported(x, num_heads):
  """Shapes the single-launch prefill kernel serves (rg_recurrent_prefill)."""
  B, T, W = x.shape
  return (x.dtype == torch.bfloat16 and W % num_heads == 0 and
          W // num_heads == 256 and T * W * 2 < 2**31 - 1)


def recurrent_prefill_chunked(B, T, W, num_heads) -> bool:
  """Whether rg_recurrent_prefill_split cuts the sequences of this shape into
  chunks (few (row, head) pairs, long rows)."""
  return _lib.lib().rg_recurrent_prefill_split_workspace_bytes(
      B, T, W, num_heads) > 0


def recurrent_prefill(x, segment_pos, conv_w, conv_b, w_x, b_x, w_a, b_a,
                      a_param, h0=None, return_h=True, return_conv_cache=True,
                      split=True, gate_branch=None):
  """conv -> gates -> recurrence of a whole prefill in one launch.

  Returns (y, h_last | None, conv_cache | None).  Only for the shapes
  recurrent_prefill_supported() accepts; other shapes go through gates_gemm +
  lru_scan_fused.  split: with few (row, head) pairs the sequences are cut
  into chunks that run side by side (rg_recurrent_prefill_split); False forces
  one workgroup per pair.  gate_branch: the output of the block's linear_y
  ([B,T,W], before its activation); y is then y * gelu(gate_branch), the input
  of linear_out (rg_recurrent_prefill_gelu_mul).
  """
  B, T, W = x.shape
  H = w_x.shape[0]
  assert conv_w.shape == (4, W) and conv_b.shape == (W,)
  assert w_x.shape == w_a.shape == (H, W // H, W // H)
  assert b_x.shape == b_a.shape == (H, W // H)
  assert a_param.shape == (W,)
  x = _dev(x, "x")
  _same(x.dtype, x.device, conv_w=conv_w, conv_b=conv_b, w_x=w_x, b_x=b_x,
        w_a=w_a, b_a=b_a, a_param=a_param)
  args = [_dev(t, n) for t, n in ((conv_w, "conv_w"), (conv_b, "conv_b"),
                                  (w_x, "w_x"), (b_x, "b_x"), (w_a, "w_a"),
                                  (b_a, "b_a"), (a_param, "a_param"))]
  seg, is64 = _segpos(segment_pos, B, T)
  if h0 is not None:
    assert h0.dtype == torch.float32, "the RG-LRU state is always float32"
    assert h0.shape == (B, W)
    h0 = _dev(h0, "h0")
  if x.numel() == 0:
    return _empty_prefill(x, h0, return_h, return_conv_cache)
  y = torch.empty_like(x)
  h_last = (torch.empty((B, W), dtype=torch.float32, device=x.device)
            if return_h else None)
  cache = x.new_empty((B, 3, W)) if return_conv_cache else None
  cw, cb, wx_, bx_, wa_, ba_, ap_ = args
  packed = packed_gate_weights(w_x, w_a)  # cached per weight version
  lib = _lib.lib()
  need = (lib.rg_recurrent_prefill_split_workspace_bytes(B, T, W, H)
          if split else 0)
  if gate_branch is not None:
    assert split, "the joined form decides about chunks itself"
    assert gate_branch.shape == x.shape
    _same(x.dtype, x.device, gate_branch=gate_branch)
    gate_branch = _dev(gate_branch, "gate_branch")
  with _on(x.device):
    if gate_branch is not None:
      ws = (torch.empty(need, dtype=torch.uint8, device=x.device)
            if need else None)
      _lib.check(lib.rg_recurrent_prefill_gelu_mul(
          _p(x), _p(gate_branch), _p(seg), is64, _p(cw), _p(cb), _p(wx_),
          _p(bx_), _p(wa_), _p(ba_), _p(packed), _p(ap_), _p(h0), _p(y),
          _p(h_last), _p(cache), _p(ws), need, B, T, W, H, _dtype_code(x),
          _stream(x)))
    elif need:
      ws = torch.empty(need, dtype=torch.uint8, device=x.device)
      _lib.check(lib.rg_recurrent_prefill_split(
          _p(x), _p(seg), is64, _p(cw), _p(cb), _p(wx_), _p(bx_), _p(wa_),
          _p(ba_), _p(packed), _p(ap_), _p(h0), _p(y), _p(h_last), _p(cache),
          _p(ws), need, B, T, W, H, _dtype_code(x), _stream(x)))
    else:
      _lib.check(lib.rg_recurrent_prefill(
          _p(x), _p(seg), is64, _p(cw), _p(cb), _p(wx_), _p(bx_), _p(wa_),
          _p(ba_), _p(packed), _p(ap_), _p(h0), _p(y), _p(h_last), _p(cache),
          B, T, W, H, _dtype_code(x), _stream(x)))
  return y, h_last, cache


def recurrent_core(x, segment_pos, conv_w, conv_b, w_x, b_x, w_a, b_a, a_param,
                   h0=None, return_h=True, return_conv_cache=True,
                   gate_branch=None):
  """conv -> RG-LRU of a prefill for any shape and dtype in one call of the
  library, which picks the kernels (rg_recurrent_core): the single prefill
  kernel where it pays, else gate GEMM + scan.  gate_branch: the block's
  linear_y output; the result is then y * gelu(gate_branch).
  conv_w = conv_b = None: x is the conv output already (RGLRU.forward on its
  own, layers.py:313-365); there is then no conv cache to return.
  Returns (y, h_last | None, conv_cache | None)."""
  B, T, W = x.shape
  H = w_x.shape[0]
  if conv_w is None:
    assert conv_b is None
    return_conv_cache = False
  else:
    assert conv_w.shape == (4, W) and conv_b.shape == (W,)
  assert w_x.shape == w_a.shape == (H, W // H, W // H)
  assert b_x.shape == b_a.shape == (H, W // H)
  assert a_param.shape == (W,)
  x = _dev(x, "x")
  _same(x.dtype, x.device, w_x=w_x, b_x=b_x, w_a=w_a, b_a=b_a,
        a_param=a_param)
  cw = cb = None
  if conv_w is not None:
    _same(x.dtype, x.device, conv_w=conv_w, conv_b=conv_b)
    cw, cb = _dev(conv_w, "conv_w"), _dev(conv_b, "conv_b")
  wx_, bx_, wa_, ba_, ap_ = [
      _dev(t, n) for t, n in ((w_x, "w_x"), (b_x, "b_x"), (w_a, "w_a"),
                              (b_a, "b_a"), (a_param, "a_param"))]
  seg, is64 = _segpos(segment_pos, B, T)
  if h0 is not None:
    assert h0.dtype == torch.float32, "the RG-LRU state is always float32"
    assert h0.shape == (B, W)
    h0 = _dev(h0, "h0")
  if gate_branch is not None:
    assert gate_branch.shape == x.shape
    _same(x.dtype, x.device, gate_branch=gate_branch)
    gate_branch = _dev(gate_branch, "gate_branch")
  if x.numel() == 0:
    return _empty_prefill(x, h0, return_h, return_conv_cache)
  y = torch.empty_like(x)
  h_last = (torch.empty((B, W), dtype=torch.float32, device=x.device)
            if return_h else None)
  cache = x.new_empty((B, 3, W)) if return_conv_cache else None
  packed = (packed_gate_weights(w_x, w_a)  # cached per weight version
            if recurrent_prefill_supported(x, H) else None)
  lib = _lib.lib()
  code = _dtype_code(x)
  need = lib.rg_recurrent_core_workspace_bytes(B, T, W, H, code)
  ws = torch.empty(need, dtype=torch.uint8, device=x.device) if need else None
  with _on(x.device):
    _lib.check(lib.rg_recurrent_core(
        _p(x), _p(gate_branch), _p(seg), is64, _p(cw), _p(cb), _p(wx_),
        _p(bx_), _p(wa_), _p(ba_), _p(packed), _p(ap_), _p(h0), _p(y),
        _p(h_last), _p(cache), _p(ws), need, B, T, W, H, code, _stream(x)))
  return y, h_last, cache


def linear_scan(x, a, reset, h0=None, split=True):
  B, T, W = x.shape
  x = _dev(x, "x")
  _same(x.dtype, x.device, a=a)
  a = _dev(a, "a")
  assert reset.shape == (B, T) and reset.dtype == torch.bool
  reset = _dev(reset, "reset")
  if h0 is not None:
    h0 = _dev(h0, "h0")
  if x.numel() == 0:
    y, h_last, _ = _empty_prefill(x, h0, True, False)
    return y, h_last
  y = torch.empty_like(x)
  h_last = torch.empty((B, W), dtype=torch.float32, device=x.device)
  ws = _scan_workspace(B, T, W, x.device, split)
  with _on(x.device):
    if ws is None:
      _lib.check(_lib.lib().rg_linear_scan(
          _p(x), _p(a), _p(reset), _p(h0), _p(y), _p(h_last), B, T, W,
          _dtype_code(x), _stream(x)))
    else:
      _lib.check(_lib.lib().rg_linear_scan_split(
          _p(x), _p(a), _p(reset), _p(h0), _p(y), _p(h_last), _p(ws),
          ws.numel(), B, T, W, _dtype_code(x), _stream(x)))
  return y, h_last


def linear_scan_backward(dy, a, reset, y, h0=None, dh_last=None):
  """Gradients of linear_scan: (dx, da, dh0 | None) from the gradient of y
  (and of the final state); one kernel, no flipped copies."""
  B, T, W = y.shape
  y = _dev(y, "y")
  _same(y.dtype, y.device, dy=dy, a=a)
  dy, a = _dev(dy, "dy"), _dev(a, "a")
  assert dy.shape == a.shape == y.shape
  assert reset.shape == (B, T) and reset.dtype == torch.bool
  reset = _dev(reset, "reset")
  if h0 is not None:
    assert h0.dtype == torch.float32 and h0.shape == (B, W)
    h0 = _dev(h0, "h0")
  if dh_last is not None:
    assert dh_last.dtype == torch.float32 and dh_last.shape == (B, W)
    dh_last = _dev(dh_last, "dh_last")
  dx, da = torch.empty_like(y), torch.empty_like(y)
  dh0 = (torch.empty((B, W), dtype=torch.float32, device=y.device)
         if h0 is not None else None)
  with _on(y.device):
    _lib.check(_lib.lib().rg_linear_scan_backward(
        _p(dy), _p(a), _p(reset), _p(y), _p(h0), _p(dh_last), _p(dx), _p(da),
        _p(dh0), B, T, W, _dtype_code(y), _stream(y)))
  return dx, da, dh0


def _workspace(B, W, dtype, device):
  """Scratch of one rg_recurrent_step call, allocated per call: under graph
  capture it then comes from the graph's own pool and stays valid for the
  replays, and calls on different streams do not share it."""
  n = _lib.lib().rg_recurrent_step_workspace_bytes(B, W, _DTYPES[dtype])
  return torch.empty(n, dtype=torch.uint8, device=device)


def gelu_mul(a, g):
  """a * gelu_tanh(g) in one pass (the x * y join of RecurrentBlock.forward)."""
  assert a.shape == g.shape
  a = _dev(a, "a")
  _same(a.dtype, a.device, g=g)
  g = _dev(g, "g")
  out = torch.empty_like(a)
  with _on(a.device):
    _lib.check(_lib.lib().rg_gelu_mul(_p(a), _p(g), _p(out), a.numel(),
                                      _dtype_code(a), _stream(a)))
  return out


def gelu_mul_backward(dout, a, g):
  """(d_a, d_g) of out = a * gelu_tanh(g), one pass."""
  assert dout.shape == a.shape == g.shape
  a = _dev(a, "a")
  _same(a.dtype, a.device, g=g, dout=dout)
  g = _dev(g, "g")
  dout = _dev(dout, "dout")
  d_a, d_g = torch.empty_like(a), torch.empty_like(g)
  with _on(a.device):
    _lib.check(_lib.lib().rg_gelu_mul_backward(
        _p(dout), _p(a), _p(g), _p(d_a), _p(d_g), a.numel(), _dtype_code(a),
        _stream(a)))
  return d_a, d_g


def rms_norm(x, scale, eps=1e-6):
  """x * rsqrt(mean(x^2, -1) + eps) * (scale + 1), one pass."""
  x = _dev(x, "x")
  _same(x.dtype, x.device, scale=scale)
  scale = _dev(scale, "scale")
  width = x.shape[-1]
  assert scale.shape == (width,)
  out = torch.empty_like(x)
  with _on(x.device):
    _lib.check(_lib.lib().rg_rms_norm(_p(x), _p(scale), _p(out),
                                      x.numel() // width, width, eps,
                                      _dtype_code(x), _stream(x)))
  return out


def add_rms_norm(x, addend, scale, eps=1e-6):
  """(x + addend, rms_norm(x + addend)) in one pass.  x may be a PartialSums
  (then addend may be None: the sum is the layer output itself)."""
  if isinstance(x, PartialSums):
    return _add_rms_norm_partial(x, addend, scale, eps)
  assert x.shape == addend.shape
  x = _dev(x, "x")
  _same(x.dtype, x.device, addend=addend, scale=scale)
  addend, scale = _dev(addend, "addend"), _dev(scale, "scale")
  width = x.shape[-1]
  assert scale.shape == (width,)
  total, out = torch.empty_like(x), torch.empty_like(x)
  with _on(x.device):
    _lib.check(_lib.lib().rg_add_rms_norm(
        _p(x), _p(addend), _p(scale), _p(total), _p(out), x.numel() // width,
        width, eps, _dtype_code(x), _stream(x)))
  return total, out


def soft_cap(x, cap):
  """tanh(x / cap) * cap, one pass."""
  x = _dev(x, "x")
  out = torch.empty_like(x)
  with _on(x.device):
    _lib.check(_lib.lib().rg_soft_cap(_p(x), _p(out), x.numel(), float(cap),
                                      _dtype_code(x), _stream(x)))
  return out


def argmax_last(x):
  """torch.argmax(x, dim=-1) (first index among equals), one pass."""
  x = _dev(x, "x")
  n = x.shape[-1]
  out = torch.empty(x.shape[:-1], dtype=torch.int64, device=x.device)
  with _on(x.device):
    _lib.check(_lib.lib().rg_argmax_rows(_p(x), _p(out), x.numel() // n, n,
                                         _dtype_code(x), _stream(x)))
  return out


def _add_rms_norm_partial(ps, addend, scale, eps):
  if ps.addend is not None:
    if addend is not None:
      raise ValueError("the partial sums already carry an addend")
    addend = ps.addend
  slices, rows, width = ps.sums.shape
  scale = _dev(scale, "scale")
  assert scale.shape == (width,) and scale.dtype == ps.dtype
  if addend is not None:
    assert tuple(addend.shape) == tuple(ps.shape)
    _same(ps.dtype, ps.sums.device, addend=addend)
    addend = _dev(addend, "addend")
  total = torch.empty(ps.shape, dtype=ps.dtype, device=ps.sums.device)
  out = torch.empty_like(total)
  with _on(total.device):
    _lib.check(_lib.lib().rg_add_rms_norm_partial(
        _p(ps.sums), slices, _p(ps.bias), _p(addend), _p(scale), _p(total),
        _p(out), rows, width, eps, _DTYPES[ps.dtype], _stream(total)))
  return total, out


def rope(x, positions, inv_freq):
  """Rotary embedding on the first half of the last dimension of
  x [B, T, heads, head_dim]; positions [B, T]; inv_freq [head_dim / 4] f32."""
  B, T, n, hd = x.shape
  x = _dev(x, "x")
  pos, is64 = _segpos(positions, B, T)
  inv = _dev(inv_freq, "inv_freq")
  assert inv.dtype == torch.float32 and inv.shape == (hd // 4,)
  out = torch.empty_like(x)
  with _on(x.device):
    _lib.check(_lib.lib().rg_rope(_p(x), _p(pos), is64, _p(inv), _p(out),
                                  B * T, n, hd, _dtype_code(x), _stream(x)))
  return out


def rope_pair(q, k, positions, inv_freq):
  """rope(q), rope(k) in one launch: q [B, T, heads, hd], k [B, T, kv_heads,
  hd], same positions."""
  B, T, n, hd = q.shape
  assert k.shape[:2] == (B, T) and k.shape[3] == hd
  q, k = _dev(q, "q"), _dev(k, "k")
  _same(q.dtype, q.device, k=k)
  pos, is64 = _segpos(positions, B, T)
  inv = _dev(inv_freq, "inv_freq")
  assert inv.dtype == torch.float32 and inv.shape == (hd // 4,)
  q_out, k_out = torch.empty_like(q), torch.empty_like(k)
  with _on(q.device):
    _lib.check(_lib.lib().rg_rope_pair(
        _p(q), _p(k), _p(pos), is64, _p(inv), _p(q_out), _p(k_out), B * T, n,
        k.shape[2], hd, _dtype_code(q), _stream(q)))
  return q_out, k_out


def attention_prefill_supported(q):
  """Shapes the prompt-pass attention kernel serves (rg_attention_prefill)."""
  return (q.is_cuda and q.dtype == torch.bfloat16 and q.ndim == 4 and
          q.shape[-1] == 256 and q.shape[1] * q.shape[2] * 512 < 2**31)


def attention_prefill(q, k, v, first_key, scale):
  """Sliding-window multi-query attention over a prompt in one kernel.
  q [B,T,H,256], k and v [B,T,1,256] or [B,T,256] (q, k after the rotary
  embedding), first_key [B,T] int32: query t sees the keys first_key[t] .. t.
  Returns [B,T,H,256]."""
  B, T, H, hd = q.shape
  q = _dev(q, "q")
  k = _dev(k.reshape(B, T, hd), "k")
  _same(q.dtype, q.device, k=k, v=v)
  assert first_key.shape == (B, T) and first_key.dtype == torch.int32
  first_key = _dev(first_key, "first_key")
  t_pad = (T + 63) // 64 * 64
  # the values transposed (keys contiguous), zeros behind the last token
  v_t = q.new_zeros((B, hd, t_pad))
  v_t[:, :, :T] = v.reshape(B, T, hd).transpose(1, 2)
  out = torch.empty_like(q)
  with _on(q.device):
    _lib.check(_lib.lib().rg_attention_prefill(
        _p(q), _p(k), _p(v_t), _p(first_key), _p(out), B, T, t_pad, H, hd,
        float(scale), _dtype_code(q), _stream(q)))
  return out


def attention_decode_probs(scores, q, k_new, num_tokens, scale):
  """softmax over the written ring slots and the new token: scores
  [B, heads, window] (unscaled), q [B, heads, hd], k_new [B, hd], num_tokens
  [B] int32 -> probs [B, heads, window + 1]."""
  B, heads, window = scores.shape
  hd = q.shape[-1]
  scores, q, k_new = _dev(scores, "scores"), _dev(q, "q"), _dev(k_new, "k_new")
  _same(scores.dtype, scores.device, q=q, k_new=k_new)
  assert q.shape == (B, heads, hd) and k_new.shape == (B, hd)
  assert num_tokens.dtype == torch.int32 and num_tokens.shape == (B,)
  nt = _dev(num_tokens, "num_tokens")
  probs = torch.empty((B, heads, window + 1), dtype=scores.dtype,
                      device=scores.device)
  with _on(scores.device):
    _lib.check(_lib.lib().rg_attention_decode_probs(
        _p(scores), _p(q), _p(k_new), _p(nt), _p(probs), B, heads, hd, window,
        scale, _dtype_code(scores), _stream(scores)))
  return probs


def attention_decode_finish(from_ring, probs, k_new, v_new, ring_keys,
                            ring_values, num_tokens, update_cache):
  """from_ring + probs[..., -1] * v_new; with update_cache the new key and
  value go into slot num_tokens % window of the ring (in place) and num_tokens
  is incremented (in place)."""
  B, heads, hd = from_ring.shape
  window = probs.shape[-1] - 1
  from_ring, probs = _dev(from_ring, "from_ring"), _dev(probs, "probs")
  k_new, v_new = _dev(k_new, "k_new"), _dev(v_new, "v_new")
  _same(from_ring.dtype, from_ring.device, probs=probs, k_new=k_new,
        v_new=v_new, ring_keys=ring_keys, ring_values=ring_values)
  for t, name in ((ring_keys, "ring_keys"), (ring_values, "ring_values"),
                  (num_tokens, "num_tokens")):
    # updated in place: no silent copies
    if not (t.is_cuda and t.is_contiguous() and t.data_ptr() % 16 == 0):
      raise ValueError(f"{name} must be a contiguous, 16-byte aligned GPU "
                       "tensor (it is updated in place)")
  assert ring_keys.numel() == B * window * hd == ring_values.numel()
  assert num_tokens.dtype == torch.int32 and num_tokens.shape == (B,)
  out = torch.empty_like(from_ring)
  with _on(out.device):
    _lib.check(_lib.lib().rg_attention_decode_finish(
        _p(from_ring), _p(probs), _p(k_new), _p(v_new), _p(out),
        _p(ring_keys), _p(ring_values), _p(num_tokens), B, heads, hd, window,
        int(bool(update_cache)), _dtype_code(out), _stream(out)))
  return out


def attention_decode_fused_supported(x, heads, head_dim, window) -> bool:
  """Whether attention_decode_fused takes this shape: bf16 on the GPU,
  head_dim 256, at most 16 heads, a window the chunk table covers."""
  return (x.is_cuda and x.dtype == torch.bfloat16 and head_dim == 256 and
          x.shape[0] <= 65535 and
          _lib.lib().rg_attention_decode_fused_workspace_bytes(
              x.shape[0], heads, window) > 0)


def _rows_view(t, name, width):
  """[B, width] with unit stride inside a row (rows may lie apart: a slice of
  a wider projection output): (tensor, row stride in elements)."""
  if t.dim() != 2 or t.shape[1] != width:
    raise ValueError(f"{name} must be [B, {width}], got {tuple(t.shape)}")
  if not t.is_cuda:
    raise ValueError(f"{name} must live on the GPU")
  if (t.shape[0] > 1 and t.stride(0) % 8) or t.stride(1) != 1 or (
      t.data_ptr() % 16):
    t = t.contiguous()
  return t, (t.stride(0) if t.shape[0] > 1 else width)


def attention_decode_fused(q, k_new, v_new, positions, inv_freq, ring_keys,
                           ring_values, num_tokens, scale, update_cache=True):
  """One new token per row against the ring cache and itself
  (modules.py:431-476): rotary embedding of q and k_new, scores, mask,
  softmax, values, the new token's share; with update_cache the rotated key
  and the value go into slot num_tokens % window (in place) and num_tokens is
  incremented (in place).  q [B, heads * 256], k_new, v_new [B, 256] as the
  projections left them (slices of one wider output are taken as they lie);
  positions [B]; ring_* [B, window, 256].  Returns [B, heads, 256]."""
  B = q.shape[0]
  hd = 256
  heads = q.shape[1] // hd
  window = ring_keys.numel() // (B * hd)
  q, ldq = _rows_view(q, "q", heads * hd)
  k_new, ldk = _rows_view(k_new, "k_new", hd)
  v_new, ldv = _rows_view(v_new, "v_new", hd)
  _same(q.dtype, q.device, k_new=k_new, v_new=v_new, ring_keys=ring_keys,
        ring_values=ring_values)
  for t, name in ((ring_keys, "ring_keys"), (ring_values, "ring_values"),
                  (num_tokens, "num_tokens")):
    # updated in place: no silent copies
    if not (t.is_cuda and t.is_contiguous() and t.data_ptr() % 16 == 0):
      raise ValueError(f"{name} must be a contiguous, 16-byte aligned GPU "
                       "tensor (it is updated in place)")
  assert ring_keys.numel() == B * window * hd == ring_values.numel()
  assert num_tokens.dtype == torch.int32 and num_tokens.shape == (B,)
  positions = _dev(positions.reshape(-1), "positions")
  assert positions.shape == (B,)
  if positions.dtype not in (torch.int32, torch.int64):
    raise TypeError("positions must be int32 or int64")
  inv_freq = _dev(inv_freq, "inv_freq")
  assert inv_freq.dtype == torch.float32 and inv_freq.numel() == hd // 4
  lib = _lib.lib()
  need = lib.rg_attention_decode_fused_workspace_bytes(B, heads, window)
  if need == 0:
    raise ValueError(f"unsupported shape heads={heads} window={window}")
  ws = torch.empty(need, dtype=torch.uint8, device=q.device)
  out = torch.empty((B, heads, hd), dtype=q.dtype, device=q.device)
  with _on(q.device):
    _lib.check(lib.rg_attention_decode_fused(
        _p(q), ldq, _p(k_new), ldk, _p(v_new), ldv, _p(positions),
        int(positions.dtype == torch.int64), _p(inv_freq), _p(ring_keys),
        _p(ring_values), _p(num_tokens), _p(out), _p(ws), need, B, heads, hd,
        window, float(scale), int(bool(update_cache)), _dtype_code(q),
        _stream(q)))
  return out


def rglru_backward(dy, x, gx_pre, ga_pre, a_param, reset, y, h0=None,
                   dh_last=None):
  """Gradients of the RG-LRU from its gate pre-activations on (the forward is
  lru_scan_fused without the conv): (dx, dgx_pre, dga_pre, d_a_param, dh0 |
  None) from the gradient of y and of the final state; one kernel."""
  B, T, W = y.shape
  y = _dev(y, "y")
  _same(y.dtype, y.device, dy=dy, x=x, gx_pre=gx_pre, ga_pre=ga_pre,
        a_param=a_param)
  assert dy.shape == x.shape == gx_pre.shape == ga_pre.shape == y.shape
  assert a_param.shape == (W,)
  dy, x, gx_pre, ga_pre, a_param = (
      _dev(dy, "dy"), _dev(x, "x"), _dev(gx_pre, "gx_pre"),
      _dev(ga_pre, "ga_pre"), _dev(a_param, "a_param"))
  assert reset.shape == (B, T) and reset.dtype == torch.bool
  reset = _dev(reset, "reset")
  if h0 is not None:
    assert h0.dtype == torch.float32 and h0.shape == (B, W)
    h0 = _dev(h0, "h0")
  if dh_last is not None:
    assert dh_last.dtype == torch.float32 and dh_last.shape == (B, W)
    dh_last = _dev(dh_last, "dh_last")
  dx, dgx, dga = (torch.empty_like(y) for _ in range(3))
  rows = torch.empty((B, W), dtype=torch.float32, device=y.device)
  dh0 = torch.empty_like(h0) if h0 is not None else None
  with _on(y.device):
    _lib.check(_lib.lib().rg_rglru_backward(
        _p(dy), _p(x), _p(gx_pre), _p(ga_pre), _p(a_param), _p(reset), _p(y),
        _p(h0), _p(dh_last), _p(dx), _p(dgx), _p(dga), _p(rows), _p(dh0), B, T,
        W, _dtype_code(y), _stream(y)))
  return dx, dgx, dga, rows.sum(0).to(a_param.dtype), dh0


_packed_weights = {}  # (id(w_x), id(w_a)) -> (ref_x, ref_a, stamp, packed)


def tensor_stamp(t):
  """(storage address, version counter) of a tensor: changes when the tensor
  is written in place or re-pointed.  Inference-mode tensors keep no version
  counter; None then stands in, and callers treat such a stamp as never equal
  to a kept one (they recompute)."""
  if t.is_inference():
    return (t.data_ptr(), None)
  return (t.data_ptr(), t._version)


def stamps_match(old, new):
  return old == new and not any(v is None for _, v in new)


def packed_gate_weights(w_x, w_a):
  """Both gate matrices in MFMA operand order (rg_pack_gate_weights), cached per
  pair of tensor objects until either is written to, re-pointed or dies."""
  import weakref
  key = (id(w_x), id(w_a))
  stamp = (tensor_stamp(w_x), tensor_stamp(w_a))
  hit = _packed_weights.get(key)
  if hit is not None:
    ref_x, ref_a, old_stamp, packed = hit
    if ref_x() is w_x and ref_a() is w_a and stamps_match(old_stamp, stamp):
      return packed
  H, bw, _ = w_x.shape
  W = H * bw
  nbytes = _lib.lib().rg_packed_gate_weights_bytes(W, H, _dtype_code(w_x))
  if nbytes == 0:
    return None
  packed = torch.empty(nbytes // 2, dtype=w_x.dtype, device=w_x.device)
  with _on(w_x.device):
    _lib.check(_lib.lib().rg_pack_gate_weights(
        _p(_dev(w_x, "w_x")), _p(_dev(w_a, "w_a")), _p(packed), W, H,
        _dtype_code(w_x), _stream(w_x)))
  for k in [k for k, v in _packed_weights.items()
            if v[0]() is None or v[1]() is None]:
    del _packed_weights[k]  # entries whose tensors are gone
  _packed_weights[key] = (weakref.ref(w_x), weakref.ref(w_a), stamp, packed)
  return packed


class PartialSums:
  """The output of a linear layer that has not been added up yet: fp32 partial
  sums over slices of K (PackedLinear.partial), its bias, and optionally a
  tensor still to be added (a skip connection).  `add_rms_norm` takes it in
  place of a tensor; `materialize()` gives the tensor it stands for."""

  def __init__(self, sums, bias, shape, dtype, addend=None):
    self.sums, self.bias = sums, bias    # [slices, M, N] float32, [N] | None
    self.shape, self.dtype = shape, dtype  # of the tensor this stands for
    self.addend = addend

  def materialize(self):
    out = (self.sums.sum(0) if self.bias is None
           else self.sums.sum(0) + self.bias.float())
    out = out.to(self.dtype).reshape(self.shape)
    return out if self.addend is None else out + self.addend


class PendingSum:
  """a + b, not added yet: the norm kernel that reads the sum next forms it
  in the same pass (add_rms_norm), which saves the pass of the add."""

  def __init__(self, a, b):
    assert a.shape == b.shape
    self.a, self.b = a, b

  def materialize(self):
    return self.a + self.b


class PackedLinear:
  """Linear layers that read the same few rows (a decode step), on the
  weight-streaming kernel (rg_linear_rows).  Holds the weights in the kernel's
  operand order, packed on first use and again whenever a parameter is written
  to or re-pointed; the parameters themselves are passed with every call.

  layout 0: `weights` are torch.nn.Linear weights [N_i, K] applied to the same
    input; several of them run as one launch and come back as a tuple of
    outputs (equal N_i) or as one output [..., sum N_i] for the caller to
    slice (unequal N_i, multiples of 32).
  layout 1: one stacked Einsum weight [G, K, E] (layers.py:76-101) with bias
    [G, 1, 1, E]; outputs as a tuple of G tensors, or, with gelu_pair (G = 2),
    gelu(out[0]) * out[1] as one tensor (modules.py:752-757).
  """

  def __init__(self, layout=0, gelu_pair=False):
    self.layout = layout
    self.gelu_pair = gelu_pair
    self._stamp = None
    self._packed = None
    self._bias = None
    self._shape = None  # (N, K, groups)

  def __deepcopy__(self, memo):
    return PackedLinear(self.layout, self.gelu_pair)

  @staticmethod
  def usable(x, K, N, gelu_pair=False) -> bool:
    """Whether x [..., K] qualifies: bf16 on the GPU, at most 64 rows, and a
    weight shape the packed layout covers."""
    return (x.is_cuda and x.dtype == torch.bfloat16 and
            x.numel() // K <= 64 and
            _lib.lib().rg_linear_packed_bytes(N, K, int(gelu_pair)) > 0)

  def _prepare(self, weights, biases):
    tensors = tuple(weights) + tuple(b for b in (biases or ()) if b is not None)
    stamp = tuple((id(t),) + tensor_stamp(t) for t in tensors)
    if stamp == self._stamp and not any(v[2] is None for v in stamp):
      return
    w0 = weights[0]
    lib = _lib.lib()
    if self.layout == 0:
      K = w0.shape[1]
      rows = [w.shape[0] for w in weights]
      if any(w.shape[1] != K for w in weights):
        raise ValueError("layers packed together must read the same input")
      if len(set(rows)) == 1:
        groups, N = len(weights), sum(rows)
      else:
        # unequal layers: one output [..., sum of rows], which the caller
        # slices (whole 32-row tiles each, so that the tiles stay apart)
        if any(r % 32 for r in rows):
          raise ValueError("unequal layers packed together need row counts "
                           "that are multiples of 32")
        groups, N = 1, sum(rows)
    else:
      assert len(weights) == 1
      groups, K, E = w0.shape
      N = groups * E
      if self.gelu_pair and groups != 2:
        raise ValueError("gelu pairs need a weight stacked [2, K, E]")
    nbytes = lib.rg_linear_packed_bytes(N, K, int(self.gelu_pair))
    if nbytes == 0:
      raise ValueError(f"unsupported linear shape N={N} K={K}")
    packed = torch.empty(nbytes // 2, dtype=w0.dtype, device=w0.device)
    with _on(w0.device):
      if self.layout == 0:
        at = 0
        for w in weights:  # tile blocks of consecutive rows are consecutive
          part = packed[at:at + w.numel()]
          _lib.check(lib.rg_linear_pack(_p(_dev(w, "weight")), 0, 1, 0, _p(part),
                                        w.shape[0], K, _stream(w)))
          at += w.numel()
      else:
        _lib.check(lib.rg_linear_pack(_p(_dev(w0, "weight")), 1, groups,
                                      int(self.gelu_pair), _p(packed), N, K,
                                      _stream(w0)))
    bias = None
    if biases is not None and any(b is not None for b in biases):
      if any(b is None for b in biases):
        raise ValueError("either every layer has a bias or none")
      bias = torch.cat([b.detach().reshape(-1) for b in biases])
      assert bias.numel() == N
    self._packed, self._bias = packed, bias
    self._shape = (N, K, groups)
    self._stamp = stamp

  @staticmethod
  def partial_slices(x, K, N) -> int:
    """In how many slices of K `partial` would run this shape; 0 = not worth
    it (enough weight rows to fill the GPU without splitting K, or a width the
    norm kernel that adds the slices does not take)."""
    if not PackedLinear.usable(x, K, N) or N % 8 or N > 4096:
      return 0
    tiles = N // 32
    return 3 if tiles <= 85 else 2 if tiles <= 128 else 0

  @torch.no_grad()
  def partial(self, x, weights, biases=None, addend=None) -> PartialSums:
    """One layer, left as partial sums for the norm that follows it
    (add_rms_norm): K is split over the grid, so three times as many
    workgroups stream the weights, and no separate pass adds the slices."""
    x = _dev(x, "x")
    self._prepare(weights, biases)
    N, K, groups = self._shape
    assert groups == 1 and not self.gelu_pair
    slices = self.partial_slices(x, K, N)
    assert slices > 0
    M = x.numel() // K
    sums = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
    with _on(x.device):
      _lib.check(_lib.lib().rg_linear_rows_partial(
          _p(x), _p(self._packed), _p(sums), M, K, N, slices, _stream(x)))
    return PartialSums(sums, self._bias, (*x.shape[:-1], N), x.dtype, addend)

  @torch.no_grad()
  def __call__(self, x, weights, biases=None, residual=None):
    """x [..., K].  Returns out [..., N] (one layer), a tuple of outputs
    (several layers / a stacked weight), or the gelu pair product [..., N/2].
    residual (one layer only): added after the output is rounded."""
    x = _dev(x, "x")
    _dtype_code(x)
    self._prepare(weights, biases)
    N, K, groups = self._shape
    if x.shape[-1] != K:
      raise ValueError(f"x has {x.shape[-1]} columns, the weights take {K}")
    _same(x.dtype, x.device, weight=weights[0], residual=residual)
    lead = x.shape[:-1]
    M = x.numel() // K
    lib = _lib.lib()
    if self.gelu_pair:
      out = torch.empty((*lead, N // 2), dtype=x.dtype, device=x.device)
      g = 1
    elif groups > 1:
      out = torch.empty((groups, *lead, N // groups), dtype=x.dtype,
                        device=x.device)
      g = groups
    else:
      out = torch.empty((*lead, N), dtype=x.dtype, device=x.device)
      g = 1
    if residual is not None:
      if g != 1 or self.gelu_pair:
        raise ValueError("a residual goes with a single plain layer")
      residual = _dev(residual, "residual")
      assert residual.shape == out.shape
    need = lib.rg_linear_rows_workspace_bytes(M, K, N)
    ws = (torch.empty(need, dtype=torch.uint8, device=x.device)
          if need and not self.gelu_pair else None)
    with _on(x.device):
      _lib.check(lib.rg_linear_rows(
          _p(x), _p(self._packed), _p(self._bias), _p(residual), _p(out),
          _p(ws), need if ws is not None else 0, M, K, N, g,
          int(self.gelu_pair), _stream(x)))
    if g > 1:
      return tuple(out[i] for i in range(g))
    return out


def recurrent_step(x, segment_pos, conv_cache, h, conv_w, conv_b, w_x, b_x, w_a,
                   b_a, a_param, in_place=False, gate_branch=None):
  """One decode step of conv -> RG-LRU.  Returns (y, h_new, conv_cache_new).

  bf16 with 256-wide heads runs as one launch on re-laid-out gate weights
  (packed once per weight version); other shapes as conv step + gate GEMM +
  scan step.  gate_branch: the block's linear_y output [B,1,W]; y is then
  y * gelu(gate_branch) (inside the one launch where that runs)."""
  B, n_tok, W = x.shape
  assert n_tok == 1
  assert conv_cache.shape == (B, 3, W)
  assert h.shape == (B, W) and h.dtype == torch.float32
  H = w_x.shape[0]
  x = _dev(x, "x")
  _same(x.dtype, x.device, conv_w=conv_w, conv_b=conv_b, w_x=w_x, b_x=b_x,
        w_a=w_a, b_a=b_a, a_param=a_param)
  if in_place and conv_cache.dtype != x.dtype:
    raise ValueError(
        f"in-place decode needs a conv state in the activation dtype "
        f"{x.dtype}, got {conv_cache.dtype}")
  cache_in = _dev(conv_cache.to(x.dtype), "conv_cache", in_place)
  h_in = _dev(h, "h", in_place)
  seg, is64 = _segpos(segment_pos, B, 1)
  args = [_dev(t, n) for t, n in ((conv_w, "conv_w"), (conv_b, "conv_b"),
                                  (w_x, "w_x"), (b_x, "b_x"), (w_a, "w_a"),
                                  (b_a, "b_a"), (a_param, "a_param"))]
  if in_place:
    cache_out, h_out = cache_in, h_in
  else:
    cache_out, h_out = torch.empty_like(cache_in), torch.empty_like(h_in)
  y = torch.empty_like(x)
  packed = None
  if x.dtype == torch.bfloat16 and W // H == 256 and W % H == 0:
    packed = packed_gate_weights(w_x, w_a)
  if gate_branch is not None:
    assert gate_branch.shape == x.shape
    _same(x.dtype, x.device, gate_branch=gate_branch)
    gate_branch = _dev(gate_branch, "gate_branch")
  if packed is not None:
    cw, cb, wx_, bx_, wa_, ba_, ap_ = args
    with _on(x.device):
      if gate_branch is not None:
        _lib.check(_lib.lib().rg_recurrent_step_gelu_mul(
            _p(x), _p(gate_branch), _p(seg), is64, _p(cache_in), _p(cache_out),
            _p(h_in), _p(h_out), _p(cw), _p(cb), _p(packed), _p(bx_), _p(ba_),
            _p(ap_), _p(y), B, W, H, _dtype_code(x), _stream(x)))
      else:
        _lib.check(_lib.lib().rg_recurrent_step_packed(
            _p(x), _p(seg), is64, _p(cache_in), _p(cache_out), _p(h_in),
            _p(h_out), _p(cw), _p(cb), _p(packed), _p(bx_), _p(ba_), _p(ap_),
            _p(y), B, W, H, _dtype_code(x), _stream(x)))
    if cache_out.dtype != conv_cache.dtype:
      cache_out = cache_out.to(conv_cache.dtype)
    return y, h_out, cache_out
  ws = _workspace(B, W, x.dtype, x.device)
  with _on(x.device):
    _lib.check(_lib.lib().rg_recurrent_step(
        _p(x), _p(seg), is64, _p(cache_in), _p(cache_out), _p(h_in), _p(h_out),
        *[_p(t) for t in args], _p(y), _p(ws), ws.numel(), B, W, H,
        _dtype_code(x), _stream(x)))
  if cache_out.dtype != conv_cache.dtype:
    cache_out = cache_out.to(conv_cache.dtype)
  if gate_branch is not None:
    y = gelu_mul(y, gate_branch)
  return y, h_out, cache_out
