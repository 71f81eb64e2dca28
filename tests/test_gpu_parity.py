"""GPU parity: the HIP path (through the C ABI) against the CPU oracle.

Tolerances (the bars this build is held to): float32 max|d|/max|ref| <= 1e-5 on y and h;
bfloat16-in / float32-state <= 1e-2 against the widened oracle (reference
semantics evaluated in float32 on the bfloat16 values, outputs rounded once).
"""

import numpy as np
import pytest
import torch

import recurrentgemma_amd as rg
from oracle import torch_ref as R
from recurrentgemma_amd import _lib
from recurrentgemma_amd import ops
from tests import helpers

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F32_TOL = 1e-5
BF16_TOL = 1e-2


def _dev(t):
  return None if t is None else t.to(DEV)


def _announce(*what):
  print("[case]", *what, flush=True)


def _mk_conv(w, b):
  m = rg.Conv1D(width=w.shape[1], temporal_width=w.shape[0], dtype=w.dtype)
  m.load_state_dict({"w": w, "b": b})
  return m.to(DEV)


def _mk_lru(prm, H):
  a_param, w_x, b_x, w_a, b_a = prm
  m = rg.RGLRU(width=a_param.shape[0], num_heads=H, dtype=a_param.dtype)
  m.load_state_dict({"a_param": a_param, "input_gate.w": w_x,
                     "input_gate.b": b_x, "a_gate.w": w_a, "a_gate.b": b_a})
  return m.to(DEV)


def _block(params, width, heads, dtype, K=4):
  blk = rg.RecurrentBlock(width=width, num_heads=heads, lru_width=width,
                          conv1d_temporal_width=K, dtype=dtype)
  blk.conv_1d.load_state_dict({"w": params["conv_w"], "b": params["conv_b"]})
  blk.rg_lru.load_state_dict({
      "a_param": params["a_param"], "input_gate.w": params["w_x"],
      "input_gate.b": params["b_x"], "a_gate.w": params["w_a"],
      "a_gate.b": params["b_a"]})
  return blk.to(DEV)


def test_library_loaded():
  assert _lib.lib().rg_abi_version() == 1
  assert torch.cuda.is_available()
  name = torch.cuda.get_device_name(0)
  arch = torch.cuda.get_device_properties(0).gcnArchName
  print("device:", name, arch, "lib:", _lib.LIB_PATH)
  assert "gfx950" in arch, arch
  # the library this process mapped is the in-tree one
  maps = open("/proc/self/maps").read()
  assert _lib.LIB_PATH in maps or "librg_lru.so" in maps


# ------------------------------------------------------------- Conv1D ------


def test_conv1d_golden(golden):
  keys = golden.cases("conv/")
  assert len(keys) == 80
  worst_vs_bf16_ref = [0.0]
  for key in keys:
    _announce(key)
    x, seg = golden.get(key + "/x"), golden.get(key + "/seg")
    conv = _mk_conv(golden.get(key + "/w"), golden.get(key + "/b"))
    xd = _dev(x)
    y, cache = conv(xd, _dev(seg))
    assert torch.equal(xd.cpu(), x), "input must not be modified"
    want = golden.get(key + "/y")
    if x.dtype == torch.float32:
      assert helpers.max_rel(y, want) < F32_TOL, key
    else:
      # the reference's own bf16 tolerance for Conv1D (layers_test.py:170)
      # against the all-bf16 reference vectors: the reference's own bf16
      # tolerance for Conv1D (layers_test.py:170); tight check: widened oracle
      torch.testing.assert_close(y.cpu(), want, rtol=1e-2, atol=3e-2)
      worst_vs_bf16_ref[0] = max(worst_vs_bf16_ref[0], helpers.max_rel(y, want))
      yo, _ = R.widened_conv1d_forward(x, seg, golden.get(key + "/w"),
                                       golden.get(key + "/b"))
      assert helpers.max_rel(y, yo) < BF16_TOL, key
    assert torch.equal(cache.cpu(), golden.get(key + "/cache")), key
    y_nc, none = conv(xd, _dev(seg), return_cache=False)
    assert none is None and torch.equal(y_nc, y)
    # int32 positions give the same result
    y32, cache32 = conv(xd, _dev(seg.to(torch.int32)))
    assert torch.equal(y32, y) and torch.equal(cache32, cache)
    xs = golden.get(key + "/step_x")
    for i in range(2):
      ys, cache = conv(_dev(xs[:, i:i + 1]), _dev(seg[:, -1:] + 1 + i), cache)
      want = golden.get(key + f"/step{i}_y")
      if x.dtype == torch.float32:
        assert helpers.max_rel(ys, want) < F32_TOL, key
      else:
        torch.testing.assert_close(ys.cpu(), want, rtol=1e-2, atol=3e-2)
      assert torch.equal(cache.cpu(), golden.get(key + f"/step{i}_cache")), key
  print("conv bf16 vs the reference's all-bf16 golden: worst max-rel",
        worst_vs_bf16_ref[0])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K", [2, 4, 8])
def test_conv1d_vs_oracle(dtype, K):
  g = torch.Generator().manual_seed(200 + K)
  B, T, W = 3, 211, 130
  x = torch.randn(B, T, W, generator=g).to(dtype)
  w = (torch.randn(K, W, generator=g) * 0.3).to(dtype)
  b = (torch.randn(W, generator=g) * 0.1).to(dtype)
  seg = helpers.document_positions(B, T, 9, seed=K)
  _announce("conv", dtype, K)
  y, cache = _mk_conv(w, b)(_dev(x), _dev(seg))
  yo, co = R.widened_conv1d_forward(x, seg, w, b)
  tol = F32_TOL if dtype == torch.float32 else BF16_TOL
  assert helpers.max_rel(y, yo) < tol
  assert torch.equal(cache.cpu(), co)


# ------------------------------------------------- BlockDiagonalLinear -----


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,blocks", [(128, 1), (128, 16), (1024, 1),
                                          (1024, 16), (512, 2), (60, 3),
                                          (2560, 10), (352, 2), (600, 3),
                                          (5632, 32)])
def test_block_diagonal_linear(dtype, width, blocks):
  g = torch.Generator().manual_seed(width + blocks)
  bw = width // blocks
  x = torch.randn(1, 2, width, generator=g).to(dtype)
  x2 = torch.randn(3, 37, width, generator=g).to(dtype)
  w = (torch.randn(blocks, bw, bw, generator=g) / bw ** 0.5).to(dtype)
  b = (torch.randn(blocks, bw, generator=g) * 0.2).to(dtype)
  m = rg.BlockDiagonalLinear(width, blocks, dtype=dtype)
  m.load_state_dict({"w": w, "b": b})
  m = m.to(DEV)
  tol = F32_TOL if dtype == torch.float32 else BF16_TOL
  cases = [x, x2]
  if 128 <= bw <= 256:  # the matrix-core kernels (bf16: narrower heads
    # padded inside the tile): many row tiles, a ragged last one
    cases.append(torch.randn(5, 1231, width, generator=g).to(dtype))
  for xi in cases:
    _announce("bdl", dtype, width, blocks, tuple(xi.shape))
    want = R.block_diagonal_linear(xi.float(), w.float(), b.float())
    assert helpers.max_rel(m(_dev(xi)), want) < tol


# --------------------------------------------------------------- scan ------


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 2, 15, 16, 17, 128, 129, 1000])
def test_rnn_scan(dtype, T):
  g = torch.Generator().manual_seed(300 + T)
  B, W = 2, 200
  x = torch.randn(B, T, W, generator=g).to(dtype)
  a = torch.rand(B, T, W, generator=g).to(dtype)
  reset = torch.rand(B, T, generator=g) < 0.05
  for h0 in (None, torch.randn(B, W, generator=g)):
    _announce("rnn_scan", dtype, T, h0 is not None)
    y, h = rg.rnn_scan(_dev(x), _dev(a), _dev(reset), _dev(h0))
    yo, ho = R.rnn_scan(x, a, reset, h0)
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    assert helpers.max_rel(y, yo) < tol
    assert helpers.max_rel(h, ho) < F32_TOL
    assert h.dtype == torch.float32


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,W,mean_doc", [
    (1, 2048, 512, 0),      # one document, chunks of equal length
    (1, 4097, 256, 300),    # ragged end, document starts in and between chunks
    (3, 1100, 130, 40),     # narrow slab, last chunk shorter than the others
    (3, 8192, 2560, 1500),  # the 2B width, long rows
])
def test_scans_cut_into_chunks(dtype, B, T, W, mean_doc):
  """rg_lru_scan_fused_split / rg_linear_scan_split (sequences cut into chunks
  that run side by side, for few rows) against the one-pass kernels on the
  same inputs: the float32 state is combined in a different order, nothing
  else differs -- fp32 1e-5, bf16 outputs within one rounding of the state;
  conv cache bit for bit.  Against the oracle: the plain recurrence below
  (all but the largest shape), and the long single row of
  test_core_vs_oracle, which runs through the split path."""
  assert _lib.lib().rg_scan_split_workspace_bytes(B, T, W) > 0
  _announce("split scan", dtype, B, T, W, mean_doc)
  g = torch.Generator().manual_seed(T + W)
  x = _dev(torch.randn(B, T, W, generator=g).to(dtype))
  gx = _dev(torch.randn(B, T, W, generator=g).to(dtype))
  ga = _dev((torch.randn(B, T, W, generator=g) * 2).to(dtype))
  a_param = _dev(R.make_params(W, 1, dtype, seed=5)["a_param"])
  cw = _dev((torch.randn(4, W, generator=g) * 0.3).to(dtype))
  cb = _dev((torch.randn(W, generator=g) * 0.1).to(dtype))
  h0 = _dev(torch.randn(B, W, generator=g))
  seg = (helpers.document_positions(B, T, mean_doc, seed=T) if mean_doc
         else torch.arange(T)[None].expand(B, T).contiguous())
  seg = _dev(seg)
  tol_y = F32_TOL if dtype == torch.float32 else 2.0 ** -7
  # element by element: one bf16 unit where the state was combined in another
  # float32 order
  elt = (dict(rtol=1e-4, atol_of_max=1e-5) if dtype == torch.float32
         else dict(rtol=2.0 ** -7, atol_of_max=2e-3))
  for conv in (None, (cw, cb)):
    for start in (None, h0):
      kw = dict(h0=start, conv=conv, return_conv_cache=conv is not None)
      y1, h1, c1 = ops.lru_scan_fused(x, gx, ga, a_param, seg, split=False, **kw)
      y2, h2, c2 = ops.lru_scan_fused(x, gx, ga, a_param, seg, split=True, **kw)
      assert helpers.max_rel(y2, y1) < tol_y
      assert helpers.max_rel(h2, h1) < F32_TOL
      helpers.assert_close_elementwise(y2, y1, what="y, chunks", **elt)
      helpers.assert_close_elementwise(h2, h1, rtol=1e-4, atol_of_max=1e-5,
                                       what="h, chunks")
      if conv is not None:
        assert torch.equal(c1, c2)
      if dtype == torch.bfloat16:  # almost every output rounds the same way
        assert (y1 != y2).float().mean().item() < 0.01
  # plain recurrence with resets
  a = _dev(torch.rand(B, T, W, generator=g).to(dtype))
  reset = seg == 0
  for start in (None, h0):
    y1, h1 = ops.linear_scan(x, a, reset, start, split=False)
    y2, h2 = ops.linear_scan(x, a, reset, start, split=True)
    assert helpers.max_rel(y2, y1) < tol_y
    assert helpers.max_rel(h2, h1) < F32_TOL
    helpers.assert_close_elementwise(y2, y1, what="y, plain chunks", **elt)
    if B * T * W <= 4097 * 256:
      yo, ho = R.rnn_scan(x.cpu(), a.cpu(), reset.cpu(),
                          None if start is None else start.cpu())
      assert helpers.max_rel(y2, yo) < (F32_TOL if dtype == torch.float32
                                        else BF16_TOL)
      assert helpers.max_rel(h2, ho) < F32_TOL


def test_rnn_scan_closed_forms():
  T, W = 3000, 64
  one = torch.ones(1, T, W, device=DEV)
  noreset = torch.zeros(1, T, dtype=torch.bool, device=DEV)
  y, h = rg.rnn_scan(one, torch.full_like(one, 0.9), noreset, None)
  t = torch.arange(1, T + 1, dtype=torch.float64)
  want = (1 - 0.9 ** t) / 0.1
  assert helpers.max_rel(y[0, :, 0], want) < F32_TOL
  y, h = rg.rnn_scan(one, torch.ones_like(one), noreset, None)
  assert torch.equal(y[0, :, 5].cpu(), torch.arange(1, T + 1).float())
  y, h = rg.rnn_scan(one, torch.zeros_like(one), noreset, None)
  assert torch.equal(y, one)


# -------------------------------------------------------------- RGLRU ------


def test_rglru_golden(golden):
  keys = golden.cases("rglru/")
  assert len(keys) == 72
  worst = {torch.float32: 0.0, torch.bfloat16: 0.0}
  worst_ref_form = [-1e9]  # max of |d| - (atol + rtol*|ref|); <= 0 passes
  worst_ref_rel = [0.0]
  for key in keys:
    _announce(key)
    pkey = "/".join(key.split("/")[:3])
    prm = [golden.get(pkey + "/" + n)
           for n in ("a_param", "w_x", "b_x", "w_a", "b_a")]
    H = prm[1].shape[0]
    lru = _mk_lru(prm, H)
    x, seg = golden.get(key + "/x"), golden.get(key + "/seg")
    h0 = golden.get(key + "/h0") if golden.has(key + "/h0") else None
    y, h = lru(_dev(x), _dev(seg), _dev(h0))
    assert h.dtype == torch.float32 and y.dtype == x.dtype
    f32 = x.dtype == torch.float32
    # fp32: the reference itself.  bf16: the reference's all-bf16 arithmetic is
    # only loosely comparable (checked with its own tolerance form); the tight
    # bf16 check is against the widened oracle.
    if f32:
      e = max(helpers.max_rel(y, golden.get(key + "/y")),
              helpers.max_rel(h, golden.get(key + "/h")))
      assert e < F32_TOL, (key, e)
    else:
      # the reference's own bf16 tolerance form (layers_test.py:131)
      gold = golden.get(key + "/y").float()
      d = (y.cpu().float() - gold).abs()
      excess = (d - (3e-2 + 1e-2 * gold.abs())).max().item()
      worst_ref_form[0] = max(worst_ref_form[0], excess)
      worst_ref_rel[0] = max(worst_ref_rel[0], helpers.max_rel(y, gold))
      yo, ho = R.widened_rglru_forward(x, seg, *prm, cache=h0)
      e = max(helpers.max_rel(y, yo), helpers.max_rel(h, ho))
      assert e < BF16_TOL, (key, e)
    worst[x.dtype] = max(worst[x.dtype], e)
    xs = golden.get(key + "/step_x")
    for i in range(2):
      segi = seg[:, -1:] + 1 + i
      ys, h_new = lru(_dev(xs[:, i:i + 1]), _dev(segi), h)
      if f32:
        e = max(helpers.max_rel(ys, golden.get(key + f"/step{i}_y")),
                helpers.max_rel(h_new, golden.get(key + f"/step{i}_h")))
        assert e < F32_TOL, (key, i, e)
      else:
        yo, ho = R.widened_rglru_forward(xs[:, i:i + 1], segi, *prm,
                                         cache=h.cpu())
        e = max(helpers.max_rel(ys, yo), helpers.max_rel(h_new, ho))
        assert e < BF16_TOL, (key, i, e)
      h = h_new
    y_nc, none = lru(_dev(x), _dev(seg), _dev(h0), return_cache=False)
    assert none is None and torch.equal(y_nc, y)
  print("worst max-rel error vs fp32 golden / widened oracle", worst)
  print("bf16 vs the reference's all-bf16 golden: max-rel", worst_ref_rel[0],
        "excess over rtol=1e-2,atol=3e-2:", worst_ref_form[0])
  assert worst_ref_form[0] <= 0.0, worst_ref_form[0]


def test_rglru_golden_256_wide_heads_in_both_forms(golden):
  """The reference-written bf16 RG-LRU vectors with a 256-wide head, through
  BOTH forms the library may pick for such a layer (the choice depends on the
  batch size, and the two forms round the gate pre-activations differently:
  the gate GEMM + scan pair to bf16 like the reference's modules, the single
  kernel keeps them in float32): each against the reference's own outputs in
  the reference's tolerance form (layers_test.py:131) and against the widened
  oracle; the two forms against each other to a bf16 ulp or two."""
  keys = [k for k in golden.cases("rglru/") if "/bfloat16/W256H1/" in k]
  assert len(keys) >= 10
  for key in keys:
    _announce(key)
    pkey = "/".join(key.split("/")[:3])
    a_param, w_x, b_x, w_a, b_a = (
        golden.get(pkey + "/" + n)
        for n in ("a_param", "w_x", "b_x", "w_a", "b_a"))
    x, seg = golden.get(key + "/x"), golden.get(key + "/seg")
    h0 = golden.get(key + "/h0") if golden.has(key + "/h0") else None
    W = x.shape[-1]
    P = [_dev(t) for t in (w_x, b_x, w_a, b_a, a_param)]
    # the single kernel with a conv that hands x through (w3 = 1)
    ident = torch.zeros(4, W, dtype=x.dtype)
    ident[3] = 1.0
    y1, h1, _ = ops.recurrent_prefill(
        _dev(x), _dev(seg), _dev(ident), _dev(torch.zeros(W, dtype=x.dtype)),
        P[0], P[1], P[2], P[3], P[4], h0=_dev(h0), split=False)
    gx, ga = ops.gates_gemm(_dev(x), P[0], P[1], P[2], P[3])
    y2, h2, _ = ops.lru_scan_fused(_dev(x), gx, ga, P[4], _dev(seg),
                                   h0=_dev(h0))
    gold_y = golden.get(key + "/y").float()
    gold_h = golden.get(key + "/h").float()
    yo, ho = R.widened_rglru_forward(x, seg, a_param, w_x, b_x, w_a, b_a,
                                     cache=h0)
    for name, y, h in (("single kernel", y1, h1), ("two kernels", y2, h2)):
      d = (y.cpu().float() - gold_y).abs()
      assert (d <= 3e-2 + 1e-2 * gold_y.abs()).all(), (key, name)
      dh = (h.cpu() - gold_h).abs()
      assert (dh <= 3e-2 + 1e-2 * gold_h.abs()).all(), (key, name)
      assert helpers.max_rel(y, yo) < BF16_TOL, (key, name)
      assert helpers.max_rel(h, ho) < BF16_TOL, (key, name)
    assert (y1.float() - y2.float()).abs().max().item() <= 0.0625, key
    assert helpers.max_rel(h1, h2) < 2e-3, key


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,W,H,mean_doc,with_h0", [
    (13, 200, 2560, 10, 40, False),  # 130 (row, head) pairs: the single kernel
    (26, 65, 1280, 5, 9, True),      # ... with a start state, ragged T
    (1, 4100, 512, 2, 700, True),    # one long row: the single kernel in chunks
    (2, 300, 512, 2, 50, True),      # few pairs: gate GEMM + scan
    (3, 77, 384, 6, 11, False),      # heads that are not 256 wide
])
def test_rglru_alone_every_route(dtype, B, T, W, H, mean_doc, with_h0):
  """RGLRU.forward on its own (layers.py:313-365) through rg_recurrent_core
  without conv weights, on each set of kernels the library may pick."""
  p = R.make_params(W, H, dtype, seed=T + B)
  prm = [p[n] for n in ("a_param", "w_x", "b_x", "w_a", "b_a")]
  lru = _mk_lru(prm, H)
  g = torch.Generator().manual_seed(11 * T + W)
  x = torch.randn(B, T, W, generator=g).to(dtype)
  h0 = torch.randn(B, W, generator=g) if with_h0 else None
  seg = helpers.document_positions(B, T, mean_doc, seed=T + W)
  seg[0, -1] = 0
  _announce("rglru alone", dtype, B, T, W, H, with_h0)
  y, h = lru(_dev(x), _dev(seg), _dev(h0))
  ref = (R.rglru_forward if dtype == torch.float32
         else R.widened_rglru_forward)
  yo, ho = ref(x, seg, *prm, cache=h0)
  tol = F32_TOL if dtype == torch.float32 else BF16_TOL
  ey, eh = helpers.max_rel(y, yo), helpers.max_rel(h, ho)
  print("max-rel y", ey, "h", eh)
  assert ey < tol and eh < tol
  elt = (dict(rtol=1e-4, atol_of_max=1e-5) if dtype == torch.float32
         else dict(rtol=1e-2, atol_of_max=2e-3))
  helpers.assert_close_elementwise(y, yo, what="y", **elt)
  # the same values as the gate GEMM and the scan called one after the other
  gx, ga = ops.gates_gemm(_dev(x), *[_dev(t) for t in prm[1:]])
  y2, h2, _ = ops.lru_scan_fused(_dev(x), gx, ga, _dev(prm[0]), _dev(seg),
                                 h0=_dev(h0))
  assert helpers.max_rel(y, y2) < tol and helpers.max_rel(h, h2) < tol
  y_nc, none = lru(_dev(x), _dev(seg), _dev(h0), return_cache=False)
  assert none is None and torch.equal(y_nc, y)
  # the join with a gate branch works without conv weights too: the same
  # values as the separate pass, bit for bit
  gb = torch.randn(B, T, W, generator=g).to(dtype)
  yj, hj, none = ops.recurrent_core(
      _dev(x), _dev(seg), None, None, *[_dev(t) for t in prm[1:]],
      _dev(prm[0]), h0=_dev(h0), gate_branch=_dev(gb))
  assert none is None and torch.equal(hj, h)
  assert torch.equal(yj, ops.gelu_mul(y, _dev(gb)))


# ------------------------------------------------- fused conv -> rg_lru ----


def _core_case(dtype, B, T, W, H, seg, seed, bias_std=0.2):
  p = R.make_params(W, H, dtype, seed=seed, gate_bias_std=bias_std)
  g = torch.Generator().manual_seed(seed + 1)
  x = torch.randn(B, T, W, generator=g).to(dtype)
  blk = _block(p, W, H, dtype)
  y, cache = rg.recurrent_core(blk.conv_1d, blk.rg_lru, _dev(x), _dev(seg))
  if dtype == torch.float32:
    yo, co = R.recurrent_core(x, seg, p)
  else:
    yo, co = R.widened_recurrent_core(x, seg, p)
  return p, x, blk, (y, cache), (yo, co)


def test_recurrent_core_shape_sweep():
  """Forty shapes drawn from a fixed seed -- head widths 64 to 256, one to four
  heads, one to 150 rows, one to 1700 tokens, both dtypes, int32 and int64
  positions, rows that start at position -1 (left padding), 0 or inside a
  document -- through rg_recurrent_core (whatever kernels it picks) against
  the oracle, with and without the join of the gate branch."""
  import random
  rnd = random.Random(20240607)
  for case in range(40):
    dtype = rnd.choice([torch.float32, torch.bfloat16])
    bw = rnd.choice([64, 128, 256, 256, 256])
    H = rnd.choice([1, 2, 3, 4])
    W = bw * H
    B = rnd.choice([1, 2, 5, 33, 70, 150]) if bw == 256 else rnd.choice([1, 3, 9])
    T = rnd.choice([1, 2, 3, 5, 63, 64, 65, 200, 513, 1700])
    if B * T * W > 40e6:
      T = 65
    p = R.make_params(W, H, dtype, seed=500 + case, gate_bias_std=0.3)
    g = torch.Generator().manual_seed(900 + case)
    x = torch.randn(B, T, W, generator=g).to(dtype)
    seg = helpers.document_positions(B, T, rnd.choice([4, 50, 4000]),
                                     seed=case)
    first = rnd.choice(["zero", "pad", "inside"])
    if first == "pad" and T > 3:
      seg[:, 2:] = seg[:, :-2].clone()
      seg[:, :2] = -1
    elif first == "inside":
      seg[0, 0] = 11
    if rnd.random() < 0.5:
      seg = seg.to(torch.int32)
    P = {k: _dev(v) for k, v in p.items()}
    joined = rnd.random() < 0.5
    gate = torch.randn(B, T, W, generator=g).to(dtype) if joined else None
    _announce(f"sweep {case}: {dtype} B{B} T{T} W{W} H{H} {first} "
              f"{seg.dtype} joined={joined}")
    y, h, c = ops.recurrent_core(
        _dev(x), _dev(seg), P["conv_w"], P["conv_b"], P["w_x"], P["b_x"],
        P["w_a"], P["b_a"], P["a_param"],
        gate_branch=None if gate is None else _dev(gate))
    ref = (R.recurrent_core if dtype == torch.float32
           else R.widened_recurrent_core)
    yo, co = ref(x, seg.to(torch.int64), p)
    if joined:
      gelu = torch.nn.functional.gelu(gate.float(), approximate="tanh")
      yo = (yo.float() * gelu.to(dtype).float()).to(dtype)
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    what = f"case {case}"
    assert helpers.max_rel(h, co.rg_lru_state) < tol, what
    assert torch.equal(c.cpu(), co.conv1d_state), what
    if dtype == torch.float32:
      assert helpers.max_rel(y, yo) < (2e-5 if joined else tol), what
    else:
      helpers.assert_close_elementwise(y, yo, rtol=2e-2, atol_of_max=4e-3,
                                       what=what)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T", [(2, 0), (0, 5)])
def test_empty_inputs(dtype, B, T):
  """No tokens or no rows: nothing is launched, outputs are empty tensors of
  the right shape, and the state is what the reference's empty loop leaves
  (layers.py:181-189: h0 or zeros; :526-527: a conv state of zeros)."""
  W, H = 512, 2
  p = R.make_params(W, H, dtype, seed=4)
  blk = _block(p, W, H, dtype)
  x = _dev(torch.zeros(B, T, W, dtype=dtype))
  seg = _dev(torch.zeros(B, T, dtype=torch.int64))
  y, cache = rg.recurrent_core(blk.conv_1d, blk.rg_lru, x, seg)
  assert y.shape == (B, T, W) and y.dtype == dtype
  assert cache.rg_lru_state.shape == (B, W)
  assert cache.rg_lru_state.dtype == torch.float32
  assert cache.conv1d_state.shape == (B, 3, W)
  assert not cache.rg_lru_state.any() and not cache.conv1d_state.any()
  out, cstate = blk.conv_1d(x, seg)
  assert out.shape == (B, T, W) and cstate.shape == (B, 3, W)
  h0 = _dev(torch.randn(B, W))
  y2, h2 = blk.rg_lru(x, seg, h0)
  assert y2.shape == (B, T, W) and torch.equal(h2, h0)
  y3, h3 = rg.rnn_scan(x, x, seg == 0, h0)
  assert y3.shape == (B, T, W) and torch.equal(h3, h0)


def test_config1_fp32_parity():
  """Benchmark configuration 1: B1 T512 W2560 H10 fp32, segment_pos = arange."""
  B, T, W, H = 1, 512, 2560, 10
  seg = torch.arange(T)[None]
  p = R.make_params(W, H, torch.float32, seed=1101)
  g = torch.Generator().manual_seed(1001)
  x = torch.randn(B, T, W, generator=g)
  blk = _block(p, W, H, torch.float32)
  _announce("config1")
  y, cache = rg.recurrent_core(blk.conv_1d, blk.rg_lru, _dev(x), _dev(seg))
  yo, co = R.recurrent_core(x, seg, p)
  ey, eh = helpers.max_rel(y, yo), helpers.max_rel(cache.rg_lru_state,
                                                   co.rg_lru_state)
  print("config1 max-rel y", ey, "h", eh)
  assert ey < F32_TOL and eh < F32_TOL
  assert torch.equal(cache.conv1d_state.cpu(), co.conv1d_state)
  # module-by-module path gives the same numbers as the fused path
  xc, cstate = blk.conv_1d(_dev(x), _dev(seg))
  y2, h2 = blk.rg_lru(xc, _dev(seg))
  assert helpers.max_rel(y2, yo) < F32_TOL
  assert torch.equal(cstate, cache.conv1d_state)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,W,H,mean_doc", [
    (2, 700, 512, 2, 60),     # bw 256: MFMA path in bf16, ragged T
    (3, 129, 768, 3, 7),      # dense document starts
    (1, 2050, 256, 1, 500),   # long row, many steps
    (2, 33, 384, 6, 5),       # bw 64: generic GEMM
    (2, 300, 704, 4, 50),     # bw 176 (the paper models' heads): padded MFMA
    (1, 130, 5632, 32, 40),   # ... at their width
    (2, 3, 256, 1, 2),        # shorter than the conv
    (5, 1, 256, 1, 1),        # single token, every row starts a document
    (2, 64, 130, 1, 16),      # width not a multiple of the slab
    (2, 40, 65, 1, 16),       # odd width: one channel per lane
])
def test_core_vs_oracle(dtype, B, T, W, H, mean_doc):
  seg = helpers.document_positions(B, T, mean_doc, seed=T + W)
  if T > 4:
    seg[0, -1] = 0   # document start in the last position
    seg[-1, -2] = 0  # ... and in the one before
  _announce("core", dtype, B, T, W, H)
  p, x, blk, (y, cache), (yo, co) = _core_case(dtype, B, T, W, H, seg, seed=T)
  tol = F32_TOL if dtype == torch.float32 else BF16_TOL
  ey = helpers.max_rel(y, yo)
  eh = helpers.max_rel(cache.rg_lru_state, co.rg_lru_state)
  print("max-rel y", ey, "h", eh)
  assert ey < tol and eh < tol
  elt = (dict(rtol=1e-4, atol_of_max=1e-5) if dtype == torch.float32
         else dict(rtol=1e-2, atol_of_max=2e-3))
  helpers.assert_close_elementwise(y, yo, what="y", **elt)
  helpers.assert_close_elementwise(cache.rg_lru_state, co.rg_lru_state,
                                   what="h", **elt)
  assert torch.equal(cache.conv1d_state.cpu(), co.conv1d_state)
  assert cache.rg_lru_state.dtype == torch.float32
  assert cache.conv1d_state.dtype == dtype
  # sampler-style positions: left padding is -1, int32
  seg32 = torch.cat([torch.full((B, T // 3), -1), torch.arange(T - T // 3)
                     .expand(B, -1)], 1).to(torch.int32)
  y, cache = rg.recurrent_core(blk.conv_1d, blk.rg_lru, _dev(x), _dev(seg32))
  ref = R.recurrent_core if dtype == torch.float32 else R.widened_recurrent_core
  yo, co = ref(x, seg32, p)
  assert helpers.max_rel(y, yo) < tol
  assert helpers.max_rel(cache.rg_lru_state, co.rg_lru_state) < tol
  assert torch.equal(cache.conv1d_state.cpu(), co.conv1d_state)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_prefill_then_decode(dtype):
  """Prefill, then 6 single-token steps with the carried cache (config 4 in
  small), and the reference's own invariant prefill(T) == prefill(T-1) o step."""
  B, T, W, H, steps = 4, 77, 512, 2, 6
  seg = torch.arange(T).expand(B, T).clone()
  p = R.make_params(W, H, dtype, seed=77, gate_bias_std=0.2)
  g = torch.Generator().manual_seed(78)
  x = torch.randn(B, T + steps, W, generator=g).to(dtype)
  blk = _block(p, W, H, dtype)
  ref = R.recurrent_core if dtype == torch.float32 else R.widened_recurrent_core
  tol = F32_TOL if dtype == torch.float32 else BF16_TOL
  _announce("decode", dtype)
  y, cache = rg.recurrent_core(blk.conv_1d, blk.rg_lru, _dev(x[:, :T]),
                               _dev(seg))
  yo, co = ref(x[:, :T], seg, p)
  for i in range(steps):
    pos = torch.full((B, 1), T + i)
    xi = x[:, T + i:T + i + 1]
    y, cache = rg.recurrent_core(blk.conv_1d, blk.rg_lru, _dev(xi), _dev(pos),
                                 cache)
    yo, co = ref(xi, pos, p, co)
    assert helpers.max_rel(y, yo) < tol, i
    assert helpers.max_rel(cache.rg_lru_state, co.rg_lru_state) < tol, i
    assert torch.equal(cache.conv1d_state.cpu(), co.conv1d_state), i
  # invariant
  full = torch.arange(T + steps).expand(B, -1)
  y_full, c_full = rg.recurrent_core(blk.conv_1d, blk.rg_lru, _dev(x),
                                     _dev(full))
  assert helpers.max_rel(y, y_full[:, -1:]) < tol
  assert helpers.max_rel(cache.rg_lru_state, c_full.rg_lru_state) < tol
  assert torch.equal(cache.conv1d_state, c_full.conv1d_state)


def test_recurrent_block_module():
  """RecurrentBlock end to end (linear_x/y/out in torch) against the oracle
  core wrapped in the same torch linears on the CPU, fp32."""
  B, T, width, H = 2, 50, 256, 1
  torch.manual_seed(5)
  blk = rg.RecurrentBlock(width=width, num_heads=H, dtype=torch.float32)
  sd = {k: v.clone() for k, v in blk.state_dict().items()}
  x = torch.randn(B, T, width)
  seg = helpers.document_positions(B, T, 20, seed=3)
  p = {"conv_w": sd["conv_1d.w"], "conv_b": sd["conv_1d.b"],
       "a_param": sd["rg_lru.a_param"], "w_x": sd["rg_lru.input_gate.w"],
       "b_x": sd["rg_lru.input_gate.b"], "w_a": sd["rg_lru.a_gate.w"],
       "b_a": sd["rg_lru.a_gate.b"]}
  lin = torch.nn.functional.linear
  yb = torch.nn.functional.gelu(lin(x, sd["linear_y.weight"],
                                    sd["linear_y.bias"]), approximate="tanh")
  xb = lin(x, sd["linear_x.weight"], sd["linear_x.bias"])
  core, cache_o = R.recurrent_core(xb, seg, p)
  want = lin(core * yb, sd["linear_out.weight"], sd["linear_out.bias"])
  blk = blk.to(DEV)
  got, cache = blk(_dev(x), _dev(seg))
  assert helpers.max_rel(got, want) < 1e-4  # torch GPU vs CPU linears
  assert isinstance(cache, rg.RecurrentBlockCache)
  assert helpers.max_rel(cache.rg_lru_state, cache_o.rg_lru_state) < 1e-4
  init = rg.RecurrentBlock.init_cache(B, width, torch.float32, device=DEV)
  assert init.rg_lru_state.dtype == torch.float32
  assert init.conv1d_state.shape == (B, 3, width)
  got1, c1 = blk(_dev(x[:, :1]), _dev(seg[:, :1]), init)
  assert helpers.max_rel(got1, want[:, :1]) < 1e-4


def test_recurrent_block_module_joined_kernel(monkeypatch):
  """bf16 RecurrentBlock with enough (row, head) pairs for the prefill kernel
  that also applies the x * gelu(y) join: the block hands its gate branch to
  the one library call (no gelu_mul call of its own), and the block output is
  bit for bit what the separate pass gives."""
  B, T, width, H = 80, 70, 512, 2  # 160 pairs
  torch.manual_seed(6)
  blk = rg.RecurrentBlock(width=width, num_heads=H,
                          dtype=torch.bfloat16).to(DEV)
  with torch.no_grad():
    blk.linear_y.bias.normal_(0, 0.3)
    blk.rg_lru.input_gate.b.normal_(0, 0.3)
  x = _dev(torch.randn(B, T, width).to(torch.bfloat16))
  seg = _dev(helpers.document_positions(B, T, 25, seed=4))
  calls = []
  real_gelu_mul, real_core = ops.gelu_mul, ops.recurrent_core
  monkeypatch.setattr(ops, "gelu_mul",
                      lambda *a, **k: calls.append("gelu_mul") or
                      real_gelu_mul(*a, **k))
  monkeypatch.setattr(ops, "recurrent_core",
                      lambda *a, **k: calls.append(
                          ("core", k.get("gate_branch") is not None)) or
                      real_core(*a, **k))
  got, cache = blk(x, seg)
  assert calls == [("core", True)], calls
  # whole rows in the single kernel: no workspace, the join is inside it
  assert _lib.lib().rg_recurrent_core_workspace_bytes(B, T, width, H, 1) == 0
  # the same block with the join as a pass of its own
  yb = blk.linear_y(x)
  core, cache2 = rg.recurrent_core(blk.conv_1d, blk.rg_lru, blk.linear_x(x),
                                   seg)
  want = blk.linear_out(real_gelu_mul(core, yb))
  assert torch.equal(got, want)
  assert torch.equal(cache.rg_lru_state, cache2.rg_lru_state)
  assert torch.equal(cache.conv1d_state, cache2.conv1d_state)


# ------------------------------------------- single-launch prefill kernel --


@pytest.mark.parametrize("B,T,W,H,mean_doc,seg_dtype,with_h0", [
    (1, 64, 256, 1, None, torch.int64, False),
    (1, 128, 256, 1, None, torch.int64, False),
    (2, 200, 512, 2, 50, torch.int64, True),
    (3, 1, 256, 1, None, torch.int32, True),
    (2, 3, 512, 2, 2, torch.int32, False),
    (2, 65, 256, 1, 16, torch.int64, True),
    (2, 1000, 768, 3, 250, torch.int32, False),
    (1, 130, 256, 1, 3, torch.int64, False),   # documents of a few tokens
    (130, 70, 256, 1, 20, torch.int64, False),  # more workgroups than CUs/2
    (2, 100, 256, 1, -7, torch.int32, False),   # left padding: positions < 0
    # few (row, head) pairs, long rows: the sequences run as chunks
    (1, 1600, 512, 2, 200, torch.int64, True),
    (2, 2048, 256, 1, None, torch.int64, False),
    (1, 1777, 768, 3, 100, torch.int32, True),
    (3, 1540, 256, 1, 7, torch.int64, False),
    (1, 8192, 256, 1, 1024, torch.int64, True),  # 64 chunks of two tiles
    (2, 1700, 256, 1, -300, torch.int32, False),  # chunks, left padding
])
def test_recurrent_prefill_single_launch(B, T, W, H, mean_doc, seg_dtype,
                                         with_h0):
  """rg_recurrent_prefill(_split) against the oracle (bf16 tolerance, also
  element by element) and against the two-kernel form.  The single-launch
  kernel keeps the gate pre-activations in float32 where the two-kernel form
  rounds them to bf16 on their way through memory (as the reference's modules
  do), so the two agree to a bf16 ulp or two, not bit for bit."""
  _announce("recurrent_prefill", B, T, W, H, mean_doc, seg_dtype, with_h0)
  seed = 7000 + T
  p = R.make_params(W, H, torch.bfloat16, seed=seed, gate_bias_std=0.5)
  g = torch.Generator().manual_seed(seed + 1)
  x = torch.randn(B, T, W, generator=g).to(torch.bfloat16)
  if mean_doc is None:
    seg = torch.arange(T).expand(B, T).contiguous()
  elif mean_doc < 0:  # the sampler's left padding: -1 ... then 0, 1, 2, ...
    seg = (torch.arange(T) + mean_doc).clamp(min=-1).expand(B, T).contiguous()
  else:
    seg = helpers.document_positions(B, T, mean_doc, seed=seed)
  h0 = torch.randn(B, W, generator=g) if with_h0 else None
  P = {k: _dev(v) for k, v in p.items()}
  xd, segd = _dev(x), _dev(seg.to(seg_dtype))
  h0d = None if h0 is None else _dev(h0)
  assert ops.recurrent_prefill_supported(xd, H)
  y, h, cache = ops.recurrent_prefill(
      xd, segd, P["conv_w"], P["conv_b"], P["w_x"], P["b_x"], P["w_a"],
      P["b_a"], P["a_param"], h0=h0d)
  gx, ga = ops.gates_gemm(xd, P["w_x"], P["b_x"], P["w_a"], P["b_a"],
                          conv=(segd, P["conv_w"], P["conv_b"]))
  y2, h2, cache2 = ops.lru_scan_fused(
      xd, gx, ga, P["a_param"], segd, h0=h0d,
      conv=(P["conv_w"], P["conv_b"]), return_conv_cache=True)
  assert helpers.max_rel(y, y2) < BF16_TOL
  assert helpers.max_rel(h, h2) < BF16_TOL
  assert torch.equal(cache, cache2)
  xc, cc = R.widened_conv1d_forward(x, seg, p["conv_w"], p["conv_b"])
  yo, ho = R.widened_rglru_forward(xc, seg, p["a_param"], p["w_x"], p["b_x"],
                                   p["w_a"], p["b_a"], cache=h0)
  assert helpers.max_rel(y, yo) < BF16_TOL
  assert helpers.max_rel(h, ho) < BF16_TOL
  helpers.assert_close_elementwise(y, yo, what="y")
  helpers.assert_close_elementwise(h, ho, what="h")
  assert torch.equal(cache.cpu(), cc)
  # whole rows and rows cut into chunks: the same arithmetic per token, the
  # state crosses chunk boundaries in another float32 association
  y1, h1, cache1 = ops.recurrent_prefill(
      xd, segd, P["conv_w"], P["conv_b"], P["w_x"], P["b_x"], P["w_a"],
      P["b_a"], P["a_param"], h0=h0d, split=False)
  assert torch.equal(cache1, cache)
  assert helpers.max_rel(h1, h) < 1e-5
  assert (y1 != y).float().mean().item() < 2e-3
  assert (y1.float() - y.float()).abs().max().item() <= 0.0625
  if not ops.recurrent_prefill_chunked(B, T, W, H):
    assert torch.equal(y1, y) and torch.equal(h1, h)


@pytest.mark.parametrize("B,T,W,H,mean_doc", [
    (2, 200, 512, 2, 37),      # whole rows, ragged last tile, documents
    (1, 70, 256, 1, None),
    (1, 2048, 512, 2, 300),    # rows in chunks
    (3, 1600, 768, 3, None),
    (40, 130, 1024, 4, 50),    # 160 (row, head) pairs
    (2, 449, 512, 2, 60),      # the shortest rows that are cut into chunks
    (1, 513, 256, 1, None),
    (1, 4096, 2560, 10, 1024), # chunks at the 2B width
    (5, 3000, 2560, 10, 5),    # ... ragged, documents of a few tokens
    (6, 1500, 768, 3, 300),
])
def test_prefill_joined_with_gate_branch(B, T, W, H, mean_doc):
  """rg_recurrent_prefill_gelu_mul (the block's x * gelu(y) join applied where
  the prefill kernel stores its output) against the same kernel followed by
  rg_gelu_mul: bit for bit, also with the output written over the gate branch;
  state outputs identical."""
  _announce("prefill joined", B, T, W, H, mean_doc)
  seed = 7300 + T
  p = R.make_params(W, H, torch.bfloat16, seed=seed, gate_bias_std=0.5)
  g = torch.Generator().manual_seed(seed + 1)
  x = _dev(torch.randn(B, T, W, generator=g).to(torch.bfloat16))
  gate = _dev((torch.randn(B, T, W, generator=g) * 2).to(torch.bfloat16))
  seg = (torch.arange(T).expand(B, T).contiguous() if mean_doc is None
         else helpers.document_positions(B, T, mean_doc, seed=seed))
  segd = _dev(seg)
  P = {k: _dev(v) for k, v in p.items()}
  args = (x, segd, P["conv_w"], P["conv_b"], P["w_x"], P["b_x"], P["w_a"],
          P["b_a"], P["a_param"])
  y, h, cache = ops.recurrent_prefill(*args)
  want = ops.gelu_mul(y, gate)
  got, h2, cache2 = ops.recurrent_prefill(*args, gate_branch=gate)
  assert torch.equal(got, want)
  assert torch.equal(h2, h) and torch.equal(cache2, cache)
  # the reference's op sequence on the same values
  ref = (y.float() * torch.nn.functional.gelu(
      gate.float(), approximate="tanh").to(torch.bfloat16).float()).to(
          torch.bfloat16)
  assert helpers.max_rel(got, ref) < BF16_TOL
  # through the C ABI with the output over the gate branch
  lib = _lib.lib()
  need = lib.rg_recurrent_prefill_split_workspace_bytes(B, T, W, H)
  ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
  over = gate.clone()
  ptr = lambda t: t.data_ptr()
  _lib.check(lib.rg_recurrent_prefill_gelu_mul(
      ptr(x), ptr(over), ptr(segd), 1, ptr(P["conv_w"]), ptr(P["conv_b"]),
      ptr(P["w_x"]), ptr(P["b_x"]), ptr(P["w_a"]), ptr(P["b_a"]), None,
      ptr(P["a_param"]), None, ptr(over), None, None,
      ptr(ws) if need else None, need, B, T, W, H, 1, None))
  torch.cuda.synchronize()
  assert torch.equal(over, want)
  # refused where the plain call is
  xf = x.float()
  rc = lib.rg_recurrent_prefill_gelu_mul(
      ptr(xf), ptr(gate), ptr(segd), 1, ptr(P["conv_w"]), ptr(P["conv_b"]),
      ptr(P["w_x"]), ptr(P["b_x"]), ptr(P["w_a"]), ptr(P["b_a"]), None,
      ptr(P["a_param"]), None, ptr(over), None, None, None, 0, B, T, W, H, 0,
      None)
  assert rc == -2


@pytest.mark.parametrize("B,W,H,in_place", [(1, 256, 1, False),
                                              (5, 512, 2, True),
                                              (33, 256, 1, False),
                                              (70, 768, 3, True)])
def test_recurrent_step_single_launch(B, W, H, in_place):
  """rg_recurrent_step_packed (decode, one launch on re-laid-out gate weights)
  against rg_recurrent_step (conv step + gate GEMM + scan step, same
  arithmetic: bit for bit) and the oracle, over three chained steps with a
  position 0 (state reset) in some rows."""
  _announce("recurrent_step packed", B, W, H, in_place)
  seed = 8100 + B
  p = R.make_params(W, H, torch.bfloat16, seed=seed, gate_bias_std=0.5)
  P = {k: _dev(v) for k, v in p.items()}
  g = torch.Generator().manual_seed(seed + 1)
  h = torch.randn(B, W, generator=g)
  cc = torch.randn(B, 3, W, generator=g).to(torch.bfloat16)
  hd, ccd = _dev(h), _dev(cc)          # single-launch chain
  h3, cc3 = _dev(h), _dev(cc)          # three-launch chain
  ho, cco = h.clone(), cc.clone()      # oracle chain
  lib = _lib.lib()
  for step in range(3):
    x = torch.randn(B, 1, W, generator=g).to(torch.bfloat16)
    seg = torch.full((B, 1), 40 + step, dtype=torch.int64)
    seg[step % B, 0] = 0  # one row starts a document
    xd, segd = _dev(x), _dev(seg)
    y, hd, ccd = ops.recurrent_step(xd, segd, ccd, hd, P["conv_w"],
                                    P["conv_b"], P["w_x"], P["b_x"], P["w_a"],
                                    P["b_a"], P["a_param"], in_place=in_place)
    # three-launch form through the C ABI
    y3 = torch.empty_like(xd)
    h3n, cc3n = torch.empty_like(h3), torch.empty_like(cc3)
    ws = torch.empty(lib.rg_recurrent_step_workspace_bytes(B, W, 1),
                     dtype=torch.uint8, device=DEV)
    ptr = lambda t: t.data_ptr()
    _lib.check(lib.rg_recurrent_step(
        ptr(xd), ptr(segd), 1, ptr(cc3), ptr(cc3n), ptr(h3), ptr(h3n),
        ptr(P["conv_w"]), ptr(P["conv_b"]), ptr(P["w_x"]), ptr(P["b_x"]),
        ptr(P["w_a"]), ptr(P["b_a"]), ptr(P["a_param"]), ptr(y3), ptr(ws),
        ws.numel(), B, W, H, 1, torch.cuda.current_stream().cuda_stream))
    h3, cc3 = h3n, cc3n
    assert torch.equal(y, y3) and torch.equal(hd, h3) and torch.equal(ccd, cc3)
    xc, cco = R.widened_conv1d_forward(x, seg, p["conv_w"], p["conv_b"],
                                       cache=cco)
    yo, ho = R.widened_rglru_forward(xc, seg, p["a_param"], p["w_x"], p["b_x"],
                                     p["w_a"], p["b_a"], cache=ho)
    assert helpers.max_rel(y, yo) < BF16_TOL
    assert helpers.max_rel(hd, ho) < BF16_TOL
    helpers.assert_close_elementwise(y, yo, what=f"y, step {step}")
    helpers.assert_close_elementwise(hd, ho, what=f"h, step {step}")
    assert torch.equal(ccd.cpu(), cco)


@pytest.mark.parametrize("B,T,W,H,mean_doc,with_h0", [
    (3, 150, 512, 2, 40, False), (2, 1000, 768, 3, 100, True),
    (1, 31, 256, 1, 5, False), (2, 4096, 1024, 4, 500, True)])
def test_recurrent_prefill_without_packed_weights(B, T, W, H, mean_doc, with_h0):
  """rg_recurrent_prefill with w_packed == NULL re-lays the gate weights out
  inside the kernel: same result, bit for bit, as with the packed buffer.

  The two calls also run two different kernels -- with packed weights whole
  rows go to the form with two waves per SIMD, without them to the form with
  one -- so this is the check that the two forms compute the same thing."""
  p = R.make_params(W, H, torch.bfloat16, seed=61, gate_bias_std=0.5)
  P = {k: _dev(v) for k, v in p.items()}
  g = torch.Generator().manual_seed(62)
  x = _dev(torch.randn(B, T, W, generator=g).to(torch.bfloat16))
  seg = _dev(helpers.document_positions(B, T, mean_doc, seed=63))
  h0 = _dev(torch.randn(B, W, generator=g)) if with_h0 else None
  y1, h1, c1 = ops.recurrent_prefill(x, seg, P["conv_w"], P["conv_b"],
                                     P["w_x"], P["b_x"], P["w_a"], P["b_a"],
                                     P["a_param"], h0=h0, split=False)
  y2 = torch.empty_like(x)
  h2 = torch.empty(B, W, dtype=torch.float32, device=DEV)
  c2 = x.new_empty(B, 3, W)
  ptr = lambda t: t.data_ptr()
  _lib.check(_lib.lib().rg_recurrent_prefill(
      ptr(x), ptr(seg), 1, ptr(P["conv_w"]), ptr(P["conv_b"]), ptr(P["w_x"]),
      ptr(P["b_x"]), ptr(P["w_a"]), ptr(P["b_a"]), None, ptr(P["a_param"]),
      ptr(h0) if with_h0 else None, ptr(y2), ptr(h2), ptr(c2), B, T, W, H, 1,
      torch.cuda.current_stream().cuda_stream))
  assert torch.equal(y1, y2) and torch.equal(h1, h2) and torch.equal(c1, c2)


@pytest.mark.parametrize("B,T,W,H,mean_doc,with_h0", [
    (1, 8192, 2560, 10, 0, False), (4, 4096, 512, 2, 300, True),
    (2, 3000, 768, 3, 50, True)])
def test_recurrent_prefill_in_chunks_without_packed_weights(B, T, W, H,
                                                            mean_doc, with_h0):
  """Rows cut into chunks (rg_recurrent_prefill_split): with and without the
  packed weights, i.e. through the kernel form with two waves per SIMD and
  the form with one -- same chunk plan, same arithmetic, same bits."""
  lib = _lib.lib()
  need = lib.rg_recurrent_prefill_split_workspace_bytes(B, T, W, H)
  assert need > 0, "this shape is meant to be cut into chunks"
  p = R.make_params(W, H, torch.bfloat16, seed=71, gate_bias_std=0.5)
  P = {k: _dev(v) for k, v in p.items()}
  g = torch.Generator().manual_seed(72)
  x = _dev(torch.randn(B, T, W, generator=g).to(torch.bfloat16))
  if mean_doc:
    seg = _dev(helpers.document_positions(B, T, mean_doc, seed=73))
  else:
    seg = _dev(torch.arange(T, dtype=torch.int64).repeat(B, 1))
  h0 = _dev(torch.randn(B, W, generator=g)) if with_h0 else None
  y1, h1, c1 = ops.recurrent_prefill(x, seg, P["conv_w"], P["conv_b"],
                                     P["w_x"], P["b_x"], P["w_a"], P["b_a"],
                                     P["a_param"], h0=h0, split=True)
  y2 = torch.empty_like(x)
  h2 = torch.empty(B, W, dtype=torch.float32, device=DEV)
  c2 = x.new_empty(B, 3, W)
  ws = torch.empty(need, dtype=torch.uint8, device=DEV)
  ptr = lambda t: t.data_ptr()
  _lib.check(lib.rg_recurrent_prefill_split(
      ptr(x), ptr(seg), 1, ptr(P["conv_w"]), ptr(P["conv_b"]), ptr(P["w_x"]),
      ptr(P["b_x"]), ptr(P["w_a"]), ptr(P["b_a"]), None, ptr(P["a_param"]),
      ptr(h0) if with_h0 else None, ptr(y2), ptr(h2), ptr(c2), ptr(ws), need,
      B, T, W, H, 1, torch.cuda.current_stream().cuda_stream))
  assert torch.equal(y1, y2) and torch.equal(h1, h2) and torch.equal(c1, c2)


@pytest.mark.parametrize("B,T,W,H", [(3, 150, 512, 2), (1, 2048, 512, 2)])
def test_recurrent_prefill_joined_without_packed_weights(B, T, W, H):
  """The block's GELU join inside the kernel (rg_recurrent_prefill_gelu_mul),
  whole rows and rows in chunks, through both kernel forms: same bits."""
  lib = _lib.lib()
  need = lib.rg_recurrent_prefill_split_workspace_bytes(B, T, W, H)
  p = R.make_params(W, H, torch.bfloat16, seed=81, gate_bias_std=0.5)
  P = {k: _dev(v) for k, v in p.items()}
  g = torch.Generator().manual_seed(82)
  x = _dev(torch.randn(B, T, W, generator=g).to(torch.bfloat16))
  gate = _dev(torch.randn(B, T, W, generator=g).to(torch.bfloat16))
  seg = _dev(helpers.document_positions(B, T, 60, seed=83))
  y1, h1, c1 = ops.recurrent_prefill(x, seg, P["conv_w"], P["conv_b"],
                                     P["w_x"], P["b_x"], P["w_a"], P["b_a"],
                                     P["a_param"], gate_branch=gate)
  y2 = torch.empty_like(x)
  h2 = torch.empty(B, W, dtype=torch.float32, device=DEV)
  c2 = x.new_empty(B, 3, W)
  ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
  ptr = lambda t: t.data_ptr()
  _lib.check(lib.rg_recurrent_prefill_gelu_mul(
      ptr(x), ptr(gate), ptr(seg), 1, ptr(P["conv_w"]), ptr(P["conv_b"]),
      ptr(P["w_x"]), ptr(P["b_x"]), ptr(P["w_a"]), ptr(P["b_a"]), None,
      ptr(P["a_param"]), None, ptr(y2), ptr(h2), ptr(c2), ptr(ws), need, B, T,
      W, H, 1, torch.cuda.current_stream().cuda_stream))
  assert torch.equal(y1, y2) and torch.equal(h1, h2) and torch.equal(c1, c2)
  # and against the plain kernel followed by the join as its own pass
  y3, _, _ = ops.recurrent_prefill(x, seg, P["conv_w"], P["conv_b"], P["w_x"],
                                   P["b_x"], P["w_a"], P["b_a"], P["a_param"])
  assert torch.equal(y1, ops.gelu_mul(y3, gate))


def test_recurrent_core_picks_single_launch():
  """With enough (row, head) pairs recurrent_core runs prefill as one launch
  and decode as one launch; both against the oracle, chained."""
  B, T, W, H = 75, 90, 512, 2
  # no workspace = whole rows in the single kernel
  assert _lib.lib().rg_recurrent_core_workspace_bytes(B, T, W, H, 1) == 0
  p, x, blk, (y, cache), (yo, co) = _core_case(
      torch.bfloat16, B, T, W, H, helpers.document_positions(B, T, 30, seed=5),
      seed=77)
  assert helpers.max_rel(y, yo) < BF16_TOL
  assert helpers.max_rel(cache.rg_lru_state, co.rg_lru_state) < BF16_TOL
  assert torch.equal(cache.conv1d_state.cpu(), co.conv1d_state)
  g = torch.Generator().manual_seed(78)
  x1 = torch.randn(B, 1, W, generator=g).to(torch.bfloat16)
  pos = torch.full((B, 1), T, dtype=torch.int64)
  y1, cache1 = rg.recurrent_core(blk.conv_1d, blk.rg_lru, _dev(x1), _dev(pos),
                                 cache)
  yo1, co1 = R.widened_recurrent_core(x1, pos, p, co)
  assert helpers.max_rel(y1, yo1) < BF16_TOL
  assert helpers.max_rel(cache1.rg_lru_state, co1.rg_lru_state) < BF16_TOL
  assert torch.equal(cache1.conv1d_state.cpu(), co1.conv1d_state)


@pytest.mark.parametrize("dtype,B,T,W,H", [
    (torch.float32, 1, 512, 2560, 10),    # float32: gate GEMM + scan in chunks
    (torch.float32, 3, 70, 384, 3),       # 128-wide heads, generic GEMM
    (torch.bfloat16, 2, 300, 512, 2),     # few pairs, short rows: single
                                          # kernel, whole rows, join apart
    (torch.bfloat16, 70, 130, 512, 2),    # 140 pairs: single kernel, whole
                                          # rows, join inside
    (torch.bfloat16, 1, 2048, 512, 2),    # long rows of few pairs: chunks
    (torch.bfloat16, 2, 600, 512, 2),     # ... from 512 tokens on
    (torch.bfloat16, 2, 65, 384, 3),      # bf16, 128-wide heads
    (torch.bfloat16, 300, 5, 512, 2),     # 600 pairs of 5 tokens: two kernels
    (torch.bfloat16, 140, 5, 512, 2),     # 280 pairs of 5: single kernel
    (torch.bfloat16, 140, 64, 512, 2),    # ... of 64: single kernel
])
@pytest.mark.parametrize("joined", [False, True])
def test_recurrent_core_entry_equals_its_parts(dtype, B, T, W, H, joined):
  """rg_recurrent_core picks the kernels itself; whatever it picks, its
  outputs are those of the separate calls it stands for, bit for bit."""
  p = R.make_params(W, H, dtype, seed=301, gate_bias_std=0.3)
  P = {k: _dev(v) for k, v in p.items()}
  g = torch.Generator().manual_seed(302)
  x = _dev(torch.randn(B, T, W, generator=g).to(dtype))
  gate = _dev(torch.randn(B, T, W, generator=g).to(dtype)) if joined else None
  h0 = _dev(torch.randn(B, W, generator=g))
  seg = _dev(helpers.document_positions(B, T, max(T // 3, 2), seed=303))
  code = 0 if dtype == torch.float32 else 1
  need = _lib.lib().rg_recurrent_core_workspace_bytes(B, T, W, H, code)
  y, h, c = ops.recurrent_core(x, seg, P["conv_w"], P["conv_b"], P["w_x"],
                               P["b_x"], P["w_a"], P["b_a"], P["a_param"],
                               h0=h0, gate_branch=gate)
  many_short = (B * H > 512 and T <= 16) or (B * H > 1024 and T <= 32)
  single = dtype == torch.bfloat16 and W // H == 256 and not many_short
  if single:
    chunked = ops.recurrent_prefill_chunked(B, T, W, H)
    assert (need > 0) == chunked
    assert chunked == (B * H <= 128 and T > 448)
    y2, h2, c2 = ops.recurrent_prefill(
        x, seg, P["conv_w"], P["conv_b"], P["w_x"], P["b_x"], P["w_a"],
        P["b_a"], P["a_param"], h0=h0)
  else:
    small_f32 = dtype == torch.float32 and W // H == 256 and B * H <= 32
    assert need >= 2 * x.numel() * x.element_size() or small_f32
    gx, ga = ops.gates_gemm(x, P["w_x"], P["b_x"], P["w_a"], P["b_a"],
                            conv=(seg, P["conv_w"], P["conv_b"]))
    y2, h2, c2 = ops.lru_scan_fused(x, gx, ga, P["a_param"], seg, h0=h0,
                                    conv=(P["conv_w"], P["conv_b"]),
                                    return_conv_cache=True)
  if joined:
    y2 = ops.gelu_mul(y2, gate)
  if dtype == torch.float32 and W // H == 256 and B * H <= 32:
    # the one-launch float32 kernel sums its products in another order than
    # the gate GEMM: float32 agreement, not bit equality (conv state: exact)
    assert need == 0
    assert helpers.max_rel(y, y2) < 2e-6 and helpers.max_rel(h, h2) < 2e-6
    assert torch.equal(c, c2)
    return
  assert torch.equal(y, y2) and torch.equal(h, h2) and torch.equal(c, c2)
  # and against the oracle
  ref = R.recurrent_core if dtype == torch.float32 else R.widened_recurrent_core
  # (the oracle's core has no h0 argument on a prefill: compare a run without)
  y3, h3, c3 = ops.recurrent_core(x, seg, P["conv_w"], P["conv_b"], P["w_x"],
                                  P["b_x"], P["w_a"], P["b_a"], P["a_param"])
  yo, co = ref(x.cpu(), seg.cpu(), p, None)
  tol = F32_TOL if dtype == torch.float32 else BF16_TOL
  assert helpers.max_rel(y3, yo) < tol
  assert helpers.max_rel(h3, co.rg_lru_state) < tol
  assert torch.equal(c3.cpu(), co.conv1d_state)


@pytest.mark.parametrize("B,T,H,mean_doc,pad,with_h0,joined,with_conv,i32", [
    (1, 1, 1, 0, 0, False, False, True, True),
    (3, 2, 2, 0, 0, True, True, True, False),
    (2, 15, 3, 5, 0, True, False, True, True),
    (1, 16, 10, 0, 0, False, True, False, True),
    (4, 17, 8, 2, 3, True, False, True, False),
    (32, 33, 1, 17, 0, False, True, True, True),
    (1, 63, 4, 0, 20, True, True, True, True),
    (8, 64, 4, 60, 0, False, False, False, False),
    (2, 65, 10, 5, 0, True, True, True, True),
    (1, 255, 2, 300, 0, False, False, True, False),
    (3, 256, 10, 17, 100, True, False, True, True),
    (1, 257, 8, 0, 0, True, True, False, True),
    (2, 511, 3, 60, 0, False, True, True, True),
    (1, 513, 10, 2, 0, True, False, True, False),
    (4, 527, 8, 300, 200, False, False, True, True),
    (1, 1023, 1, 0, 0, True, True, True, True),
    (1, 1025, 10, 300, 0, False, True, True, False),
    (2, 1300, 4, 60, 7, True, False, False, True),
    (1, 3001, 2, 1000, 0, True, True, True, True),
])
def test_float32_one_launch_sweep(B, T, H, mean_doc, pad, with_h0, joined,
                                  with_conv, i32):
  """The float32 chain in one launch (256-wide heads, at most 32 (row, head)
  pairs) against the oracle: one token to several 512-token segments, lengths
  below, at and off the kernel's 16-token tiles and chunks, documents of a few
  tokens, left padding, int32 / int64 positions, with and without a carried-in
  state, the block's join and the conv (without: RGLRU.forward alone).  y and
  the state within 1e-5 of the largest magnitude, conv state exact."""
  W = 256 * H
  assert B * H <= 32
  dtype = torch.float32
  p = R.make_params(W, H, dtype, seed=T + H, gate_bias_std=0.3)
  P = {k: _dev(v) for k, v in p.items()}
  g = torch.Generator().manual_seed(1000 + T + B)
  x = torch.randn(B, T, W, generator=g)
  gate = torch.randn(B, T, W, generator=g) if joined else None
  seg = (helpers.document_positions(B, T, mean_doc, seed=T + 2) if mean_doc
         else torch.arange(T).repeat(B, 1))
  if pad:
    seg = torch.cat([torch.full((B, pad), -1), seg[:, :T - pad]], 1)
  seg = seg.to(torch.int32 if i32 else torch.int64)
  h0 = torch.randn(B, W, generator=g) if with_h0 else None
  lib = _lib.lib()
  assert lib.rg_recurrent_core_workspace_bytes(B, T, W, H, 0) == 0
  _announce("float32 one launch", (B, T, H, mean_doc, pad, with_h0, joined,
                                   with_conv, i32))
  cw, cb = (P["conv_w"], P["conv_b"]) if with_conv else (None, None)
  y, h, c = ops.recurrent_core(
      _dev(x), _dev(seg), cw, cb, P["w_x"], P["b_x"], P["w_a"], P["b_a"],
      P["a_param"], h0=None if h0 is None else _dev(h0),
      gate_branch=None if gate is None else _dev(gate))
  if with_conv:
    xc, conv_state = R.conv1d_forward(x, seg, p["conv_w"], p["conv_b"])
    assert torch.equal(c.cpu(), conv_state)
  else:
    xc = x
    assert c is None
  yo, ho = R.rglru_forward(xc, seg, p["a_param"], p["w_x"], p["b_x"], p["w_a"],
                           p["b_a"], cache=h0)
  if joined:
    yo = yo * torch.nn.functional.gelu(gate, approximate="tanh")
  assert torch.isfinite(y).all()
  assert helpers.max_rel(y, yo) < F32_TOL
  assert helpers.max_rel(h, ho) < F32_TOL


def test_recurrent_core_entry_rejects_a_short_workspace():
  B, T, W, H = 1, 512, 512, 4  # float32, 128-wide heads: the two-kernel form
  x = _dev(torch.zeros(B, T, W))
  seg = _dev(torch.arange(T).expand(B, T).contiguous())
  p = {k: _dev(v) for k, v in R.make_params(W, H, torch.float32, seed=1).items()}
  y = torch.empty_like(x)
  need = _lib.lib().rg_recurrent_core_workspace_bytes(B, T, W, H, 0)
  assert need > 0
  ws = torch.empty(need - 16, dtype=torch.uint8, device=DEV)
  ptr = lambda t: t.data_ptr()
  rc = _lib.lib().rg_recurrent_core(
      ptr(x), None, ptr(seg), 1, ptr(p["conv_w"]), ptr(p["conv_b"]),
      ptr(p["w_x"]), ptr(p["b_x"]), ptr(p["w_a"]), ptr(p["b_a"]), None,
      ptr(p["a_param"]), None, ptr(y), None, None, ptr(ws), need - 16, B, T, W,
      H, 0, torch.cuda.current_stream().cuda_stream)
  assert rc == -4
  assert b"workspace" in _lib.lib().rg_last_error()


@pytest.mark.parametrize("B,W,H", [(1, 256, 1), (33, 512, 2), (70, 768, 3),
                                   (256, 1024, 4)])
def test_recurrent_step_joined_with_gate_branch(B, W, H):
  """rg_recurrent_step_gelu_mul: the decode step with the block's join in its
  output stage gives, bit for bit, the step followed by rg_gelu_mul -- new
  tensors and in place, ragged row tiles, document starts among the rows, and
  with the output written over the gate branch."""
  p = R.make_params(W, H, torch.bfloat16, seed=B + 7, gate_bias_std=0.4)
  P = {k: _dev(v) for k, v in p.items()}
  g = torch.Generator().manual_seed(B)
  x = _dev(torch.randn(B, 1, W, generator=g).to(torch.bfloat16))
  gate = _dev(torch.randn(B, 1, W, generator=g).to(torch.bfloat16))
  h = _dev(torch.randn(B, W, generator=g))
  cc = _dev(torch.randn(B, 3, W, generator=g).to(torch.bfloat16))
  seg = torch.full((B, 1), 9, dtype=torch.int64)
  seg[B // 2, 0] = 0
  seg = _dev(seg)
  args = (P["conv_w"], P["conv_b"], P["w_x"], P["b_x"], P["w_a"], P["b_a"],
          P["a_param"])
  y0, h0, c0 = ops.recurrent_step(x, seg, cc, h, *args)
  want = ops.gelu_mul(y0, gate)
  y1, h1, c1 = ops.recurrent_step(x, seg, cc, h, *args, gate_branch=gate)
  assert torch.equal(y1, want) and torch.equal(h1, h0) and torch.equal(c1, c0)
  h2, c2 = h.clone(), cc.clone()
  y2, h2b, c2b = ops.recurrent_step(x, seg, c2, h2, *args, in_place=True,
                                    gate_branch=gate)
  assert h2b.data_ptr() == h2.data_ptr() and c2b.data_ptr() == c2.data_ptr()
  assert torch.equal(y2, want) and torch.equal(h2, h0) and torch.equal(c2, c0)
  # through the C ABI, the output over the gate branch
  packed = ops.packed_gate_weights(P["w_x"], P["w_a"])
  over = gate.clone()
  h3, c3 = torch.empty_like(h), torch.empty_like(cc)
  ptr = lambda t: t.data_ptr()
  _lib.check(_lib.lib().rg_recurrent_step_gelu_mul(
      ptr(x), ptr(over), ptr(seg), 1, ptr(cc), ptr(c3), ptr(h), ptr(h3),
      ptr(P["conv_w"]), ptr(P["conv_b"]), ptr(packed), ptr(P["b_x"]),
      ptr(P["b_a"]), ptr(P["a_param"]), ptr(over), B, W, H, 1,
      torch.cuda.current_stream().cuda_stream))
  assert torch.equal(over, want) and torch.equal(h3, h0) and torch.equal(c3, c0)
  # float32 has no joined kernel: the wrapper adds the pass itself
  pf = {k: _dev(v) for k, v in
        R.make_params(W, H, torch.float32, seed=3).items()}
  argsf = (pf["conv_w"], pf["conv_b"], pf["w_x"], pf["b_x"], pf["w_a"],
           pf["b_a"], pf["a_param"])
  yf, _, _ = ops.recurrent_step(x.float(), seg, cc.float(), h, *argsf)
  yj, _, _ = ops.recurrent_step(x.float(), seg, cc.float(), h, *argsf,
                                gate_branch=gate.float())
  assert torch.equal(yj, ops.gelu_mul(yf, gate.float()))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_recurrent_block_traces_as_one_graph(dtype):
  """torch.compile follows RecurrentBlock without a graph break (fullgraph):
  the conv -> RG-LRU core is one custom operator node each for a prefill and
  for a decode step (recurrentgemma_amd/compiled.py).  Backend aot_eager: the
  traced, functionalised graph is run by torch's own kernels plus ours, and
  must give what the eager module gives, bit for bit."""
  B, T, width, H = 3, 40, 512, 2
  torch.manual_seed(12)
  blk = rg.RecurrentBlock(width=width, num_heads=H, dtype=dtype).to(DEV)
  x = _dev(torch.randn(B, T, width).to(dtype))
  seg = _dev(helpers.document_positions(B, T, 15, seed=8))
  want, cache = blk(x, seg)
  traced = torch.compile(blk, backend="aot_eager", fullgraph=True)
  got, cache_t = traced(x, seg)
  assert torch.equal(got, want)
  assert torch.equal(cache_t.rg_lru_state, cache.rg_lru_state)
  assert torch.equal(cache_t.conv1d_state, cache.conv1d_state)
  x1 = _dev(torch.randn(B, 1, width).to(dtype))
  pos = _dev(torch.full((B, 1), T, dtype=torch.int64))
  want1, cache1 = blk(x1, pos, cache)
  got1, cache1_t = traced(x1, pos, cache)
  assert torch.equal(got1, want1)
  assert torch.equal(cache1_t.rg_lru_state, cache1.rg_lru_state)
  assert torch.equal(cache1_t.conv1d_state, cache1.conv1d_state)


def test_decode_step_under_graph_capture():
  """The decode step allocates nothing, never synchronises and only uses the
  stream it is given, so a HIP graph can hold it: capture one in-place step,
  replay it several times with eager work and synchronisation in between, and
  compare every replay with the same step run eagerly."""
  B, W, H = 48, 512, 2
  p = R.make_params(W, H, torch.bfloat16, seed=91, gate_bias_std=0.5)
  P = {k: _dev(v) for k, v in p.items()}
  g = torch.Generator().manual_seed(92)
  x = _dev(torch.randn(B, 1, W, generator=g).to(torch.bfloat16))
  seg = _dev(torch.full((B, 1), 17, dtype=torch.int64))
  h_g = _dev(torch.randn(B, W, generator=g))
  cc_g = _dev(torch.randn(B, 3, W, generator=g).to(torch.bfloat16))
  h_e, cc_e = h_g.clone(), cc_g.clone()
  ops.packed_gate_weights(P["w_x"], P["w_a"])  # packed outside the capture

  def step(h, cc):
    return ops.recurrent_step(x, seg, cc, h, P["conv_w"], P["conv_b"],
                              P["w_x"], P["b_x"], P["w_a"], P["b_a"],
                              P["a_param"], in_place=True)

  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    step(h_g.clone(), cc_g.clone())  # warm-up off the capture
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    y_g, _, _ = step(h_g, cc_g)
  for i in range(4):
    x.copy_(torch.randn(B, 1, W, generator=g).to(torch.bfloat16))  # eager work
    torch.cuda.synchronize()
    graph.replay()
    y_e, h_e, cc_e = step(h_e, cc_e)
    torch.cuda.synchronize()
    assert torch.equal(y_g, y_e), i
    assert torch.equal(h_g, h_e) and torch.equal(cc_g, cc_e), i


def test_recurrent_prefill_unsupported_shapes():
  """fp32 and heads that are not 256 wide are refused with RG_ERR_UNSUPPORTED
  (callers use the two-kernel form), nothing is launched."""
  for dtype, W, H in ((torch.float32, 256, 1), (torch.bfloat16, 256, 2)):
    p = {k: _dev(v) for k, v in R.make_params(W, H, dtype, seed=3).items()}
    x = _dev(torch.zeros(1, 8, W, dtype=dtype))
    seg = _dev(torch.arange(8).expand(1, 8).contiguous())
    assert not ops.recurrent_prefill_supported(x, H)
    with pytest.raises(_lib.KernelError) as e:
      ops.recurrent_prefill(x, seg, p["conv_w"], p["conv_b"], p["w_x"],
                            p["b_x"], p["w_a"], p["b_a"], p["a_param"])
    assert "unsupported" in str(e.value)


# ------------------------------------------- the x * gelu(y) join, 1 pass --


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [1, 7, 8, 2055, 3 * 100 * 256, 8 * 1024 * 1024 + 3])
def test_gelu_mul(dtype, n):
  """rg_gelu_mul against torch's own two passes (gelu(approximate="tanh")
  evaluated in float32 on the CPU, rounded to the activation dtype as the
  reference's tensor `y` is, then the product): fp32 within 1e-5 of the
  largest magnitude; bf16 within one bf16 ulp of each element (the fast
  sigmoid may land a gelu value on the neighbouring bf16) plus 1e-6 |a|: in
  the negative tail 1 + tanh(u) is a multiple of 2^-24, and two float32 tanh
  that differ in the last place differ there by 0.5 |g| 2^-24 in gelu."""
  _announce("gelu_mul", dtype, n)
  gen = torch.Generator().manual_seed(n)
  a = torch.randn(n, generator=gen).to(dtype)
  g = (3.0 * torch.randn(n, generator=gen)).to(dtype)
  if n >= 7:
    g[:7] = torch.tensor([0.0, -0.0, 20.0, -20.0, 1e-3, -9.0, 9.0]).to(dtype)
  y = torch.nn.functional.gelu(g.float(), approximate="tanh").to(dtype)
  want = (a.float() * y.float()).to(dtype)
  got = ops.gelu_mul(_dev(a), _dev(g)).cpu()
  assert got.dtype == dtype and got.shape == a.shape
  assert torch.isfinite(got.float()).all()
  if dtype == torch.float32:
    assert helpers.max_rel(got, want) < 1e-5
  else:
    err = (got.float() - want.float()).abs()
    ulp = want.float().abs() * 2.0 ** -7 + 1e-6 * a.float().abs()
    assert (err <= ulp).all(), float((err / ulp).max())
    assert (err > 0).float().mean() < 0.02  # neighbouring-bf16 cases are rare
  # in place on either operand
  a_d, g_d = _dev(a), _dev(g)
  code = 0 if dtype == torch.float32 else 1
  a_io, g_io = a_d.clone(), g_d.clone()
  for src_a, src_g, dst in ((a_io, g_d, a_io), (a_d, g_io, g_io)):
    _lib.check(_lib.lib().rg_gelu_mul(src_a.data_ptr(), src_g.data_ptr(),
                                      dst.data_ptr(), n, code,
                                      torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(dst.cpu(), got)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(1, 1), (3, 7), (5, 256), (64, 2560),
                                        (2 * 33, 4096), (2, 10007)])
def test_rms_norm(dtype, rows, width):
  """rg_rms_norm against the reference's chain of tensor ops (layers.py:65-73)
  evaluated by torch in the same dtype: fp32 on the CPU, 1e-5 of the largest
  magnitude; bf16 by torch's own GPU kernels (torch's CPU rsqrt rounds the
  square root to bf16 before taking the reciprocal, its GPU kernel and this
  one round once), one bf16 ulp per element: the sum of squares is taken in a
  different order, which can move the rounded mean or rsqrt by one ulp, and
  that moves every element of the row."""
  _announce("rms_norm", dtype, rows, width)
  gen = torch.Generator().manual_seed(rows * 131 + width)
  x = (2.0 * torch.randn(rows, width, generator=gen)).to(dtype)
  scale = (0.3 * torch.randn(width, generator=gen)).to(dtype)
  eps = 1e-6

  def chain(x, scale):
    var = torch.mean(torch.square(x), dim=-1, keepdim=True)
    return x * torch.rsqrt(var + eps) * (scale + 1)

  got = ops.rms_norm(_dev(x), _dev(scale), eps).cpu()
  assert got.dtype == dtype and got.shape == x.shape
  if dtype == torch.float32:
    assert helpers.max_rel(got, chain(x, scale)) < 1e-5
  else:
    want = chain(_dev(x), _dev(scale)).cpu()
    err = (got.float() - want.float()).abs()
    assert (err <= want.float().abs() * 2.0 ** -7 + 1e-30).all()
    assert (err > 0).float().mean() < 0.35
  x3 = x.reshape(1, rows, width)  # leading dimensions are rows
  assert torch.equal(ops.rms_norm(_dev(x3), _dev(scale), eps).cpu()[0], got)
  # the residual sum fused in front: identical to add, then norm
  other = torch.randn(rows, width, generator=gen).to(dtype)
  total, normed = ops.add_rms_norm(_dev(x), _dev(other), _dev(scale), eps)
  want_total = _dev(x) + _dev(other)
  assert torch.equal(total, want_total)
  assert torch.equal(normed, ops.rms_norm(want_total, _dev(scale), eps))


# --------------------------------- full-size, size-independent properties --


def _full_size_properties(B, T, W, H, seg, seed):
  dtype = torch.bfloat16
  p = R.make_params(W, H, dtype, seed=seed)
  p["conv_b"].zero_()  # so that the conv is exactly linear
  g = torch.Generator().manual_seed(seed - 100)
  x = torch.randn(B, T, W, generator=g).to(dtype).to(DEV)
  blk = _block(p, W, H, dtype)
  segd = seg.to(DEV)
  y, cache = rg.recurrent_core(blk.conv_1d, blk.rg_lru, x, segd)
  torch.cuda.synchronize()
  assert torch.isfinite(y.float()).all()
  # (0) recurrent_core may take the single-launch kernel (one workgroup per
  #     row and head) or the two-kernel form; the two differ only in the fp32
  #     association of the recurrence: rare 1-ulp bf16 flips in y
  gx, ga = ops.gates_gemm(x, blk.rg_lru.input_gate.w, blk.rg_lru.input_gate.b,
                          blk.rg_lru.a_gate.w, blk.rg_lru.a_gate.b,
                          conv=(segd, blk.conv_1d.w, blk.conv_1d.b))
  y1, h1, c1 = ops.lru_scan_fused(x, gx, ga, blk.rg_lru.a_param, segd,
                                  conv=(blk.conv_1d.w, blk.conv_1d.b),
                                  return_conv_cache=True)
  # (the single-launch kernel keeps the pre-activations in float32, the
  # two-kernel form rounds them to bf16: a bf16 ulp or two apart)
  assert (y1 != y).float().mean().item() < 0.15
  assert (y1.float() - y.float()).abs().max().item() <= 0.125
  assert helpers.max_rel(y1, y) < BF16_TOL
  assert helpers.max_rel(cache.rg_lru_state, h1) < BF16_TOL
  assert torch.equal(c1, cache.conv1d_state)
  if ops.recurrent_prefill_supported(x, H):
    yf, hf, cf = ops.recurrent_prefill(
        x, segd, blk.conv_1d.w, blk.conv_1d.b, blk.rg_lru.input_gate.w,
        blk.rg_lru.input_gate.b, blk.rg_lru.a_gate.w, blk.rg_lru.a_gate.b,
        blk.rg_lru.a_param)
    assert (y1 != yf).float().mean().item() < 0.15
    assert (y1.float() - yf.float()).abs().max().item() <= 0.125
    assert helpers.max_rel(yf, y1) < BF16_TOL
    assert helpers.max_rel(hf, h1) < BF16_TOL
    assert torch.equal(cf, c1)
  y_core, y = y, y1  # the exact statements below are about the two-kernel form
  cache_core, cache = cache, rg.RecurrentBlockCache(rg_lru_state=h1,
                                                    conv1d_state=c1)
  # (1) module-by-module: the stand-alone conv followed by the RG-LRU on its
  #     own (the same choice of kernels as the fused call, without conv
  #     weights; the single kernel sums its conv taps in another order than
  #     the stand-alone conv: a rare bf16 ulp in the conv output) ...
  xc, cstate = blk.conv_1d(x, segd)
  y2, h2 = blk.rg_lru(xc, segd)
  assert (y2 != y_core).float().mean().item() < 0.15
  assert (y2.float() - y_core.float()).abs().max().item() <= 0.125
  assert helpers.max_rel(y2, y_core) < BF16_TOL
  assert helpers.max_rel(h2, cache_core.rg_lru_state) < BF16_TOL
  assert torch.equal(cstate, cache.conv1d_state)
  #     ... and, bit for bit, the two-kernel form with and without the conv
  #     on load
  gx2, ga2 = ops.gates_gemm(xc, blk.rg_lru.input_gate.w,
                            blk.rg_lru.input_gate.b, blk.rg_lru.a_gate.w,
                            blk.rg_lru.a_gate.b)
  assert torch.equal(gx2, gx) and torch.equal(ga2, ga)
  y3, h3, _ = ops.lru_scan_fused(xc, gx2, ga2, blk.rg_lru.a_param, segd)
  assert torch.equal(y3, y) and torch.equal(h3, cache.rg_lru_state)
  # (2) splitting the sequence and carrying the state changes nothing beyond
  #     fp32 re-association of the carry (rows cut into other chunks included)
  cut = T // 2 + 5
  ya, ha = blk.rg_lru(xc[:, :cut].contiguous(), segd[:, :cut].contiguous())
  yb, hb = blk.rg_lru(xc[:, cut:].contiguous(), segd[:, cut:].contiguous(), ha)
  assert helpers.max_rel(hb, h2) < 1e-5
  for part, whole in ((ya, y2[:, :cut]), (yb, y2[:, cut:])):
    assert (part.float() - whole.float()).abs().max().item() <= 0.0625
    mism = (part != whole).float().mean().item()
    assert mism < 1e-3, mism
  # (3) with the gate pre-activations held fixed the path is linear in x:
  #     doubling x doubles y and h exactly (powers of two are exact)
  yd, hd, _ = ops.lru_scan_fused(x * 2, gx, ga, blk.rg_lru.a_param, segd,
                                 conv=(blk.conv_1d.w, blk.conv_1d.b))
  assert torch.equal(yd.float(), y1.float() * 2) and torch.equal(hd, h1 * 2)
  # (4) at every document start y == conv(x) * sigmoid(gx_pre)
  starts = segd == 0
  want = (xc.float() * torch.sigmoid(gx.float()))[starts]
  got = y[starts].float()
  assert ((got - want).abs() <= 0.01 * want.abs() + 1e-3).all()
  # (5) a row's result does not depend on its neighbours (first row alone)
  y_row, c_row = rg.recurrent_core(blk.conv_1d, blk.rg_lru, x[:1].contiguous(),
                                   segd[:1].contiguous())
  # (a one-row launch may use another lane width / step length, i.e. another
  # fp32 association of the carry: equal up to rare 1-ulp bf16 flips)
  assert (y_row != y[:1]).float().mean().item() < 0.15
  assert (y_row.float() - y[:1].float()).abs().max().item() <= 0.125
  assert helpers.max_rel(c_row.rg_lru_state, cache.rg_lru_state[:1]) < BF16_TOL
  assert torch.equal(c_row.conv1d_state, cache.conv1d_state[:1])
  # (7) the block's join inside the call (the single kernels carry it in
  #     their output stage, whole rows and rows in chunks) == the separate
  #     pass over the call's plain output, bit for bit; states unchanged
  gate = torch.randn(B, T, W, generator=g).to(dtype).to(DEV)
  y_join, cache_join = rg.recurrent_core(blk.conv_1d, blk.rg_lru, x, segd,
                                         gate_branch=gate)
  assert torch.equal(y_join, ops.gelu_mul(y_core, gate))
  assert torch.equal(cache_join.rg_lru_state, cache_core.rg_lru_state)
  assert torch.equal(cache_join.conv1d_state, cache_core.conv1d_state)
  del gate, y_join, cache_join
  # (6) parity against the oracle over the WHOLE sequence on two sampled rows
  #     (not row 0): y element by element, the final state and the conv state,
  #     for what recurrent_core ran at this grid (every chunk boundary of a
  #     chunked launch and the tail of the row included) and for the
  #     two-kernel form
  for row in sorted({B // 2, B - 1}):
    _announce("full size: oracle on row", row)
    yo, co = R.widened_recurrent_core(x[row:row + 1].cpu(), seg[row:row + 1], p)
    for name, yy, hh, cc in (
        ("recurrent_core", y_core, cache_core.rg_lru_state,
         cache_core.conv1d_state),
        ("two kernels", y, cache.rg_lru_state, cache.conv1d_state)):
      helpers.assert_close_elementwise(yy[row:row + 1], yo,
                                       what=f"{name} row {row} y")
      assert helpers.max_rel(yy[row:row + 1], yo) < BF16_TOL
      assert helpers.max_rel(hh[row:row + 1], co.rg_lru_state) < 2e-3, name
      assert torch.equal(cc[row:row + 1].cpu(), co.conv1d_state), name


def test_config2_full_size_properties():
  """Benchmark configuration 2: B8 T4096 W2560 H10 bf16, documents ~ Geometric(1024)."""
  B, T, W, H = 8, 4096, 2560, 10
  seg = helpers.document_positions(B, T, 1024, seed=1002)
  _announce("config2 full size")
  _full_size_properties(B, T, W, H, seg, seed=1102)


def test_config3_full_size_properties():
  """Benchmark configuration 3: B16 T8192 W4096 H16 bf16, one document per row."""
  B, T, W, H = 16, 8192, 4096, 16
  seg = torch.arange(T).expand(B, T).contiguous()
  _announce("config3 full size")
  _full_size_properties(B, T, W, H, seg, seed=1103)


# ------------------------------------------------- config 4 at full size --


def test_config4_full_size_decode():
  """Benchmark configuration 4 at its full shape: B256 W4096 H16 bf16, a
  2048-token prefill through recurrent_core, then 64 chained single-token
  steps.  Every step: single launch == three-launch form bit for bit (8 row
  tiles x 16 heads, the grid of this shape); at the end: the state and the
  last y equal those of one prefill over all 2112 tokens up to the fp32
  association of the recurrence; a few rows against the oracle end to end."""
  B, T, W, H, steps = 256, 2048, 4096, 16, 64
  dtype = torch.bfloat16
  p = R.make_params(W, H, dtype, seed=1104 + 100)
  P = {k: _dev(v) for k, v in p.items()}
  blk = _block(p, W, H, dtype)
  g = torch.Generator().manual_seed(1104)
  x = torch.randn(B, T + steps, W, generator=g).to(dtype)
  xd = _dev(x)
  seg = torch.arange(T + steps).expand(B, -1).contiguous()
  segd = _dev(seg)
  _announce("config4 full size: prefill")
  y, cache = rg.recurrent_core(blk.conv_1d, blk.rg_lru,
                               xd[:, :T].contiguous(),
                               segd[:, :T].contiguous())
  lib = _lib.lib()
  ws = torch.empty(lib.rg_recurrent_step_workspace_bytes(B, W, 1),
                   dtype=torch.uint8, device=DEV)
  ptr = lambda t: t.data_ptr()
  h3, cc3 = cache.rg_lru_state.clone(), cache.conv1d_state.clone()
  ys = []
  for i in range(steps):
    if i % 16 == 0:
      _announce("config4 full size: step", i)
    xi = xd[:, T + i:T + i + 1].contiguous()
    pos = segd[:, T + i:T + i + 1].contiguous()
    y1, cache = rg.recurrent_core(blk.conv_1d, blk.rg_lru, xi, pos, cache)
    y3 = torch.empty_like(xi)
    h3n, cc3n = torch.empty_like(h3), torch.empty_like(cc3)
    _lib.check(lib.rg_recurrent_step(
        ptr(xi), ptr(pos), 1, ptr(cc3), ptr(cc3n), ptr(h3), ptr(h3n),
        ptr(P["conv_w"]), ptr(P["conv_b"]), ptr(P["w_x"]), ptr(P["b_x"]),
        ptr(P["w_a"]), ptr(P["b_a"]), ptr(P["a_param"]), ptr(y3), ptr(ws),
        ws.numel(), B, W, H, 1, torch.cuda.current_stream().cuda_stream))
    h3, cc3 = h3n, cc3n
    assert torch.equal(y1, y3), i
    assert torch.equal(cache.rg_lru_state, h3), i
    assert torch.equal(cache.conv1d_state, cc3), i
    ys.append(y1)
  _announce("config4 full size: one prefill over all tokens")
  y_full, c_full = rg.recurrent_core(blk.conv_1d, blk.rg_lru, xd, segd)
  torch.cuda.synchronize()
  # (the decode step rounds the gate pre-activations to bf16 like the
  # reference's modules, the prefill kernel keeps them in float32)
  assert helpers.max_rel(cache.rg_lru_state, c_full.rg_lru_state) < 2e-3
  assert torch.equal(cache.conv1d_state, c_full.conv1d_state)
  y_steps = torch.cat(ys, dim=1)
  d = (y_steps.float() - y_full[:, T:].float()).abs()
  assert d.max().item() <= 0.125
  assert helpers.max_rel(y_steps, y_full[:, T:]) < BF16_TOL
  assert (y_steps != y_full[:, T:]).float().mean().item() < 0.15
  # oracle, end to end, on three rows (prefill + 64 steps)
  rows = [0, 131, 255]
  xo, sego = x[rows], seg[rows]
  yo, co = R.widened_recurrent_core(xo[:, :T], sego[:, :T], p)
  assert helpers.max_rel(y[rows], yo) < BF16_TOL
  for i in range(steps):
    yo, co = R.widened_recurrent_core(xo[:, T + i:T + i + 1],
                                      sego[:, T + i:T + i + 1], p, co)
    assert helpers.max_rel(ys[i][rows], yo) < BF16_TOL, i
  assert helpers.max_rel(cache.rg_lru_state[rows], co.rg_lru_state) < BF16_TOL
  assert torch.equal(cache.conv1d_state[rows].cpu(), co.conv1d_state)


# ------------------------------------ repeated launches are bit-identical --


@pytest.mark.parametrize("B,T,W,H,mean_doc", [
    (40, 512, 1024, 4, None),    # 160 workgroups, full tiles
    (9, 1000, 512, 2, 120),      # ragged last tile, document starts
    (300, 70, 256, 1, 20),       # more workgroups than CUs, short rows
])
def test_repeated_launches_are_bit_identical(B, T, W, H, mean_doc):
  """200 launches each of rg_recurrent_prefill and rg_gates_gemm on the same
  inputs give the same bits every time.  Regression test for 16-byte buffer
  stores whose data registers were overwritten by the next vector instruction
  before the store had read them (0-64 wrong elements per launch, not
  deterministic): every such store goes through buffer_store_16() now."""
  _announce("repeat launches", B, T, W, H, mean_doc)
  seed = 9100 + B
  p = R.make_params(W, H, torch.bfloat16, seed=seed, gate_bias_std=0.5)
  P = {k: _dev(v) for k, v in p.items()}
  g = torch.Generator().manual_seed(seed + 1)
  x = _dev(torch.randn(B, T, W, generator=g).to(torch.bfloat16))
  seg = (torch.arange(T).expand(B, T).contiguous() if mean_doc is None
         else helpers.document_positions(B, T, mean_doc, seed=seed))
  seg = _dev(seg)

  def prefill():
    return ops.recurrent_prefill(x, seg, P["conv_w"], P["conv_b"], P["w_x"],
                                 P["b_x"], P["w_a"], P["b_a"], P["a_param"])

  def gemm():
    return ops.gates_gemm(x, P["w_x"], P["b_x"], P["w_a"], P["b_a"],
                          conv=(seg, P["conv_w"], P["conv_b"]))

  for fn in (prefill, gemm):
    first = fn()
    bad = torch.zeros((), dtype=torch.int64, device=DEV)
    for _ in range(200):
      out = fn()
      for a, b in zip(out, first):
        bad += (a != b).sum()
    torch.cuda.synchronize()
    assert bad.item() == 0, (fn.__name__, bad.item())


# ------------------------------------------- scratch of the decode step --


def test_step_scratch_survives_other_shapes_under_graph():
  """The three-launch decode step (fp32, or heads that are not 256 wide)
  exchanges its intermediates through scratch memory.  A captured step keeps
  that memory's address: an eager step of another shape in between must not
  take it away.  Capture at one shape, run eager steps of other shapes, replay,
  and compare every replay with the same step run eagerly, bit for bit."""
  W, H = 256, 2
  dtype = torch.float32
  p = R.make_params(W, H, dtype, seed=123, gate_bias_std=0.5)
  P = {k: _dev(v) for k, v in p.items()}
  g = torch.Generator().manual_seed(124)

  def make(B, Wd):
    return (_dev(torch.randn(B, 1, Wd, generator=g)),
            _dev(torch.full((B, 1), 5, dtype=torch.int64)),
            _dev(torch.randn(B, 3, Wd, generator=g)),
            _dev(torch.randn(B, Wd, generator=g)))

  def step(x, seg, cc, h, prm=P, in_place=True):
    return ops.recurrent_step(x, seg, cc, h, prm["conv_w"], prm["conv_b"],
                              prm["w_x"], prm["b_x"], prm["w_a"], prm["b_a"],
                              prm["a_param"], in_place=in_place)

  x, seg, cc_g, h_g = make(3, W)
  cc_e, h_e = cc_g.clone(), h_g.clone()
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    step(x, seg, cc_g.clone(), h_g.clone())  # warm-up off the capture
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    y_g, _, _ = step(x, seg, cc_g, h_g)
  W2, H2 = 512, 4
  P2 = {k: _dev(v) for k, v in
        R.make_params(W2, H2, dtype, seed=125, gate_bias_std=0.5).items()}
  for i in range(3):
    # eager steps of other shapes: their scratch must be other memory
    junk = [step(*make(7 + i, W2), prm=P2, in_place=False) for _ in range(2)]
    x.copy_(torch.randn(3, 1, W, generator=g))
    torch.cuda.synchronize()
    graph.replay()
    y_e, h_e, cc_e = step(x, seg, cc_e, h_e)
    torch.cuda.synchronize()
    assert torch.equal(y_g, y_e), i
    assert torch.equal(h_g, h_e) and torch.equal(cc_g, cc_e), i
    del junk


def test_in_place_step_refuses_tensors_it_would_have_to_copy():
  """An in-place decode step on a misaligned or non-contiguous cache tensor
  would update a private copy: it raises instead."""
  B, W, H = 4, 256, 1
  p = {k: _dev(v) for k, v in
       R.make_params(W, H, torch.bfloat16, seed=3).items()}
  x = _dev(torch.zeros(B, 1, W, dtype=torch.bfloat16))
  seg = _dev(torch.full((B, 1), 3, dtype=torch.int64))
  cc = _dev(torch.zeros(B, 3, W, dtype=torch.bfloat16))
  h_odd = _dev(torch.zeros(B * W + 1))[1:].view(B, W)  # 4-byte aligned only
  args = (p["conv_w"], p["conv_b"], p["w_x"], p["b_x"], p["w_a"], p["b_a"],
          p["a_param"])
  with pytest.raises(ValueError):
    ops.recurrent_step(x, seg, cc, h_odd, *args, in_place=True)
  cc_t = _dev(torch.zeros(3, B, W, dtype=torch.bfloat16)).transpose(0, 1)
  h = _dev(torch.zeros(B, W))
  with pytest.raises(ValueError):
    ops.recurrent_step(x, seg, cc_t, h, *args, in_place=True)
  with pytest.raises(ValueError):  # a conv state that needs a dtype cast
    ops.recurrent_step(x, seg, cc.float(), h, *args, in_place=True)
  y, h2, cc2 = ops.recurrent_step(x, seg, cc, h, *args, in_place=True)
  assert h2.data_ptr() == h.data_ptr() and cc2.data_ptr() == cc.data_ptr()
