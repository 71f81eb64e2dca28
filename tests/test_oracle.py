"""Pins the CPU oracle (oracle/torch_ref.py, oracle/rglru_ref.c).

Nothing here re-types the oracle's formulas: every check is a golden vector
written from the reference, a library routine that coincides with a special
case, a brute-force loop straight from the definition, a closed form, or an
invariant.  A dropped tap, a wrong mask index, a transposed gate weight or a
wrong sign in the recurrence fails at least one of them.
"""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import c_ref
from oracle import torch_ref as R
from tests import helpers


def _tol(dtype):
  # fp32: a few ulp (different CPU vector paths); bf16: 2 ulp.
  if dtype == torch.bfloat16:
    return dict(rtol=1.6e-2, atol=1e-2)
  return dict(rtol=3e-6, atol=2e-6)


def _close(got, want, frac_equal=0.97):
  torch.testing.assert_close(got, want, **_tol(want.dtype))
  same = (got == want).float().mean().item()
  assert same >= frac_equal, f"only {same:.3f} of elements identical"


# ---------------------------------------------------------------- golden ---


def test_golden_conv1d(golden):
  keys = golden.cases("conv/")
  assert len(keys) == 80
  for key in keys:
    x, seg = golden.get(key + "/x"), golden.get(key + "/seg")
    w, b = golden.get(key + "/w"), golden.get(key + "/b")
    xin = x.clone()
    y, cache = R.conv1d_forward(xin, seg, w, b, mutate_input=True)
    _close(y, golden.get(key + "/y"))
    assert torch.equal(cache, golden.get(key + "/cache")), key
    assert torch.equal(xin, golden.get(key + "/x_after")), key
    # default call leaves the input alone but returns the same (masked) cache
    x2 = x.clone()
    y2, cache2 = R.conv1d_forward(x2, seg, w, b)
    assert torch.equal(x2, x) and torch.equal(y2, y)
    assert torch.equal(cache2, cache)
    y3, none = R.conv1d_forward(x.clone(), seg, w, b, return_cache=False)
    assert none is None and torch.equal(y3, y)
    xs = golden.get(key + "/step_x")
    for i in range(2):
      ys, cache = R.conv1d_forward(xs[:, i:i + 1], seg[:, -1:] + 1 + i, w, b,
                                   cache)
      _close(ys, golden.get(key + f"/step{i}_y"))
      assert torch.equal(cache, golden.get(key + f"/step{i}_cache")), key


def _rglru_params(golden, key):
  pkey = "/".join(key.split("/")[:3])
  return [golden.get(pkey + "/" + n)
          for n in ("a_param", "w_x", "b_x", "w_a", "b_a")]


def test_golden_rglru(golden):
  keys = golden.cases("rglru/")
  assert len(keys) == 72
  for key in keys:
    prm = _rglru_params(golden, key)
    x, seg = golden.get(key + "/x"), golden.get(key + "/seg")
    h0 = golden.get(key + "/h0") if golden.has(key + "/h0") else None
    y, h = R.rglru_forward(x, seg, *prm, cache=h0)
    assert h.dtype == torch.float32
    _close(y, golden.get(key + "/y"))
    torch.testing.assert_close(h, golden.get(key + "/h"), rtol=1e-5, atol=1e-5)
    xs = golden.get(key + "/step_x")
    for i in range(2):
      ys, h = R.rglru_forward(xs[:, i:i + 1], seg[:, -1:] + 1 + i, *prm,
                              cache=h)
      _close(ys, golden.get(key + f"/step{i}_y"))
      torch.testing.assert_close(h, golden.get(key + f"/step{i}_h"),
                                 rtol=1e-5, atol=1e-5)


def test_golden_param_init(golden):
  for seed in (0, 1, 2):
    torch.manual_seed(seed)
    t = torch.empty(64)
    R.rnn_param_init(t, 0.9, 0.999)
    torch.testing.assert_close(t, golden.get(f"init/seed{seed}"), rtol=1e-6,
                               atol=1e-6)


# ------------------------------------------------------------------ conv ---


def _conv_brute(x, seg, w, b):
  """out[t] = b + sum_s w[K-1-s] x[t-s] * [no boundary in (t-s, t]]."""
  B, T, W = x.shape
  K = w.shape[0]
  out = torch.zeros(B, T, W, dtype=torch.float64)
  for bi in range(B):
    for t in range(T):
      for s in range(K):
        if t - s < 0:
          continue
        if any(seg[bi, j] == 0 for j in range(t - s + 1, t + 1)):
          continue
        out[bi, t] += w[K - 1 - s].double() * x[bi, t - s].double()
      out[bi, t] += b.double()
  return out


@pytest.mark.parametrize("K", [2, 4, 8])
def test_conv_single_document_is_depthwise_conv(K):
  g = torch.Generator().manual_seed(K)
  B, T, W = 3, 37, 24
  x = torch.randn(B, T, W, generator=g, dtype=torch.float64)
  w = torch.randn(K, W, generator=g, dtype=torch.float64)
  b = torch.randn(W, generator=g, dtype=torch.float64)
  seg = torch.arange(T).expand(B, T)
  y, cache = R.conv1d_forward(x, seg, w, b)
  want = F.conv1d(x.transpose(1, 2), w.t()[:, None, :], b, padding=K - 1,
                  groups=W)[..., :T].transpose(1, 2)
  torch.testing.assert_close(y, want, rtol=1e-12, atol=1e-12)
  if K > 1:
    assert torch.equal(cache, x[:, T - (K - 1):])


@pytest.mark.parametrize("K", [2, 4, 8])
@pytest.mark.parametrize("T", [1, 2, 3, 7, 19])
def test_conv_brute_force_with_boundaries(K, T):
  g = torch.Generator().manual_seed(100 * K + T)
  B, W = 4, 5
  x = torch.randn(B, T, W, generator=g, dtype=torch.float64)
  w = torch.randn(K, W, generator=g, dtype=torch.float64)
  b = torch.randn(W, generator=g, dtype=torch.float64)
  seg = torch.randint(-1, 3, (B, T), generator=g)
  y, _ = R.conv1d_forward(x, seg, w, b)
  torch.testing.assert_close(y, _conv_brute(x, seg, w, b), rtol=1e-12,
                             atol=1e-12)
  yc, cache_c = c_ref.conv1d_prefill(x.numpy(), seg.numpy(), w.numpy(),
                                     b.numpy())
  np.testing.assert_allclose(yc, y.numpy(), rtol=1e-12, atol=1e-12)
  _, cache = R.conv1d_forward(x, seg, w, b)
  np.testing.assert_array_equal(cache_c, cache.numpy())


def test_conv_packed_equals_per_document():
  g = torch.Generator().manual_seed(5)
  W, K = 6, 4
  lens = [1, 5, 2, 9, 3]
  T = sum(lens)
  x = torch.randn(1, T, W, generator=g, dtype=torch.float64)
  w = torch.randn(K, W, generator=g, dtype=torch.float64)
  b = torch.randn(W, generator=g, dtype=torch.float64)
  seg = torch.cat([torch.arange(n) for n in lens])[None]
  y, _ = R.conv1d_forward(x, seg, w, b)
  t = 0
  for n in lens:
    yd, _ = R.conv1d_forward(x[:, t:t + n], torch.arange(n)[None], w, b)
    torch.testing.assert_close(y[:, t:t + n], yd, rtol=1e-12, atol=1e-12)
    t += n


def test_conv_special_weights():
  g = torch.Generator().manual_seed(6)
  x = torch.randn(2, 11, 3, generator=g)
  seg = torch.arange(11).expand(2, 11)
  zero = torch.zeros(3)
  ident = torch.zeros(4, 3)
  ident[3] = 1
  y, _ = R.conv1d_forward(x, seg, ident, zero)
  assert torch.equal(y, x)
  shift = torch.zeros(4, 3)
  shift[0] = 1
  y, _ = R.conv1d_forward(x, seg, shift, zero)
  assert torch.equal(y[:, 3:], x[:, :-3]) and torch.all(y[:, :3] == 0)
  seg2 = seg.clone()
  seg2[:, 6] = 0  # boundary at t=6 cuts outputs 6,7,8 off x[3],x[4],x[5]
  y, _ = R.conv1d_forward(x, seg2, shift, zero)
  assert torch.all(y[:, 6:9] == 0) and torch.equal(y[:, 9:], x[:, 6:8])


def test_conv_decode_matches_prefill_and_c():
  g = torch.Generator().manual_seed(7)
  B, T, W, K = 2, 9, 8, 4
  x = torch.randn(B, T, W, generator=g, dtype=torch.float64)
  w = torch.randn(K, W, generator=g, dtype=torch.float64)
  b = torch.randn(W, generator=g, dtype=torch.float64)
  seg = torch.arange(T).expand(B, T)
  y_full, cache_full = R.conv1d_forward(x, seg, w, b)
  y_pre, cache = R.conv1d_forward(x[:, :-1], seg[:, :-1], w, b)
  y_last, cache2 = R.conv1d_forward(x[:, -1:], seg[:, -1:], w, b, cache)
  torch.testing.assert_close(y_last, y_full[:, -1:], rtol=1e-12, atol=1e-12)
  assert torch.equal(cache2, cache_full)
  # direct definition of the decode branch
  want = (torch.cat([cache, x[:, -1:]], 1) * w).sum(1, keepdim=True) + b
  torch.testing.assert_close(y_last, want, rtol=1e-12, atol=1e-12)
  yc, cc = c_ref.conv1d_step(x[:, -1:].numpy(), cache.numpy(), w.numpy(),
                             b.numpy())
  np.testing.assert_allclose(yc, y_last.numpy(), rtol=1e-12, atol=1e-12)
  np.testing.assert_array_equal(cc, cache2.numpy())
  # cache dtype is kept in decode mode, activation dtype in prefill mode
  c16 = R.conv1d_init_cache(B, W, torch.bfloat16, K)
  _, c_new = R.conv1d_forward(x[:, :1].float(), seg[:, :1], w.float(),
                              b.float(), c16)
  assert c_new.dtype == torch.bfloat16 and c_new.shape == (B, K - 1, W)


# ----------------------------------------------------- block-diag linear ---


@pytest.mark.parametrize("H,bw", [(1, 8), (4, 16), (3, 5)])
def test_block_diagonal_linear_is_dense_block_diag(H, bw):
  g = torch.Generator().manual_seed(H * 31 + bw)
  x = torch.randn(2, 3, H * bw, generator=g, dtype=torch.float64)
  w = torch.randn(H, bw, bw, generator=g, dtype=torch.float64)
  b = torch.randn(H, bw, generator=g, dtype=torch.float64)
  y = R.block_diagonal_linear(x, w, b)
  want = x @ torch.block_diag(*w) + b.flatten()
  torch.testing.assert_close(y, want, rtol=1e-12, atol=1e-12)
  yc = c_ref.block_diag_linear(x.numpy(), w.numpy(), b.numpy())
  np.testing.assert_allclose(yc, want.numpy(), rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------ scan ---


def test_scan_closed_forms():
  T, W = 50, 4
  one = torch.ones(1, T, W)
  no_reset = torch.zeros(1, T, dtype=torch.bool)
  a = torch.full((1, T, W), 0.9)
  y, h = R.rnn_scan(one, a, no_reset, None)
  t = torch.arange(1, T + 1, dtype=torch.float64)
  want = (1 - 0.9 ** t) / (1 - 0.9)
  torch.testing.assert_close(y[0, :, 0].double(), want, rtol=1e-5, atol=1e-5)
  torch.testing.assert_close(h[0, 0].double(), want[-1], rtol=1e-5, atol=1e-5)
  y, _ = R.rnn_scan(one, torch.zeros(1, T, W), no_reset, None)
  assert torch.equal(y, one)
  y, _ = R.rnn_scan(one, torch.ones(1, T, W), no_reset, None)
  assert torch.equal(y[0, :, 0], torch.arange(1, T + 1).float())
  # h0 decays geometrically under zero input
  h0 = torch.full((1, W), 3.0)
  y, _ = R.rnn_scan(torch.zeros(1, T, W), a, no_reset, h0)
  torch.testing.assert_close(y[0, :, 0].double(), 3.0 * 0.9 ** t, rtol=1e-5,
                             atol=1e-6)


def test_scan_resets_and_chunking():
  g = torch.Generator().manual_seed(11)
  B, T, W = 2, 40, 3
  x = torch.randn(B, T, W, generator=g)
  a = torch.rand(B, T, W, generator=g)
  reset = torch.rand(B, T, generator=g) < 0.15
  h0 = torch.randn(B, W, generator=g)
  y, h = R.rnn_scan(x, a, reset, h0)
  # fp64 definition
  hd = h0.double()
  for t in range(T):
    at = torch.where(reset[:, t, None], 0.0, a[:, t].double())
    hd = at * hd + x[:, t].double()
    torch.testing.assert_close(y[:, t].double(), hd, rtol=1e-5, atol=1e-5)
  torch.testing.assert_close(h.double(), hd, rtol=1e-5, atol=1e-5)
  # any split into chunks carries the state exactly (incl. 1-token chunks)
  for cut in (1, 2, 7, 39):
    y1, h1 = R.rnn_scan(x[:, :cut], a[:, :cut], reset[:, :cut], h0)
    y2, h2 = R.rnn_scan(x[:, cut:], a[:, cut:], reset[:, cut:], h1)
    assert torch.equal(torch.cat([y1, y2], 1), y) and torch.equal(h2, h)
  # single token without a state: output is the input itself
  y1, h1 = R.rnn_scan(x[:, :1], a[:, :1], reset[:, :1], None)
  assert torch.equal(y1, x[:, :1]) and torch.equal(h1, x[:, 0])


# ----------------------------------------------------------------- rglru ---


def test_rglru_zero_gates_closed_form():
  # gate weights and biases 0 -> both gates 1/2 -> a = exp(-4 softplus(L))
  W, H, T = 8, 2, 64
  g = torch.Generator().manual_seed(13)
  x = torch.randn(1, T, W, generator=g, dtype=torch.float64)
  lam = torch.linspace(-5.0, -2.5, W, dtype=torch.float64)
  zw = torch.zeros(H, W // H, W // H, dtype=torch.float64)
  zb = torch.zeros(H, W // H, dtype=torch.float64)
  seg = torch.arange(1, T + 1)[None]  # no boundary at all
  y, h = R.rglru_forward(x, seg, lam, zw, zb, zw, zb,
                         acc_dtype=torch.float64,
                         cache=torch.zeros(1, W, dtype=torch.float64))
  a = torch.exp(-4.0 * torch.log1p(torch.exp(lam)))
  k = 0.5 * torch.sqrt(1 - a * a)
  want = torch.zeros(W, dtype=torch.float64)
  for t in range(T):
    want = a * want + k * x[0, t]
    torch.testing.assert_close(y[0, t], want, rtol=1e-12, atol=1e-12)
  torch.testing.assert_close(h[0], want, rtol=1e-12, atol=1e-12)


def test_rglru_reset_identity_and_c_oracle():
  p = R.make_params(32, 4, torch.float64, seed=17, gate_bias_std=0.3)
  g = torch.Generator().manual_seed(18)
  B, T = 3, 21
  x = torch.randn(B, T, 32, generator=g, dtype=torch.float64)
  seg = helpers.document_positions(B, T, 4, seed=19)
  h0 = torch.randn(B, 32, generator=g, dtype=torch.float64)
  args = (p["a_param"], p["w_x"], p["b_x"], p["w_a"], p["b_a"])
  y, h = R.rglru_forward(x, seg, *args, cache=h0, acc_dtype=torch.float64)
  gate_x = torch.sigmoid(x @ torch.block_diag(*p["w_x"]) + p["b_x"].flatten())
  at_reset = seg == 0
  assert at_reset.sum() > 3
  torch.testing.assert_close(y[at_reset], (x * gate_x)[at_reset], rtol=1e-12,
                             atol=1e-12)
  yc, hc = c_ref.rglru(x.numpy(), seg.numpy(), *[a.numpy() for a in args],
                       h0=h0.numpy())
  np.testing.assert_allclose(yc, y.numpy(), rtol=1e-11, atol=1e-12)
  np.testing.assert_allclose(hc, h.numpy(), rtol=1e-11, atol=1e-12)
  # fp32 C oracle against the fp32 torch oracle
  p32 = {k: v.float() for k, v in p.items()}
  a32 = (p32["a_param"], p32["w_x"], p32["b_x"], p32["w_a"], p32["b_a"])
  y32, h32 = R.rglru_forward(x.float(), seg, *a32, cache=h0.float())
  yc, hc = c_ref.rglru(x.float().numpy(), seg.numpy(),
                       *[a.numpy() for a in a32], h0=h0.float().numpy())
  assert helpers.max_rel(torch.from_numpy(yc), y32) < 1e-5
  assert helpers.max_rel(torch.from_numpy(hc), h32) < 1e-5
  assert helpers.max_rel(y32, y) < 1e-5


def test_rglru_stationary_variance():
  # gates == 1/2, iid N(0,1) input: Var(h) -> (1/4)(1-a^2)/(1-a^2) = 1/4
  W, T = 16, 6000
  g = torch.Generator().manual_seed(23)
  x = torch.randn(8, T, W, generator=g)
  lam = torch.empty(W)
  torch.manual_seed(3)
  R.rnn_param_init(lam, 0.9, 0.999)
  zw, zb = torch.zeros(1, W, W), torch.zeros(1, W)
  seg = torch.arange(1, T + 1).expand(8, T)
  y, _ = R.rglru_forward(x, seg, lam, zw, zb, zw, zb)
  var = y[:, 2000:].double().var(dim=(0, 1))
  assert torch.all((var - 0.25).abs() < 0.04), var


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_core_prefill_equals_prefill_then_step(dtype):
  W, H, T, B = 64, 4, 17, 2
  p = R.make_params(W, H, dtype, seed=29, gate_bias_std=0.2)
  g = torch.Generator().manual_seed(30)
  x = torch.randn(B, T, W, generator=g).to(dtype)
  seg = torch.stack([torch.arange(T), torch.cat([torch.arange(5),
                                                 torch.arange(T - 5)])])
  y_full, c_full = R.recurrent_core(x, seg, p)
  y_pre, cache = R.recurrent_core(x[:, :-1], seg[:, :-1], p)
  y_last, c_last = R.recurrent_core(x[:, -1:], seg[:, -1:], p, cache)
  torch.testing.assert_close(torch.cat([y_pre, y_last], 1), y_full,
                             **_tol(dtype))
  torch.testing.assert_close(c_last.rg_lru_state, c_full.rg_lru_state,
                             rtol=1e-5, atol=1e-5)
  assert torch.equal(c_last.conv1d_state, c_full.conv1d_state)
  assert c_full.rg_lru_state.dtype == torch.float32
  assert c_full.conv1d_state.dtype == dtype
  y_nc, none = R.recurrent_core(x, seg, p, return_cache=False)
  assert none is None and torch.equal(y_nc, y_full)


def test_widened_close_to_truth_and_native_bf16():
  W, H, T, B = 256, 1, 96, 2
  p = R.make_params(W, H, torch.bfloat16, seed=31)
  g = torch.Generator().manual_seed(32)
  x = torch.randn(B, T, W, generator=g).to(torch.bfloat16)
  seg = helpers.document_positions(B, T, 24, seed=33)
  y_nat, _ = R.recurrent_core(x, seg, p)
  y_wide, c_wide = R.widened_recurrent_core(x, seg, p)
  p64 = {k: v.double() for k, v in p.items()}
  xc64, _ = R.conv1d_forward(x.double(), seg, p64["conv_w"], p64["conv_b"])
  y64, h64 = R.rglru_forward(xc64, seg, p64["a_param"], p64["w_x"],
                             p64["b_x"], p64["w_a"], p64["b_a"],
                             acc_dtype=torch.float64)
  e_wide = helpers.max_rel(y_wide, y64)
  e_nat = helpers.max_rel(y_nat, y64)
  assert e_wide < 5e-3, e_wide          # bf16 output rounding only
  assert e_nat < 6e-2 and e_nat > e_wide  # native bf16 is the noisier one
  assert c_wide.rg_lru_state.dtype == torch.float32
  assert helpers.max_rel(c_wide.rg_lru_state, h64) < 5e-3


# ------------------------------------------------------------ param init ---


def test_param_init_ring():
  torch.manual_seed(41)
  lam = torch.empty(20000, dtype=torch.float64)
  R.rnn_param_init(lam, 0.9, 0.999)
  radius = torch.exp(-F.softplus(lam))
  assert radius.min() >= 0.9 - 1e-6 and radius.max() <= 0.999 + 1e-6
  u = radius ** 2  # uniform on [0.81, 0.998]
  assert abs(u.mean().item() - (0.81 + 0.998001) / 2) < 2e-3
  assert abs(u.var().item() - (0.998001 - 0.81) ** 2 / 12) < 2e-4
  p = R.make_params(4096, 16, torch.float32, seed=1)
  r = torch.exp(-F.softplus(p["a_param"].double()))
  assert r.min() >= 0.9 - 1e-4 and r.max() <= 0.999 + 1e-4
  assert abs(p["w_x"].std().item() - 1 / 16) < 1e-3
  assert abs(p["conv_w"].std().item() - 0.05) < 2e-3
