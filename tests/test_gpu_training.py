"""The differentiable path (training.differentiable()) on the GPU against
gradients written by the reference's own modules under torch autograd
(tests/golden/make_grad_golden.py; float32, tiny shapes).  Tolerance 1e-4 of
the largest reference magnitude per tensor (sums in a different order on a
different device)."""

import os

import numpy as np
import pytest
import torch

import recurrentgemma_amd as rg
from recurrentgemma_amd import training

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "grad_golden.npz")
TOL = 1e-4


@pytest.fixture(scope="module")
def golden():
  return np.load(GOLDEN)


def close(got, want, what):
  want = torch.from_numpy(np.asarray(want))
  got = got.detach().cpu()
  assert got.shape == want.shape, (what, got.shape, want.shape)
  err = (got - want).abs().max().item()
  scale = max(want.abs().max().item(), 1e-6)
  assert err <= TOL * scale, (what, err, scale)


def dev(a):
  return torch.from_numpy(np.asarray(a)).to(DEV)


def test_recurrent_block_gradients(golden):
  blk = rg.RecurrentBlock(width=32, num_heads=2, lru_width=64,
                          dtype=torch.float32)
  sd = {k[len("blk/param/"):]: torch.from_numpy(golden[k])
        for k in golden.files if k.startswith("blk/param/")}
  blk.load_state_dict(sd)
  blk = blk.to(DEV)
  x = dev(golden["blk/x"]).requires_grad_(True)
  seg = dev(golden["blk/seg"])
  with training.differentiable():
    y, cache = blk(x, seg)
    loss = (y * dev(golden["blk/r"])).sum() + (
        cache.rg_lru_state * dev(golden["blk/rh"])).sum()
  loss.backward()
  close(y, golden["blk/y"], "y")
  close(cache.rg_lru_state, golden["blk/h"], "h")
  close(x.grad, golden["blk/grad/x"], "dx")
  for name, p in blk.named_parameters():
    close(p.grad, golden[f"blk/grad/{name}"], "d" + name)
  # outside the context the same module runs the inference kernels again and
  # builds no graph
  assert not training.is_enabled()
  y2, _ = blk(x, seg)
  assert not y2.requires_grad
  close(y2, golden["blk/y"], "y (kernels)")
  # the conv state returned in differentiable mode is the kernels' masked tail
  _, cache2 = blk(x, seg)
  assert torch.equal(cache.conv1d_state, cache2.conv1d_state)


def test_rglru_gradients_with_initial_state(golden):
  lru = rg.RGLRU(width=64, num_heads=2, dtype=torch.float32)
  lru.load_state_dict({k[len("lru/param/"):]: torch.from_numpy(golden[k])
                       for k in golden.files if k.startswith("lru/param/")})
  lru = lru.to(DEV)
  x = dev(golden["lru/x"]).requires_grad_(True)
  h0 = dev(golden["lru/h0"]).requires_grad_(True)
  seg = dev(golden["lru/seg"])
  with training.differentiable():
    y, h = lru(x, seg, h0)
    loss = (y * dev(golden["lru/r"])).sum() + (h * dev(golden["lru/rh"])).sum()
  loss.backward()
  close(y, golden["lru/y"], "y")
  close(h, golden["lru/h"], "h")
  close(x.grad, golden["lru/grad/x"], "dx")
  close(h0.grad, golden["lru/grad/h0"], "dh0")
  for name, p in lru.named_parameters():
    close(p.grad, golden[f"lru/grad/{name}"], "d" + name)


@pytest.mark.parametrize("T", [1, 2, 65, 300, 2050])
def test_scan_gradients_against_sequential_loop(T):
  """The scan Function alone against autograd through a float64 Python loop
  on the CPU, with resets and an initial state, at lengths that span one and
  several steps of the scan kernel."""
  gen = torch.Generator().manual_seed(T)
  B, W = 3, 96
  x = torch.randn(B, T, W, generator=gen)
  a = torch.rand(B, T, W, generator=gen) * 0.5 + 0.5
  h0 = torch.randn(B, W, generator=gen)
  reset = torch.rand(B, T, generator=gen) < 0.1
  r, rh = torch.randn(B, T, W, generator=gen), torch.randn(B, W, generator=gen)

  xd, ad, hd = (t.double().requires_grad_(True) for t in (x, a, h0))
  h, ys = hd, []
  for t in range(T):
    h = ad[:, t] * (~reset[:, t])[:, None] * h + xd[:, t]
    ys.append(h)
  ((torch.stack(ys, 1) * r).sum() + (h * rh).sum()).backward()

  xg, ag, hg = (t.to(DEV).requires_grad_(True) for t in (x, a, h0))
  with training.differentiable():
    y, hl = rg.rnn_scan(xg, ag, reset.to(DEV), hg)
  ((y * r.to(DEV)).sum() + (hl * rh.to(DEV)).sum()).backward()
  close(y, torch.stack(ys, 1).float().detach().numpy(), "y")
  close(xg.grad, xd.grad.float().numpy(), "dx")
  close(ag.grad, ad.grad.float().numpy(), "da")
  close(hg.grad, hd.grad.float().numpy(), "dh0")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,W", [(2, 1, 64), (3, 17, 96), (1, 333, 130),
                                   (2, 1000, 257), (1, 4099, 512)])
def test_scan_backward_kernel(dtype, B, T, W):
  """rg_linear_scan_backward against its definition evaluated step by step in
  float64 on the same (dtype-valued) inputs: g_t = dy_t + a'_{t+1} g_{t+1}
  with dh_last behind the last token, dx = g, da = g h_{t-1} masked at resets,
  dh0 = a'_0 g_0; widths that take two channels per lane and one, sequences
  from one token to several rows per wave, with and without h0 / dh_last."""
  from recurrentgemma_amd import ops
  gen = torch.Generator().manual_seed(B * 1000 + T)
  dy = torch.randn(B, T, W, generator=gen).to(dtype)
  a = (torch.rand(B, T, W, generator=gen) * 0.6 + 0.4).to(dtype)
  y = torch.randn(B, T, W, generator=gen).to(dtype)
  reset = torch.rand(B, T, generator=gen) < 0.05
  h0 = torch.randn(B, W, generator=gen)
  dh_last = torch.randn(B, W, generator=gen)
  tol = 1e-5 if dtype == torch.float32 else 1e-2
  for with_state in (True, False):
    got_dx, got_da, got_dh0 = ops.linear_scan_backward(
        dy.to(DEV), a.to(DEV), reset.to(DEV), y.to(DEV),
        h0.to(DEV) if with_state else None,
        dh_last.to(DEV) if with_state else None)
    ae = a.double() * (~reset)[..., None]
    g = dh_last.double() if with_state else torch.zeros(B, W, dtype=torch.float64)
    dx = torch.zeros(B, T, W, dtype=torch.float64)
    for t in range(T - 1, -1, -1):
      coef = ae[:, t + 1] if t + 1 < T else 1.0
      g = dy[:, t].double() + coef * g
      dx[:, t] = g
    first = (h0.to(dtype).double() if with_state
             else torch.zeros(B, W, dtype=torch.float64))
    h_prev = torch.cat([first[:, None], y[:, :-1].double()], dim=1)
    da = dx * h_prev * (~reset)[..., None]
    scale = lambda t: t.abs().max().clamp_min(1e-30)
    assert ((got_dx.double().cpu() - dx).abs().max() / scale(dx)) < tol
    assert ((got_da.double().cpu() - da).abs().max() / scale(da)) < tol
    assert got_dx.dtype == dtype and got_da.dtype == dtype
    if with_state:
      dh0 = ae[:, 0] * dx[:, 0]
      assert ((got_dh0.double().cpu() - dh0).abs().max() / scale(dh0)) < 1e-5
    else:
      assert got_dh0 is None


def _rglru_against_float64(dtype, B, T, W, H, where):
  """Runs training.rg_lru forward and backward on the GPU and the reference's
  formulas under float64 autograd with a loop over time on `where`, on the
  same dtype-valued inputs; compares y, h_last and every gradient."""
  from oracle import torch_ref as R
  gen = torch.Generator().manual_seed(B * 1000 + T)
  p = R.make_params(W, H, dtype, seed=T + 5, gate_bias_std=0.3)
  x = torch.randn(B, T, W, generator=gen).to(dtype)
  h0 = torch.randn(B, W, generator=gen)
  seg = torch.arange(T).expand(B, T).clone()
  for b in range(B):
    for start in torch.nonzero(torch.rand(T, generator=gen) < 0.04).flatten():
      seg[b, start:] = torch.arange(T - int(start))
  if T > 1:
    seg[0, 0] = 7  # a row that continues a document: h0 counts
  r = torch.randn(B, T, W, generator=gen)
  rh = torch.randn(B, W, generator=gen)
  names = ("a_param", "w_x", "b_x", "w_a", "b_a")

  # float64
  q = {k: p[k].double().to(where).requires_grad_(True) for k in names}
  xd = x.double().to(where).requires_grad_(True)
  hd = h0.double().to(where).requires_grad_(True)
  reset = (seg == 0).to(where)

  class BoundedSqrt(torch.autograd.Function):
    @staticmethod
    def forward(ctx, v):
      ctx.save_for_backward(v)
      return torch.sqrt(v)

    @staticmethod
    def backward(ctx, grad):
      (v,) = ctx.saved_tensors
      return grad / torch.sqrt(torch.clip(4.0 * v, min=1 / 1000.0 ** 2))

  def bdl(v, w, b):
    vs = v.reshape(B, T, H, W // H)
    return (torch.einsum("bthi,hij->bthj", vs, w) + b).reshape(B, T, W)

  # the kernels take the pre-activations as tensors of the activation dtype
  def as_dtype(v):
    return v + (v.detach().to(dtype).double() - v.detach())
  gx = torch.sigmoid(as_dtype(bdl(xd, q["w_x"], q["b_x"])))
  ga = torch.sigmoid(as_dtype(bdl(xd, q["w_a"], q["b_a"])))
  log_a = -8.0 * ga * torch.nn.functional.softplus(q["a_param"])
  a = torch.exp(log_a)
  mult = BoundedSqrt.apply(1 - torch.exp(2 * log_a))
  mult = reset[..., None] + ~reset[..., None] * mult
  xn = xd * gx * mult
  h, ys = hd, []
  for t in range(T):
    h = a[:, t] * (~reset[:, t])[:, None] * h + xn[:, t]
    ys.append(h)
  yd = torch.stack(ys, 1)
  ((yd * r.to(where)).sum() + (h * rh.to(where)).sum()).backward()

  # the kernels
  qg = {k: p[k].to(DEV).requires_grad_(True) for k in names}
  xg, hg = x.to(DEV).requires_grad_(True), h0.to(DEV).requires_grad_(True)
  with training.differentiable():
    y, hl = training.rg_lru(xg, seg.to(DEV), qg["a_param"], qg["w_x"],
                            qg["b_x"], qg["w_a"], qg["b_a"], hg)
  ((y.float() * r.to(DEV)).sum() + (hl * rh.to(DEV)).sum()).backward()

  tol = 1e-4 if dtype == torch.float32 else 2e-2

  def near(got, want, what):
    want = want.detach().double().cpu()
    err = (got.detach().double().cpu() - want).abs().max().item()
    scale = max(want.abs().max().item(), 1e-12)
    assert err <= tol * scale, (what, err, scale)

  near(y, yd, "y")
  near(hl, h, "h_last")
  near(xg.grad, xd.grad, "dx")
  near(hg.grad, hd.grad, "dh0")
  for k in names:
    assert qg[k].grad.dtype == dtype
    near(qg[k].grad, q[k].grad, "d" + k)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,W,H", [(2, 1, 64, 2), (3, 19, 96, 3),
                                     (1, 333, 130, 1), (2, 700, 256, 2),
                                     (2, 150, 512, 2)])
def test_rglru_backward_kernel(dtype, B, T, W, H):
  """training.rg_lru (forward and backward kernels from the gate
  pre-activations on) against autograd through the reference's formulas
  (layers.py:335-360, the sqrt with its clipped derivative :216-230) evaluated
  in float64 on the CPU with a loop over time, on the same dtype-valued
  inputs: y, h_last and the gradients of x, both gate matrices and biases,
  a_param and h0; document starts, one and two channels per lane, sequences of
  one token up to several rows per wave; the last shape has 256-wide heads
  (bf16: the gate projections and all their gradients on the matrix kernels).  Tolerance relative to the largest
  magnitude of each tensor: 1e-4 float32 (sums in another order), 2e-2 bf16
  (the kernels round x, the pre-activations, y and each gradient to bf16)."""
  _rglru_against_float64(dtype, B, T, W, H, "cpu")


@pytest.mark.parametrize("dtype,B,T,W,H", [
    (torch.bfloat16, 4, 2048, 2560, 10), (torch.float32, 4, 2048, 2560, 10),
    (torch.bfloat16, 2, 8192, 4096, 16)])
def test_rglru_backward_kernel_full_size_rows(dtype, B, T, W, H):
  """The same comparison at the lengths and widths of the listed
  configurations (2B: 2048 tokens x 2560, 10 heads; 9B: two rows of 8192
  tokens x 4096, 16 heads), the float64 loop over time on the GPU: every
  chunk boundary of a full-length row, the gate projections' kernels at their
  real row counts.  Same tolerances."""
  _rglru_against_float64(dtype, B, T, W, H, DEV)


def test_rglru_forms_agree():
  """The fused form against the same layer as tensor ops around the scan
  kernels, both on the GPU in float32."""
  from oracle import torch_ref as R
  B, T, W, H = 2, 500, 512, 2
  gen = torch.Generator().manual_seed(3)
  p = R.make_params(W, H, torch.float32, seed=9, gate_bias_std=0.3)
  x = torch.randn(B, T, W, generator=gen)
  seg = torch.arange(T).expand(B, T).clone()
  seg[1, 200:] -= 200
  r = torch.randn(B, T, W, generator=gen).to(DEV)
  names = ("a_param", "w_x", "b_x", "w_a", "b_a")
  grads = []
  for fn in (training.rg_lru, training.rg_lru_tensor_ops):
    q = {k: p[k].to(DEV).requires_grad_(True) for k in names}
    xg = x.to(DEV).requires_grad_(True)
    with training.differentiable():
      y, _ = fn(xg, seg.to(DEV), *(q[k] for k in names))
    (y * r).sum().backward()
    grads.append([y, xg.grad] + [q[k].grad for k in names])
  for got, want, what in zip(grads[0], grads[1], ("y", "dx") + names):
    err = (got - want).abs().max().item()
    assert err <= 1e-4 * want.abs().max().item(), (what, err)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,W,H", [(2, 70, 512, 2), (1, 300, 2560, 10),
                                     (3, 17, 192, 3), (2, 5, 64, 1)])
def test_block_diagonal_linear_gradients(dtype, B, T, W, H):
  """BlockDiagonalLinear in differentiable mode (kernels both ways) against
  the reference's two tensor ops (layers.py:127-137) under autograd in
  float32 on the same values."""
  gen = torch.Generator().manual_seed(B * T + W)
  bw = W // H
  x = torch.randn(B, T, W, generator=gen).to(dtype)
  w = (torch.randn(H, bw, bw, generator=gen) / bw ** 0.5).to(dtype)
  b = (torch.randn(H, bw, generator=gen) * 0.3).to(dtype)
  r = torch.randn(B, T, W, generator=gen).to(dtype).to(DEV)
  m = rg.BlockDiagonalLinear(W, H, dtype=dtype)
  m.load_state_dict({"w": w, "b": b})
  m = m.to(DEV)
  xg = x.to(DEV).requires_grad_(True)
  with training.differentiable():
    y = m(xg)
    if dtype == torch.float32:
      # (float32 takes the library's batched products by default: call the
      # kernel form directly)
      y = training._BlockDiagLinear.apply(xg, m.w, m.b)
  assert y.requires_grad and y.dtype == dtype
  y.backward(r)
  ref = [t.to(DEV).float().requires_grad_(True) for t in (x, w, b)]
  yr = training.block_diag_linear_tensor_ops(*ref)
  yr.backward(r.float())
  tol = 1e-5 if dtype == torch.float32 else 1e-2
  for got, want, what in ((y, yr, "y"), (xg.grad, ref[0].grad, "dx"),
                          (m.w.grad, ref[1].grad, "dw"),
                          (m.b.grad, ref[2].grad, "db")):
    assert got.dtype == dtype and got.shape == want.shape, what
    err = (got.float() - want).abs().max().item()
    assert err <= tol * want.abs().max().item(), (what, err)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,W,K", [(2, 1, 64, 4), (3, 19, 96, 4),
                                     (2, 100, 300, 4), (1, 70, 64, 2),
                                     (2, 45, 130, 7)])
def test_conv_backward_kernel(dtype, B, T, W, K):
  """training.conv1d (conv kernel forwards, rg_conv1d_backward backwards)
  against autograd through the conv's definition written out token by token
  in float64 on the CPU (tap s of token t is x[t-s] unless a document starts
  at one of t-s+1 .. t; layers.py:477-520), same dtype-valued inputs: output
  and the gradients of x, w and b; document starts including in the last and
  first positions, temporal widths 2, 4 and 7, row counts that fill one
  32-row chunk of the kernel, several and a part of one.  Tolerance relative
  to each tensor's largest magnitude: 1e-5 float32, 1e-2 bf16."""
  gen = torch.Generator().manual_seed(B * 100 + T + K)
  x = torch.randn(B, T, W, generator=gen).to(dtype)
  w = (torch.randn(K, W, generator=gen) * 0.5).to(dtype)
  b = torch.randn(W, generator=gen).to(dtype)
  r = torch.randn(B, T, W, generator=gen).to(dtype)
  seg = torch.arange(T).expand(B, T).clone()
  for row in range(B):
    for start in torch.nonzero(torch.rand(T, generator=gen) < 0.1).flatten():
      seg[row, start:] = torch.arange(T - int(start))
  seg[-1, T - 1] = 0
  if T > 1:
    seg[0, 0] = 5

  xd, wd, bd = (t.double().requires_grad_(True) for t in (x, w, b))
  rows = []
  for t in range(T):
    acc = bd.expand(B, W)
    alive = torch.ones(B, dtype=torch.bool)
    for s in range(min(K, t + 1)):
      if s > 0:
        alive = alive & (seg[:, t - s + 1] != 0)
      acc = acc + xd[:, t - s] * alive[:, None] * wd[K - 1 - s]
    rows.append(acc)
  outd = torch.stack(rows, 1)
  (outd * r.double()).sum().backward()

  xg, wg, bg = (t.to(DEV).requires_grad_(True) for t in (x, w, b))
  with training.differentiable():
    out = training.conv1d(xg, seg.to(DEV), wg, bg)
  (out.float() * r.to(DEV).float()).sum().backward()
  tol = 1e-5 if dtype == torch.float32 else 1e-2

  def near(got, want, what):
    want = want.detach().double()
    err = (got.detach().double().cpu() - want).abs().max().item()
    assert err <= tol * max(want.abs().max().item(), 1e-12), (what, err)

  near(out, outd, "out")
  near(xg.grad, xd.grad, "dx")
  near(wg.grad, wd.grad, "dw")
  near(bg.grad, bd.grad, "db")
  assert xg.grad.dtype == dtype and wg.grad.dtype == dtype

  # and the tensor-op form of the same conv on the GPU
  x2, w2, b2 = (t.to(DEV).requires_grad_(True) for t in (x, w, b))
  out2 = training.conv1d_tensor_ops(x2, seg.to(DEV), w2, b2)
  (out2.float() * r.to(DEV).float()).sum().backward()
  near(x2.grad, xd.grad, "dx (tensor ops)")



@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,W,K", [(2, 40000, 64, 4), (3, 9000, 64, 4),
                                     (1, 70000, 32, 2)])
def test_conv_backward_kernel_many_rows(dtype, B, T, W, K):
  """rg_conv1d_backward where a chunk of its partial sums covers more than 32
  rows (64, 128 or 256: the kernel widens its chunks once there would be more
  than 512 of them): dx, dw and db against autograd through the tensor-op
  form of the same conv (training.conv1d_tensor_ops, which the test above
  pins to the definition) evaluated in float64 on the same dtype-valued
  inputs.  Tolerances as above; the number of planes is what the library
  says."""
  from tests import helpers
  from recurrentgemma_amd import _lib
  gen = torch.Generator().manual_seed(B + T + K)
  x = torch.randn(B, T, W, generator=gen).to(dtype)
  w = (torch.randn(K, W, generator=gen) * 0.5).to(dtype)
  b = torch.randn(W, generator=gen).to(dtype)
  r = (torch.randn(B, T, W, generator=gen) / (B * T) ** 0.5).to(dtype)
  seg = helpers.document_positions(B, T, 300, seed=T)
  seg[-1, T - 1] = 0

  lib = _lib.lib()
  planes = lib.rg_conv1d_backward_workspace_bytes(B, T, W, K) // ((K + 1) * W * 4)
  assert planes <= 512 and planes * 32 < B * T <= planes * 256

  x2, w2, b2 = (t.to(DEV).double().requires_grad_(True) for t in (x, w, b))
  out2 = training.conv1d_tensor_ops(x2, seg.to(DEV), w2, b2)
  (out2 * r.to(DEV).double()).sum().backward()

  xg, wg, bg = (t.to(DEV).requires_grad_(True) for t in (x, w, b))
  with training.differentiable():
    out = training.conv1d(xg, seg.to(DEV), wg, bg)
  (out.float() * r.to(DEV).float()).sum().backward()
  tol = 1e-5 if dtype == torch.float32 else 1e-2

  def near(got, want, what):
    want = want.detach().double()
    err = (got.detach().double() - want).abs().max().item()
    assert err <= tol * max(want.abs().max().item(), 1e-12), (what, err)

  near(xg.grad, x2.grad, "dx")
  near(wg.grad, w2.grad, "dw")
  near(bg.grad, b2.grad, "db")


@pytest.mark.parametrize("M,H", [(1, 1), (64, 1), (100, 2), (257, 3),
                                 (4099, 3), (8192, 10), (300, 16),
                                 (131072, 16)])
def test_gate_weight_gradients_kernel(M, H):
  """rg_gates_weight_grads (both gate projections' dw and db in one pass,
  bf16, 256-wide heads) against the definition
  dw[h,i,j] = sum_m x[m,h,i] dy[m,h,j], db[h,j] = sum_m dy[m,h,j]
  (autograd of layers.py:134-136) in float64 on the same bf16-valued inputs:
  one row, row counts below, at and off the kernel's 64-row steps and its
  splits of the rows, 1 to 16 heads, up to the 16 x 8192 rows of the widest
  configuration.  Tolerance: the bf16 rounding of the
  result (2^-8 of each tensor's largest magnitude); the same bits on a second
  run (fixed summation order)."""
  W = 256 * H
  gen = torch.Generator().manual_seed(M * 31 + H)
  x = torch.randn(M, W, generator=gen).to(torch.bfloat16).to(DEV)
  d0 = torch.randn(M, W, generator=gen).to(torch.bfloat16).to(DEV)
  d1 = (torch.randn(M, W, generator=gen) * 3).to(torch.bfloat16).to(DEV)
  got = rg.ops.gates_weight_grads(x, d0, d1, H)
  again = rg.ops.gates_weight_grads(x, d0, d1, H)
  xh = x.double().view(M, H, 256)
  for d, dw, db, dw2, db2 in ((d0, got[0], got[2], again[0], again[2]),
                              (d1, got[1], got[3], again[1], again[3])):
    dh = d.double().view(M, H, 256)
    want_w = torch.einsum("mhi,mhj->hij", xh, dh)
    want_b = dh.sum(0)
    assert dw.shape == (H, 256, 256) and db.shape == (H, 256)
    assert dw.dtype == torch.bfloat16 and db.dtype == torch.bfloat16
    assert (dw.double() - want_w).abs().max() <= 2 ** -8 * want_w.abs().max()
    assert (db.double() - want_b).abs().max() <= 2 ** -8 * want_b.abs().max()
    assert torch.equal(dw, dw2) and torch.equal(db, db2)
  # without the bias gradients
  only_w = rg.ops.gates_weight_grads(x, d0, d1, H, with_bias=False)
  assert only_w[2] is None and only_w[3] is None
  assert torch.equal(only_w[0], got[0]) and torch.equal(only_w[1], got[1])


def test_gate_weight_gradients_kernel_refuses_other_shapes():
  x = torch.zeros(8, 384, dtype=torch.bfloat16, device=DEV)
  with pytest.raises(ValueError, match="256-wide"):
    rg.ops.gates_weight_grads(x, x, x, 3)
  lib = rg._lib.lib()
  assert lib.rg_gates_weight_grads_workspace_bytes(8, 384, 3) == 0
  p = x.data_ptr()
  rc = lib.rg_gates_weight_grads(p, p, p, p, p, None, None, p, 1 << 20, 8, 384,
                                 3, 1, None)
  assert rc == -2 and b"256-wide" in lib.rg_last_error()
  x = torch.zeros(8, 256, dtype=torch.float32, device=DEV)
  rc = lib.rg_gates_weight_grads(p, p, p, p, p, None, None, p, 1 << 20, 8, 256,
                                 1, 0, None)
  assert rc == -2
  # a workspace that is too small
  need = lib.rg_gates_weight_grads_workspace_bytes(8, 256, 1)
  assert need > 0
  rc = lib.rg_gates_weight_grads(p, p, p, p, p, None, None, p, need - 1, 8, 256,
                                 1, 1, None)
  assert rc == -4 and b"workspace" in lib.rg_last_error()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(1, 1, 3), (1, 1, 7), (2, 17, 96),
                                   (1, 343, 3), (3, 333, 130),
                                   (4, 2048, 2560)])
def test_gelu_join_backward_kernel(dtype, shape):
  """rg_gelu_mul_backward against float64 autograd of torch's own
  a * gelu(g, approximate="tanh") (modules.py:289-291, :644) on the same
  inputs: element counts below, at and off the kernel's 16-byte items, g over
  both tails of the activation.  Per element: float32 1e-5 of the value plus
  the cancellation in 1 + tanh (1e-6 of |dout| max(1,|a|) max(1,|g|)); bf16 the
  two roundings the reference's graph has as well (2^-7 of the value) plus the
  same absolute term at 1e-5."""
  gen = torch.Generator().manual_seed(sum(shape))
  a = torch.randn(shape, generator=gen).to(dtype).to(DEV)
  g = (torch.randn(shape, generator=gen) * 3).to(dtype).to(DEV)
  dout = torch.randn(shape, generator=gen).to(dtype).to(DEV)
  d_a, d_g = rg.ops.gelu_mul_backward(dout, a, g)
  assert d_a.dtype == dtype and d_g.dtype == dtype
  assert d_a.shape == a.shape and d_g.shape == g.shape
  a64 = a.double().requires_grad_()
  g64 = g.double().requires_grad_()
  out = a64 * torch.nn.functional.gelu(g64, approximate="tanh")
  out.backward(dout.double())
  rel, floor = (1e-5, 1e-6) if dtype == torch.float32 else (2.0 ** -7, 1e-5)
  slack = floor * dout.double().abs() * a64.detach().abs().clamp(min=1) * \
      g64.detach().abs().clamp(min=1)
  for got, want, what in ((d_a, a64.grad, "d_a"), (d_g, g64.grad, "d_g")):
    over = (got.double() - want).abs() - (rel * want.abs() + slack)
    assert over.max().item() <= 0, (what, over.max().item())


def test_gelu_join_under_autograd_matches_tensor_ops():
  """training.gelu_mul (kernels both ways) against the same join written as
  tensor ops, values and both gradients, float32 (1e-5) and bf16 (1e-2 of the
  largest magnitude)."""
  for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
    gen = torch.Generator().manual_seed(5)
    a0 = torch.randn(2, 300, 512, generator=gen).to(dtype).to(DEV)
    g0 = (torch.randn(2, 300, 512, generator=gen) * 2).to(dtype).to(DEV)
    dout = torch.randn(2, 300, 512, generator=gen).to(dtype).to(DEV)
    a1, g1 = a0.clone().requires_grad_(), g0.clone().requires_grad_()
    a2, g2 = a0.clone().requires_grad_(), g0.clone().requires_grad_()
    out1 = training.gelu_mul(a1, g1)
    out1.backward(dout)
    out2 = a2 * torch.nn.functional.gelu(g2, approximate="tanh")
    out2.backward(dout)
    for got, want, what in ((out1, out2, "out"), (a1.grad, a2.grad, "d_a"),
                            (g1.grad, g2.grad, "d_g")):
      err = (got.float() - want.float()).abs().max().item()
      assert err <= tol * want.float().abs().max().item(), (dtype, what, err)


def test_gelu_join_backward_entry_rejects_bad_arguments():
  lib = rg._lib.lib()
  x = torch.zeros(64, dtype=torch.float32, device=DEV)
  y = torch.zeros(64, dtype=torch.float32, device=DEV)
  z = torch.zeros(64, dtype=torch.float32, device=DEV)
  p, q, r = x.data_ptr(), y.data_ptr(), z.data_ptr()
  assert lib.rg_gelu_mul_backward(p, p, p, q, r, 0, 0, None) == -1
  assert lib.rg_gelu_mul_backward(p, p, p, q, q, 64, 0, None) == -1
  assert b"alias" in lib.rg_last_error()
  assert lib.rg_gelu_mul_backward(p, p, p, p, r, 64, 0, None) == -1
  assert lib.rg_gelu_mul_backward(p, p, p, q + 4, r, 32, 0, None) == -1
  assert b"aligned" in lib.rg_last_error()
  assert lib.rg_gelu_mul_backward(p, p, p, q, r, 64, 7, None) == -2
  assert lib.rg_gelu_mul_backward(None, p, p, q, r, 64, 0, None) == -1
