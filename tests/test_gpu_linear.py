"""The linear layers for few rows (rg_linear_pack / rg_linear_rows), on the GPU.

Reference: the exact product in float64 on the host.  The kernel accumulates
in float32 and rounds once to bf16, so a result may differ from the rounded
exact value by the float32 accumulation error (bounded here by 2e-5 of the
sum of absolute terms) plus one bf16 ulp where that error crosses a rounding
boundary.  Residual add, gelu pairs and grouped outputs are checked bit for
bit against the same kernel's plain output followed by the separate steps
(torch's add, this package's rg_gelu_mul)."""

import copy

import pytest
import torch

from recurrentgemma_amd import griffin as G
from recurrentgemma_amd import ops

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
BF = torch.bfloat16


def _rand(gen, *shape, scale=1.0):
  return (torch.randn(*shape, generator=gen) * scale).to(BF)


def _check(got, x, w_rows, bias):
  """got [M, N] against x [M, K] @ w_rows [N, K]^T + bias in float64."""
  xd, wd = x.double(), w_rows.double()
  exact = xd @ wd.T
  bound = 2e-5 * (xd.abs() @ wd.abs().T)
  if bias is not None:
    exact = exact + bias.double()
    bound = bound + 2e-5 * bias.double().abs()
  ulp = torch.maximum(exact.abs(), torch.tensor(1e-30, dtype=torch.float64))
  ulp = 2.0 ** (torch.floor(torch.log2(ulp)) - 7)
  err = (got.cpu().double() - exact).abs()
  worst = (err - bound - ulp).max().item()
  assert worst <= 0, worst


@pytest.mark.parametrize("M,K,N,with_bias", [
    (64, 2560, 2560, True),    # one tile of 32 weight rows per workgroup
    (5, 128, 64, False),       # fewer rows than a tile, two chunks of K
    (33, 192, 96, True),       # second half-tile partly filled, odd chunk count
    (64, 7680, 2560, True),    # K split over the grid, finished by a second pass
    (1, 2560, 15360, True),    # two tiles per workgroup
])
def test_linear_rows(M, K, N, with_bias):
  gen = torch.Generator().manual_seed(M * 7 + K + N)
  x = _rand(gen, M, K)
  w = _rand(gen, N, K, scale=K ** -0.5)
  b = _rand(gen, N) if with_bias else None
  layer = ops.PackedLinear()
  xg, wg = x.to(DEV), w.to(DEV)
  bg = None if b is None else b.to(DEV)
  got = layer(xg, (wg,), None if bg is None else (bg,))
  assert got.shape == (M, N) and got.dtype == BF
  _check(got, x, w, b)
  # leading dimensions are rows; same bits on a second run
  again = layer(xg.reshape(1, M, K), (wg,), None if bg is None else (bg,))
  assert torch.equal(again[0], got)
  for _ in range(10):  # whichever workgroup adds the slices of K, same sum
    assert torch.equal(layer(xg, (wg,), None if bg is None else (bg,)), got)
  # residual: added after the product is rounded, like a separate add
  res = _rand(gen, M, N).to(DEV)
  with_res = layer(xg, (wg,), None if bg is None else (bg,), residual=res)
  assert torch.equal(with_res, got + res)
  # against the library product of the same operands: a few bf16 ulps
  lib = torch.nn.functional.linear(xg, wg, bg)
  scale = lib.float().abs().max().item()
  assert (lib.float() - got.float()).abs().max().item() <= 2 ** -6 * scale


def test_linear_rows_shape_sweep():
  """Seeded sweep over row counts, depths and widths the packed layout takes
  (every M from 1 to 64 occurs among the tile boundaries 31/32/33/63/64; odd
  numbers of K chunks; widths that leave the last workgroups short)."""
  rng = torch.Generator().manual_seed(2024)
  shapes = [(1, 64, 32), (31, 64, 32), (32, 128, 96), (33, 320, 160),
            (63, 448, 32), (64, 704, 416), (17, 1088, 64), (48, 64, 2048)]
  for _ in range(12):
    M = int(torch.randint(1, 65, (1,), generator=rng))
    K = 64 * int(torch.randint(1, 24, (1,), generator=rng))
    N = 32 * int(torch.randint(1, 40, (1,), generator=rng))
    shapes.append((M, K, N))
  for M, K, N in shapes:
    x = _rand(rng, M, K)
    w = _rand(rng, N, K, scale=K ** -0.5)
    b = _rand(rng, N) if (M + N) % 2 else None
    got = ops.PackedLinear()(x.to(DEV), (w.to(DEV),),
                             None if b is None else (b.to(DEV),))
    _check(got, x, w, b)


def test_layers_packed_together():
  """Two nn.Linear layers on the same input as one launch: each output equals
  the layer run alone."""
  gen = torch.Generator().manual_seed(11)
  M, K, N = 64, 2560, 2560
  x = _rand(gen, M, K).to(DEV)
  w1, w2 = (_rand(gen, N, K, scale=K ** -0.5).to(DEV) for _ in range(2))
  b1, b2 = (_rand(gen, N).to(DEV) for _ in range(2))
  both = ops.PackedLinear()(x, (w1, w2), (b1, b2))
  assert len(both) == 2
  assert torch.equal(both[0], ops.PackedLinear()(x, (w1,), (b1,)))
  assert torch.equal(both[1], ops.PackedLinear()(x, (w2,), (b2,)))
  # unequal layers: one output, each slice the layer run alone
  joined = ops.PackedLinear()(x, (w1, w2[:64], w2[64:320]),
                              (b1, b2[:64], b2[64:320]))
  assert joined.shape == (M, N + 320)
  assert torch.equal(joined[:, :N], both[0])
  assert torch.equal(joined[:, N:], both[1][:, :320])
  with pytest.raises(ValueError):
    ops.PackedLinear()(x, (w1, w2[:40]), (b1, b2[:40]))


@pytest.mark.parametrize("M,K,E", [(64, 2560, 7680), (3, 128, 96)])
def test_stacked_weight_and_gelu_pairs(M, K, E):
  """The MLP's stacked up-projection [2, K, E] (Einsum "cdD" layout): plain
  outputs against float64, the fused gelu(gate) * up against rg_gelu_mul on
  those outputs."""
  gen = torch.Generator().manual_seed(E)
  x = _rand(gen, M, K)
  w = _rand(gen, 2, K, E, scale=K ** -0.5)
  b = _rand(gen, 2, 1, 1, E)
  xg, wg, bg = x.to(DEV), w.to(DEV), b.to(DEV)
  gate, up = ops.PackedLinear(layout=1)(xg, (wg,), (bg,))
  _check(gate, x, w[0].T, b[0].reshape(-1))
  _check(up, x, w[1].T, b[1].reshape(-1))
  if E % 32 == 0:
    fused = ops.PackedLinear(layout=1, gelu_pair=True)(xg, (wg,), (bg,))
    assert fused.shape == (M, E)
    assert torch.equal(fused, ops.gelu_mul(up.contiguous(), gate.contiguous()))


@pytest.mark.parametrize("M,K,N,with_addend", [
    (64, 2560, 2560, True), (64, 7680, 2560, True), (7, 256, 256, False)])
def test_partial_sums_into_the_norm(M, K, N, with_addend):
  """A layer left as partial sums over slices of K and the norm kernel that
  adds them: the values of adding the slices in order, bias, rounding, the
  addend, rounding and rg_rms_norm as separate steps."""
  gen = torch.Generator().manual_seed(K + N + M)
  x = _rand(gen, M, K)
  w = _rand(gen, N, K, scale=K ** -0.5)
  b = _rand(gen, N)
  scale = _rand(gen, N, scale=0.3).to(DEV)
  addend = _rand(gen, 1, M, N).to(DEV) if with_addend else None
  layer = ops.PackedLinear()
  xg = x.to(DEV).reshape(1, M, K)
  assert ops.PackedLinear.partial_slices(xg, K, N) == 3
  ps = layer.partial(xg, (w.to(DEV),), (b.to(DEV),))
  assert ps.sums.shape == (3, M, N) and ps.shape == (1, M, N)
  plain = ps.materialize()
  _check(plain[0], x, w, b)
  want_total = plain if addend is None else plain + addend
  total, normed = ops.add_rms_norm(ps, addend, scale)
  assert torch.equal(total, want_total)
  assert torch.equal(normed, ops.rms_norm(want_total, scale))
  # the addend may also ride in the partial sums (a skip connection)
  if addend is not None:
    ps.addend = addend
    assert torch.equal(ps.materialize(), want_total)
    total2, normed2 = ops.add_rms_norm(ps, None, scale)
    assert torch.equal(total2, total) and torch.equal(normed2, normed)
    with pytest.raises(ValueError):
      ops.add_rms_norm(ps, addend, scale)
  # many weight rows: splitting K is not worth it
  assert ops.PackedLinear.partial_slices(xg, K, 15360) == 0


def test_repacks_when_a_weight_changes():
  gen = torch.Generator().manual_seed(3)
  x = _rand(gen, 8, 128).to(DEV)
  w = _rand(gen, 64, 128).to(DEV)
  layer = ops.PackedLinear()
  first = layer(x, (w,))
  w.mul_(2.0)  # exact in bf16
  assert torch.equal(layer(x, (w,)), first * 2.0)
  other = _rand(gen, 64, 128).to(DEV)
  _check(layer(x, (other,)), x.cpu(), other.cpu(), None)
  assert copy.deepcopy(layer)._packed is None


def test_unsupported_shapes_are_refused():
  x = torch.zeros(4, 100, dtype=BF, device=DEV)
  assert not ops.PackedLinear.usable(x, 100, 64)         # K % 64
  assert not ops.PackedLinear.usable(x.float(), 100, 64)
  x = torch.zeros(65, 128, dtype=BF, device=DEV)
  assert not ops.PackedLinear.usable(x, 128, 64)         # more than 64 rows
  assert ops.PackedLinear.usable(x[:64], 128, 64)
  with pytest.raises(ValueError):
    ops.PackedLinear()(x[:4], (torch.zeros(48, 128, dtype=BF, device=DEV),))


def test_decode_steps_with_and_without_the_row_kernels(monkeypatch):
  """A small bf16 model: prompt, then three cached steps, once with the
  linear layers of the steps on rg_linear_rows and once on the library
  products.  Same weights, different summation order: logits agree to bf16
  noise."""
  R, A = G.TemporalBlockType.RECURRENT, G.TemporalBlockType.ATTENTION
  cfg = G.GriffinConfig(
      vocab_size=512, width=256, mlp_expanded_width=768, num_heads=2,
      block_types=(R, A, R), embeddings_scale_by_sqrt_dim=True,
      attention_window_size=16, logits_soft_cap=30.0, lru_width=256)
  torch.manual_seed(5)
  model = G.Griffin(cfg, dtype=BF).to(DEV).eval()
  gen = torch.Generator().manual_seed(6)
  B, T = 4, 20  # 80 rows: the prompt pass stays on the library products
  tokens = torch.randint(0, 512, (B, T + 3), generator=gen).to(DEV)
  pos = torch.arange(T + 3, device=DEV)[None].expand(B, -1).to(torch.int32)

  def run():
    _, cache = model(tokens[:, :T], pos[:, :T], None, return_logits=False,
                     return_cache=True)
    outs = []
    for i in range(T, T + 3):
      logits, cache = model(tokens[:, i:i + 1], pos[:, i:i + 1], cache,
                            return_logits=True, return_cache=True)
      outs.append(logits.float())
    return torch.stack(outs)

  calls = []
  real = ops.PackedLinear.__call__

  def counting(self, *a, **k):
    calls.append(1)
    return real(self, *a, **k)

  partials = []
  real_partial = ops.PackedLinear.partial

  def counting_partial(self, *a, **k):
    partials.append(1)
    calls.append(1)
    return real_partial(self, *a, **k)

  monkeypatch.setattr(ops.PackedLinear, "__call__", counting)
  monkeypatch.setattr(ops.PackedLinear, "partial", counting_partial)
  with_rows = run()
  # per step: recurrent 2 x (2 + 2 MLP) + attention (3 + 2 MLP)
  assert len(calls) == 3 * 13, len(calls)
  # 6 of the 13 feed a norm next and are left as partial sums for it
  assert len(partials) == 3 * 6, len(partials)
  monkeypatch.setattr(ops.PackedLinear, "usable",
                      staticmethod(lambda *a, **k: False))
  library = run()
  assert len(calls) == 3 * 13
  scale = library.abs().max().item()
  assert (with_rows - library).abs().max().item() <= 0.03 * scale
