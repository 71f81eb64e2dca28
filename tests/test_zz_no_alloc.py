"""rg_recurrent_step_static: the decode step for callers that cannot allocate.

It exchanges the conv output and the gate pre-activations of a step through a
buffer inside the library's code object instead of a caller-supplied
workspace.  Checked through the C ABI against rg_recurrent_step (bit for bit:
the same three kernels on the same inputs), on two calls in a row, the second
with a smaller input.  Collected last (file name), so that a failure here does
not hide the other GPU tests under `pytest -x`.
"""

import pytest
import torch

from oracle import torch_ref as R
from recurrentgemma_amd import _lib

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _ptr(t):
  return None if t is None else t.data_ptr()


def _step(lib, static, P, x, seg, cc, h, B, W, H, code):
  """One step through the C ABI; returns (y, h_out, cache_out)."""
  y = torch.empty_like(x)
  h_out, cc_out = torch.empty_like(h), torch.empty_like(cc)
  stream = torch.cuda.current_stream().cuda_stream
  head = [_ptr(x), _ptr(seg), 1, _ptr(cc), _ptr(cc_out), _ptr(h), _ptr(h_out),
          _ptr(P["conv_w"]), _ptr(P["conv_b"]), _ptr(P["w_x"]), _ptr(P["b_x"]),
          _ptr(P["w_a"]), _ptr(P["b_a"]), _ptr(P["a_param"]), _ptr(y)]
  if static:
    _lib.check(lib.rg_recurrent_step_static(*head, B, W, H, code, stream))
  else:
    ws = torch.empty(lib.rg_recurrent_step_workspace_bytes(B, W, code),
                     dtype=torch.uint8, device=DEV)
    _lib.check(lib.rg_recurrent_step(*head, _ptr(ws), ws.numel(), B, W, H, code,
                                     stream))
  return y, h_out, cc_out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_static_scratch_step_equals_workspace_step(dtype):
  lib = _lib.lib()
  code = 0 if dtype == torch.float32 else 1
  W, H = 512, 4  # 128-wide heads: the three-launch form in both dtypes
  p = R.make_params(W, H, dtype, seed=4242, gate_bias_std=0.5)
  P = {k: v.to(DEV) for k, v in p.items()}
  g = torch.Generator().manual_seed(4243)
  # two calls in a row, the second smaller: stale scratch of the first call
  # beyond the second one's extent must not matter
  for B in (37, 5):
    print("[case] static scratch step", dtype, B, flush=True)
    x = torch.randn(B, 1, W, generator=g).to(dtype).to(DEV)
    cc = torch.randn(B, 3, W, generator=g).to(dtype).to(DEV)
    h = torch.randn(B, W, generator=g).to(DEV)
    seg = torch.full((B, 1), 9, dtype=torch.int64)
    seg[B // 2, 0] = 0  # one row starts a document
    seg = seg.to(DEV)
    got = _step(lib, True, P, x, seg, cc, h, B, W, H, code)
    want = _step(lib, False, P, x, seg, cc, h, B, W, H, code)
    torch.cuda.synchronize()
    for a, b, name in zip(got, want, ("y", "h", "conv state")):
      assert torch.equal(a, b), (name, B)
    # and the oracle, to the bars of the other decode tests
    ref = (R.recurrent_core if dtype == torch.float32
           else R.widened_recurrent_core)
    cache = R.CoreCache(rg_lru_state=h.cpu(), conv1d_state=cc.cpu())
    yo, co = ref(x.cpu(), seg.cpu(), p, cache)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    err = ((got[0].double().cpu() - yo.double()).abs().max() /
           yo.double().abs().max()).item()
    assert err < tol, err
    assert torch.equal(got[2].cpu(), co.conv1d_state)


def test_static_scratch_step_rejects_large_shapes():
  lib = _lib.lib()
  ok = 256  # aligned, never dereferenced: the size check comes first
  B, W = 4096, 4096
  assert (lib.rg_recurrent_step_workspace_bytes(B, W, 0) >
          _lib.RG_STEP_STATIC_SCRATCH_BYTES)
  rc = lib.rg_recurrent_step_static(ok, ok, 1, ok, ok, ok, ok, ok, ok, ok, ok,
                                    ok, ok, ok, ok, B, W, 16, 0, None)
  assert rc == -4 and b"built-in buffer" in lib.rg_last_error()
