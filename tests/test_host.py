"""Host-side checks that need no GPU: the C-ABI library loads and exports what
include/rg_lru.h declares, argument validation happens before any launch, and
the drop-in modules keep the reference's surface (names, shapes, caches)."""

import ctypes
import os
import re

import pytest
import torch

import recurrentgemma_amd as rg
from oracle import torch_ref as R
from recurrentgemma_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
  text = open(os.path.join(ROOT, "include", "rg_lru.h")).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  return sorted(set(re.findall(r"\b(rg_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
  names = _declared_symbols()
  assert len(names) == 51, names
  lib = ctypes.CDLL(_lib.LIB_PATH)
  for n in names:
    assert hasattr(lib, n), n
  assert set(names) == set(_lib.SIGNATURES)
  assert _lib.lib().rg_abi_version() == 1


def test_c_side_validation_without_launch():
  lib = _lib.lib()
  ok = ctypes.c_void_p(256)  # aligned, never dereferenced: checks fail first
  rc = lib.rg_conv1d_prefill(None, ok, 1, ok, ok, ok, None, 1, 1, 8, 4, 0, None)
  assert rc == -1 and b"x is null" in lib.rg_last_error()
  rc = lib.rg_conv1d_prefill(ok, ok, 1, ok, ok, ok, None, 1, 1, 8, 1, 0, None)
  assert rc == -2 and b"temporal width" in lib.rg_last_error()
  rc = lib.rg_conv1d_prefill(ok, ok, 1, ok, ok, ok, None, 1, 0, 8, 4, 0, None)
  assert rc == -1 and b"positive" in lib.rg_last_error()
  rc = lib.rg_conv1d_prefill(ok, ok, 1, ok, ok, ok, None, 1, 1, 8, 4, 7, None)
  assert rc == -2 and b"dtype" in lib.rg_last_error()
  odd = ctypes.c_void_p(257)
  rc = lib.rg_gates_gemm(odd, 0, None, 0, None, None, ok, ok, ok, ok, ok, ok, 1,
                         1, 256, 1, 1, None)
  assert rc == -1 and b"aligned" in lib.rg_last_error()
  rc = lib.rg_gates_gemm(ok, 0, None, 0, None, None, ok, ok, ok, ok, ok, ok, 1,
                         1, 250, 3, 1, None)
  assert rc == -1 and b"multiple" in lib.rg_last_error()
  y = ctypes.c_void_p(512)
  rc = lib.rg_lru_scan_fused(ok, 0, None, None, ok, ok, ok, ok, 1, None, y,
                             None, ok, 1, 1, 8, 1, None)
  assert rc == -1 and b"apply_conv" in lib.rg_last_error()
  assert lib.rg_recurrent_step_workspace_bytes(256, 4096, 1) == 3 * 256 * 4096 * 2
  rc = lib.rg_recurrent_step(ok, ok, 1, ok, ok, ok, ok, ok, ok, ok, ok, ok, ok,
                             ok, ok, None, 0, 2, 256, 1, 1, None)
  assert rc == -4 and b"workspace" in lib.rg_last_error()
  # rows cut into chunks for the single-launch prefill kernel
  assert lib.rg_recurrent_prefill_split_workspace_bytes(16, 8192, 4096, 16) == 0
  assert lib.rg_recurrent_prefill_split_workspace_bytes(1, 320, 2560, 10) == 0  # < 6 tiles
  need = lib.rg_recurrent_prefill_split_workspace_bytes(1, 8192, 2560, 10)
  assert need > 0 and need % (2 * 2560 * 4) == 0
  rc = lib.rg_recurrent_prefill_split(ok, ok, 1, ok, ok, ok, ok, ok, ok, None,
                                      ok, None, y, None, None, None, 0, 1, 8192,
                                      2560, 10, 1, None)
  assert rc == -4 and b"workspace" in lib.rg_last_error()
  rc = lib.rg_recurrent_prefill_split(ok, ok, 1, ok, ok, ok, ok, ok, ok, None,
                                      ok, None, y, None, None, None, 0, 1, 8192,
                                      2560, 10, 0, None)
  assert rc == -2 and b"unsupported" in lib.rg_last_error()
  # the entries added for the whole block
  rc = lib.rg_gelu_mul(ok, ok, ok, 0, 1, None)
  assert rc == -1 and b"positive" in lib.rg_last_error()
  rc = lib.rg_gelu_mul(ok, odd, ok, 8, 1, None)
  assert rc == -1 and b"aligned" in lib.rg_last_error()
  rc = lib.rg_gelu_mul(ok, ok, None, 8, 1, None)
  assert rc == -1 and b"null" in lib.rg_last_error()
  rc = lib.rg_gelu_mul(ok, ok, ok, 8, 3, None)
  assert rc == -2 and b"dtype" in lib.rg_last_error()
  rc = lib.rg_add_rms_norm(ok, ok, ok, y, y, 4, 64, 1e-6, 1, None)
  assert rc == -1 and b"alias" in lib.rg_last_error()
  rc = lib.rg_add_rms_norm(ok, None, ok, ok, y, 4, 64, 1e-6, 1, None)
  assert rc == -1 and b"null" in lib.rg_last_error()
  # linear layers for few rows
  assert lib.rg_linear_packed_bytes(2560, 2560, 0) == 2560 * 2560 * 2
  assert lib.rg_linear_packed_bytes(2560, 2500, 0) == 0   # K % 64
  assert lib.rg_linear_packed_bytes(2576, 2560, 0) == 0   # N % 32
  assert lib.rg_linear_packed_bytes(2592, 2560, 1) == 0   # pairs: N % 64
  rc = lib.rg_linear_pack(ok, 0, 1, 0, y, 2576, 2560, None)
  assert rc == -2 and b"N=2576" in lib.rg_last_error()
  rc = lib.rg_linear_pack(ok, 2, 1, 0, y, 64, 64, None)
  assert rc == -1 and b"layout" in lib.rg_last_error()
  rc = lib.rg_linear_pack(ok, 0, 1, 0, ok, 64, 64, None)
  assert rc == -1 and b"alias" in lib.rg_last_error()
  assert lib.rg_linear_rows_workspace_bytes(64, 2560, 2560) == 0
  assert lib.rg_linear_rows_workspace_bytes(64, 7680, 2560) == 3 * 64 * 2560 * 4
  rc = lib.rg_linear_rows(ok, ok, None, None, y, None, 0, 65, 64, 64, 1, 0, None)
  assert rc == -2 and b"M <= 64" in lib.rg_last_error()
  rc = lib.rg_linear_rows(ok, ok, None, None, ok, None, 0, 4, 64, 64, 1, 0, None)
  assert rc == -1 and b"alias" in lib.rg_last_error()
  rc = lib.rg_linear_rows(ok, ok, None, ok, y, None, 0, 4, 64, 64, 1, 1, None)
  assert rc == -1 and b"gelu pairs" in lib.rg_last_error()
  rc = lib.rg_linear_rows(ok, ok, None, None, y, None, 0, 4, 64, 64, 3, 0, None)
  assert rc == -1 and b"groups" in lib.rg_last_error()
  rc = lib.rg_linear_rows(ok, ok, None, None, y, None, 0, 64, 7680, 2560, 1, 0,
                          None)
  assert rc == -4 and b"workspace" in lib.rg_last_error()
  # scans cut into chunks: only for few rows and long sequences
  # the backward entry points and the prompt attention check their arguments
  # before any launch
  rc = lib.rg_rglru_backward(ok, ok, ok, ok, ok, ok, ok, None, None, ok, ok, ok,
                             ok, None, 1, 4, 8, 0, None)
  assert rc == -1 and b"alias" in lib.rg_last_error()
  rc = lib.rg_rglru_backward(None, ok, ok, ok, ok, ok, ok, None, None, ok, ok,
                             ok, ok, None, 1, 4, 8, 0, None)
  assert rc == -1 and b"dy is null" in lib.rg_last_error()
  assert lib.rg_conv1d_backward_workspace_bytes(2, 100, 64, 4) == 7 * 5 * 64 * 4
  # chunks of 32 rows while that leaves at most 512 of them, then 64, 128, 256
  assert lib.rg_conv1d_backward_workspace_bytes(16, 1024, 64, 4) == 512 * 5 * 64 * 4
  assert lib.rg_conv1d_backward_workspace_bytes(16, 1025, 64, 4) == 257 * 5 * 64 * 4
  assert lib.rg_conv1d_backward_workspace_bytes(16, 8192, 64, 4) == 512 * 5 * 64 * 4
  assert lib.rg_conv1d_backward_workspace_bytes(32, 8192, 64, 4) == 1024 * 5 * 64 * 4
  assert lib.rg_conv1d_backward_workspace_bytes(2, 100, 64, 1) == 0
  rc = lib.rg_conv1d_backward(ok, ok, ok, 1, ok, ctypes.c_void_p(512), None, 0,
                              2, 100, 64, 4, 0, None)
  assert rc == -4 and b"partial sums" in lib.rg_last_error()
  rc = lib.rg_conv1d_backward(ok, ok, ok, 1, ok, ctypes.c_void_p(512), ok, 1 << 20,
                              2, 100, 64, 17, 0, None)
  assert rc == -2 and b"temporal width" in lib.rg_last_error()
  two = ctypes.c_void_p(512)
  rc = lib.rg_attention_prefill(ok, two, two, two, ctypes.c_void_p(768), 1, 100,
                                128, 2, 128, 1.0, 1, None)
  assert rc == -2 and b"head_dim == 256" in lib.rg_last_error()
  rc = lib.rg_attention_prefill(ok, two, two, two, ctypes.c_void_p(768), 1, 100,
                                96, 2, 256, 1.0, 1, None)
  assert rc == -1 and b"multiple of 64" in lib.rg_last_error()
  rc = lib.rg_attention_prefill(ok, two, two, two, ok, 1, 100, 128, 2, 256, 1.0,
                                1, None)
  assert rc == -1 and b"alias" in lib.rg_last_error()
  rc = lib.rg_recurrent_step_gelu_mul(ok, None, ok, 1, ok, ok, ok, ok, ok, ok,
                                      ok, ok, ok, ok, two, 4, 512, 2, 1, None)
  assert rc == -1 and b"gate_branch is null" in lib.rg_last_error()
  # one decoded token of the attention block: shapes, strides, workspace
  assert lib.rg_attention_decode_fused_workspace_bytes(64, 10, 2048) == (
      64 * 8 * 10 * 258 * 4)
  assert lib.rg_attention_decode_fused_workspace_bytes(2, 17, 2048) == 0
  assert lib.rg_attention_decode_fused_workspace_bytes(2, 10, 16385) == 0
  assert lib.rg_attention_decode_fused_workspace_bytes(2, 1, 300) == (
      2 * 2 * 1 * 258 * 4)

  def decode(ldq=3072, hd=256, dtype=1, ws=ok, ws_bytes=1 << 30, heads=10):
    return lib.rg_attention_decode_fused(
        ok, ldq, ok, 3072, ok, 3072, ok, 1, ok, ok, ok, ok, ok, ws, ws_bytes, 4,
        heads, hd, 2048, 0.0625, 1, dtype, None)

  assert decode(hd=128) == -2 and b"head_dim 256" in lib.rg_last_error()
  assert decode(dtype=0) == -2
  assert decode(heads=17) == -2
  assert decode(ldq=2559) == -1 and b"row strides" in lib.rg_last_error()
  assert decode(ldq=2564) == -1
  assert decode(ws=None) == -4 and b"workspace" in lib.rg_last_error()
  assert decode(ws_bytes=1000) == -4
  # rg_recurrent_core: nothing for whole rows in the single kernel, the chunk
  # summaries for rows in chunks, both gates' pre-activations (+ the scan's
  # chunk summaries) for the two-kernel form
  assert lib.rg_recurrent_core_workspace_bytes(16, 8192, 4096, 16, 1) == 0
  assert (lib.rg_recurrent_core_workspace_bytes(1, 8192, 2560, 10, 1) ==
          lib.rg_recurrent_prefill_split_workspace_bytes(1, 8192, 2560, 10))
  # float32 with 256-wide heads and at most 32 (row, head) pairs: one launch,
  # no workspace; more pairs or other head widths: the two-kernel form
  assert lib.rg_recurrent_core_workspace_bytes(1, 512, 2560, 10, 0) == 0
  assert lib.rg_recurrent_core_workspace_bytes(3, 512, 2560, 10, 0) == 0
  assert (lib.rg_recurrent_core_workspace_bytes(4, 512, 2560, 10, 0) ==
          2 * 4 * 512 * 2560 * 4 + lib.rg_scan_split_workspace_bytes(4, 512, 2560))
  assert (lib.rg_recurrent_core_workspace_bytes(1, 512, 2560, 20, 0) ==
          2 * 512 * 2560 * 4 + lib.rg_scan_split_workspace_bytes(1, 512, 2560))
  # bf16 with 256-wide heads: the single kernel whatever the number of rows ...
  assert lib.rg_recurrent_core_workspace_bytes(2, 100, 512, 2, 1) == 0
  # ... other head widths: the two-kernel form
  assert lib.rg_recurrent_core_workspace_bytes(2, 100, 512, 4, 1) == 2 * 2 * 100 * 512 * 2
  assert lib.rg_recurrent_core_workspace_bytes(2, 100, 512, 3, 1) == 0  # W % H
  # many very short rows: twice as many (row, head) pairs as CUs and a few
  # tokens each take the two-kernel form (both gates' pre-activations in the
  # workspace)
  assert lib.rg_recurrent_core_workspace_bytes(256, 1, 4096, 16, 1) == (
      2 * 256 * 4096 * 2)
  assert lib.rg_recurrent_core_workspace_bytes(256, 32, 4096, 16, 1) == (
      2 * 256 * 32 * 4096 * 2)
  assert lib.rg_recurrent_core_workspace_bytes(256, 33, 4096, 16, 1) == 0
  assert lib.rg_recurrent_core_workspace_bytes(32, 16, 4096, 16, 1) == 0
  assert lib.rg_recurrent_core_workspace_bytes(33, 16, 4096, 16, 1) == (
      2 * 33 * 16 * 4096 * 2)
  assert lib.rg_recurrent_core_workspace_bytes(256, 64, 4096, 16, 1) == 0
  # rows in chunks: from 512 tokens on for at most 128 pairs
  assert lib.rg_recurrent_prefill_split_workspace_bytes(1, 512, 2560, 10) > 0
  assert lib.rg_recurrent_prefill_split_workspace_bytes(1, 448, 2560, 10) == 0
  assert lib.rg_recurrent_prefill_split_workspace_bytes(12, 512, 2560, 10) == 0
  assert lib.rg_recurrent_prefill_split_workspace_bytes(12, 768, 2560, 10) > 0
  assert lib.rg_recurrent_prefill_split_workspace_bytes(13, 4096, 2560, 10) == 0
  rc = lib.rg_recurrent_core(ok, None, ok, 1, ok, ok, ok, ok, ok, ok, None, ok,
                             None, ok, None, None, None, 0, 2, 100, 512, 4, 1,
                             None)
  assert rc == -4 and b"rg_recurrent_core: workspace" in lib.rg_last_error()
  rc = lib.rg_recurrent_core(ok, ok, ok, 1, ok, ok, ok, ok, ok, ok, None, ok,
                             None, ok, None, None, None, 0, 16, 64, 4096, 16, 1,
                             None)
  assert rc == -1 and b"alias" in lib.rg_last_error()
  # without conv weights (the RG-LRU on its own): both or neither, and no
  # conv state to return
  rc = lib.rg_recurrent_core(ok, None, ok, 1, ok, None, ok, ok, ok, ok, None, ok,
                             None, y, None, None, None, 0, 16, 64, 4096, 16, 1,
                             None)
  assert rc == -1 and b"go together" in lib.rg_last_error()
  rc = lib.rg_recurrent_core(ok, None, ok, 1, None, None, ok, ok, ok, ok, None,
                             ok, None, y, None, y, None, 0, 16, 64, 4096, 16, 1,
                             None)
  assert rc == -1 and b"no conv state" in lib.rg_last_error()
  assert lib.rg_scan_split_workspace_bytes(16, 8192, 4096) == 0
  assert lib.rg_scan_split_workspace_bytes(1, 500, 2560) == 0
  assert lib.rg_scan_split_workspace_bytes(1, 8192, 2560) == 2 * 22 * 2560 * 4
  rc = lib.rg_lru_scan_fused_split(ok, 0, None, None, ok, ok, ok, ok, 1, None, y,
                                   None, None, None, 0, 1, 8192, 2560, 1, None)
  assert rc == -4 and b"rg_lru_scan_fused_split: workspace" in lib.rg_last_error()
  rc = lib.rg_linear_scan_split(ok, ok, ok, None, None, None, None, 0, 1, 8192,
                                2560, 1, None)
  assert rc == -1 and b"rg_linear_scan_split: y is null" in lib.rg_last_error()
  rc = lib.rg_linear_rows_partial(ok, ok, y, 64, 2560, 2560, 9, None)
  assert rc == -1 and b"slices" in lib.rg_last_error()
  rc = lib.rg_linear_rows_partial(ok, ok, y, 64, 2560, 2570, 3, None)
  assert rc == -2
  rc = lib.rg_add_rms_norm_partial(ok, 3, None, None, ok, y, y, 4, 64, 1e-6, 1,
                                   None)
  assert rc == -1 and b"alias" in lib.rg_last_error()
  rc = lib.rg_add_rms_norm_partial(ok, 3, None, None, ok, ok, y, 4, 64, 1e-6, 0,
                                   None)
  assert rc == -2 and b"bf16" in lib.rg_last_error()
  rc = lib.rg_add_rms_norm_partial(ok, 3, None, None, ok, ok, y, 4, 60, 1e-6, 1,
                                   None)
  assert rc == -2
  args = [ok, ok, 1, ok, ok, ok, ok, ok, ok, None, ok, None, y, None, None]
  rc = lib.rg_recurrent_prefill(*args, 1, 8, 256, 1, 0, None)
  assert rc == -2 and b"unsupported" in lib.rg_last_error().lower()  # fp32
  rc = lib.rg_recurrent_prefill(*args, 1, 8, 512, 1, 1, None)
  assert rc == -2  # head width 512
  rc = lib.rg_recurrent_prefill(*args, 1, 0, 256, 1, 1, None)
  assert rc == -1 and b"positive" in lib.rg_last_error()
  args[12] = ok  # y aliases x
  rc = lib.rg_recurrent_prefill(*args, 1, 8, 256, 1, 1, None)
  assert rc == -1 and b"alias" in lib.rg_last_error()
  assert lib.rg_packed_gate_weights_bytes(4096, 16, 1) == 2 * 4096 * 256 * 2
  assert lib.rg_packed_gate_weights_bytes(4096, 8, 1) == 0  # 512-wide heads


def test_prefill_kernel_keeps_its_hand_numbered_registers():
  """The prefill kernel's gate weights sit in accumulation registers that the
  source numbers itself; the compiled kernels may touch those registers only
  in the hand-written instructions, and may not spill."""
  import shutil
  import subprocess
  if shutil.which("make") is None or not os.path.exists("/opt/rocm/bin/hipcc"):
    pytest.skip("needs make and hipcc")
  subprocess.check_call(["make", "-C", _lib.CSRC, "check-registers"],
                        stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)


def test_build_check_for_early_reads_of_matrix_results(tmp_path):
  """check_mfma_wait.py (part of `make check-registers`): an instruction that
  touches the result registers of a matrix instruction right behind it is
  reported; the same instruction behind the kernel's own wait, a matrix
  instruction that accumulates into the same registers, and instructions on
  other registers are not."""
  import subprocess
  import sys
  script = os.path.join(_lib.CSRC, "check_mfma_wait.py")
  mfma = ("\tv_mfma_f32_16x16x4_f32 v[2:5], v17, a[63], v[2:5]\n"
          "\tv_mfma_f32_16x16x4_f32 v[6:9], v17, a[0x7f], v[6:9]\n")
  wait = "\ts_nop 15\n\ts_nop 3\n"
  cases = {
      "copy_before_wait": (mfma + "\ts_nop 0\n\tv_mov_b64_e32 v[16:17], v[8:9]\n"
                           + wait, 1),
      "copy_after_wait": (mfma + wait + "\tv_mov_b64_e32 v[16:17], v[8:9]\n", 0),
      "other_registers": (mfma + "\tv_mul_f32_e32 v10, v11, v12\n"
                          "\tds_read_b128 v[18:21], v83\n" + wait, 0),
      "accumulating": (mfma + mfma + wait, 0),
      "store_of_result": ("\tv_mfma_f32_32x32x16_bf16 v[2:17], v[100:103], "
                          "a[31*4:31*4+3], v[2:17]\n"
                          "\tds_write_b32 v40, v17\n" + wait, 1),
      "far_enough": (mfma + "\ts_mov_b32 s0, s1\n" * 24
                     + "\tv_mov_b32_e32 v20, v9\n", 0),
  }
  for name, (text, want) in cases.items():
    path = tmp_path / (name + ".s")
    path.write_text(text)
    rc = subprocess.run([sys.executable, script, str(path)],
                        stdout=subprocess.DEVNULL).returncode
    assert rc == want, name


def test_bench_refuses_more_than_one_gpu():
  """bench.py measures one GPU; any other --gpus ends with a message, not a
  number."""
  import subprocess
  import sys
  root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
  r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus",
                      "2"], capture_output=True, text=True)
  assert r.returncode != 0
  assert "one GPU" in (r.stderr + r.stdout)
  assert "{" not in r.stdout


def test_no_cpu_fallback():
  conv = rg.Conv1D(width=8, temporal_width=4)
  with pytest.raises(RuntimeError, match="GPU only"):
    conv(torch.randn(1, 5, 8), torch.arange(5)[None])
  lru = rg.RGLRU(width=8, num_heads=2)
  with pytest.raises(RuntimeError, match="GPU only"):
    lru(torch.randn(1, 5, 8), torch.arange(5)[None])
  with pytest.raises(AssertionError):
    lru(torch.randn(1, 5, 8), torch.arange(4)[None])  # layers.py:334
  with pytest.raises(AssertionError):
    conv(torch.randn(1, 2, 8), torch.arange(2)[None],
         cache=torch.zeros(1, 3, 8))  # layers.py:549: one token with a cache
  with pytest.raises(AssertionError):
    rg.rnn_scan(torch.zeros(1, 2, 4), torch.zeros(1, 2, 4, dtype=torch.bfloat16),
                torch.zeros(1, 2, dtype=torch.bool), None)  # layers.py:163


def test_missing_library_fails_loudly(monkeypatch):
  monkeypatch.setattr(_lib, "_lib", None)
  monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/librg_lru.so")
  with pytest.raises(RuntimeError, match="no fallback"):
    _lib.lib()


def test_module_surface_matches_reference():
  blk = rg.RecurrentBlock(width=64, num_heads=4, lru_width=128)
  # recurrentgemma/torch/modules.py:549-580, layers.py:105-112,262-278,409-412
  want = {
      "linear_y.weight": (128, 64), "linear_y.bias": (128,),
      "linear_x.weight": (128, 64), "linear_x.bias": (128,),
      "linear_out.weight": (64, 128), "linear_out.bias": (64,),
      "conv_1d.w": (4, 128), "conv_1d.b": (128,),
      "rg_lru.a_param": (128,),
      "rg_lru.input_gate.w": (4, 32, 32), "rg_lru.input_gate.b": (4, 32),
      "rg_lru.a_gate.w": (4, 32, 32), "rg_lru.a_gate.b": (4, 32),
  }
  got = {k: tuple(v.shape) for k, v in blk.state_dict().items()}
  assert got == want
  assert rg.RecurrentBlockCache._fields == ("rg_lru_state", "conv1d_state")
  c = rg.RecurrentBlock.init_cache(batch_size=3, lru_width=128,
                                   dtype=torch.bfloat16)
  assert c.rg_lru_state.dtype == torch.float32
  assert c.rg_lru_state.shape == (3, 128)
  assert c.conv1d_state.dtype == torch.bfloat16
  assert c.conv1d_state.shape == (3, 3, 128)
  assert rg.Conv1D.init_cache(batch_size=2, width=8, dtype=torch.float32,
                              conv1d_temporal_width=8).shape == (2, 7, 8)
  assert rg.RGLRU.init_cache(2, 8).dtype == torch.float32
  # initial distributions (layers.py:122-125, 422-425, 289-291)
  torch.manual_seed(0)
  big = rg.RGLRU(width=4096, num_heads=16)
  assert abs(big.input_gate.w.std().item() - 1 / 16) < 1e-3
  assert torch.all(big.input_gate.b == 0)
  r = torch.exp(-torch.nn.functional.softplus(big.a_param.double()))
  assert r.min() >= 0.9 - 1e-4 and r.max() <= 0.999 + 1e-4
  conv = rg.Conv1D(width=4096, temporal_width=4)
  assert abs(conv.w.std().item() - 0.05) < 2e-3


def test_param_init_same_draws_as_oracle():
  torch.manual_seed(7)
  a = torch.empty(100)
  rg.rnn_param_init(a, 0.9, 0.999)
  torch.manual_seed(7)
  b = torch.empty(100)
  R.rnn_param_init(b, 0.9, 0.999)
  assert torch.equal(a, b)


def test_custom_operators_have_shape_functions():
  """The traced form of the hot path (recurrentgemma_amd/compiled.py): both
  operators are registered and infer their outputs' shapes and dtypes from
  fake tensors, without touching a GPU."""
  from torch._subclasses.fake_tensor import FakeTensorMode
  from recurrentgemma_amd import compiled  # noqa: F401 (registers the ops)
  with FakeTensorMode():
    B, T, W, H = 3, 7, 512, 2
    x = torch.empty(B, T, W, dtype=torch.bfloat16)
    seg = torch.empty(B, T, dtype=torch.int64)
    cw = torch.empty(4, W, dtype=torch.bfloat16)
    cb = torch.empty(W, dtype=torch.bfloat16)
    w = torch.empty(H, W // H, W // H, dtype=torch.bfloat16)
    b = torch.empty(H, W // H, dtype=torch.bfloat16)
    y, h, c = torch.ops.recurrentgemma_amd.recurrent_core(
        x, seg, cw, cb, w, b, w, b, cb, None, x)
    assert y.shape == (B, T, W) and y.dtype == torch.bfloat16
    assert h.shape == (B, W) and h.dtype == torch.float32
    assert c.shape == (B, 3, W) and c.dtype == torch.bfloat16
    x1 = torch.empty(B, 1, W, dtype=torch.bfloat16)
    y1, h1, c1 = torch.ops.recurrentgemma_amd.recurrent_step(
        x1, seg[:, :1], c, h, cw, cb, w, b, w, b, cb, None)
    assert y1.shape == (B, 1, W) and h1.shape == (B, W) and c1.shape == (B, 3, W)
