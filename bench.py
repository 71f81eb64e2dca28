"""Benchmark of the Conv1D + RG-LRU recurrent-block core on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A "step" is one pass of the hot path (Conv1D -> RG-LRU of the recurrent block)
over one synthetic batch that is already resident in HBM, called through the C
ABI on torch's current stream.  Two forms of the path exist (--path):
  single  rg_recurrent_prefill: conv, gate projections (bf16 MFMA), gate
          arithmetic and recurrence in ONE kernel, nothing but x and y moves
          through HBM.  Default where one workgroup per row and head fills the
          GPU, and where rows are long enough to be cut into time chunks that
          do (rg_recurrent_prefill_split: a summary pass, a carry pass and a
          replay pass, x read twice)
  split   rg_gates_gemm (conv on load, both gate projections on bf16 MFMA)
          followed by rg_lru_scan_fused (conv + gates + chunked scan); the gate
          pre-activations go through HBM
Prints ONE JSON line.

Workloads (the benchmark configurations this build is measured on):
  9b_prefill  B16 T8192 W4096 H16 bf16 / fp32 state, one document per row
              (the configuration the >= 70 % HBM-roofline target is stated on;
              default)
  2b_prefill  B8 T4096 W2560 H10 bf16, documents ~ Geometric(mean 1024)
  2b_f32      B1 T512 W2560 H10 fp32 (the reference's own CPU-runnable case;
              21 MB, i.e. cache resident: warm-cache figures)
  2b_attention_prompt  prompt-pass attention of one local-attention block of
              the 2B model (B64 T2047, 10 query heads, head_dim 256)
  2b_attention_decode  one decoded token of that block against a full ring
              cache (B64, window 2048): rg_attention_decode_fused, with the
              separate calls it replaces timed after it
  9b_modules  the drop-in modules called one by one at the 9b_prefill shape:
              Conv1D, BlockDiagonalLinear (one gate), RGLRU, each with its own
              algorithmic bytes and HBM fraction
  2b_block_training  RecurrentBlock forward + backward under
              training.differentiable() (B4 T2048 W2560 H10 bf16), with the
              backward kernels of the recurrent path timed by themselves
  9b_decode   B256 W4096 H16 bf16, one token per row and step with the caches
              carried in place (rg_recurrent_step); `roofline` then describes
              the whole step (all its launches) against its algorithmic bytes

`roofline` describes the dominant kernel of the timed path: its algorithmic
bytes per launch (single: read x, write y; split: the scan kernel's read x,
read both gate pre-activations, write y; plus the small terms) over the mean
launch duration measured with HIP events inside the timed region.  With the
default path the JSON also carries `two_kernel_path`, the split form measured
after the timed region (scan-kernel roofline and gate GEMM figures).
`cpu_baseline` times the CPU oracle (an op-for-op torch restatement of the
reference's path, bf16 like the reference would run it) on a bounded sample of
the same workload on this machine's host cores.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

WORKLOADS = {
    "9b_prefill": dict(B=16, T=8192, W=4096, H=16, mean_doc=None, seed=1003),
    "2b_prefill": dict(B=8, T=4096, W=2560, H=10, mean_doc=1024, seed=1002),
    "2b_f32": dict(B=1, T=512, W=2560, H=10, mean_doc=None, seed=1001,
                   dtype="f32"),
    "9b_decode": dict(B=256, T=1, W=4096, H=16, mean_doc=None, seed=1004,
                      decode=True),
    # one long prompt: 10 (row, channel slab) pairs, the scan runs its
    # sequence as chunks side by side
    "2b_single_prompt": dict(B=1, T=8192, W=2560, H=10, mean_doc=None,
                             seed=1006),
    # random-init 2B residual stack, greedy decoding: 64 prompts of 2048 random
    # token ids, 256 new tokens each (--steps sets the number of new tokens)
    "2b_griffin_decode": dict(B=64, T=2048, new_tokens=256, seed=1005,
                              griffin=True),
    # prompt-pass attention of one local-attention block of that model: 64
    # prompts of 2047 tokens (what the sampler's prompt pass sees), 10 query
    # heads on one key/value head, head_dim 256, window 2048
    "2b_attention_prompt": dict(B=64, T=2047, H=10, window=2048, seed=1007,
                                attention=True),
    # the differentiable path: one block, forward and backward
    "2b_block_training": dict(B=4, T=2048, W=2560, H=10, mean_doc=512,
                              seed=1010, training=True),
    # the modules of the path called stand-alone, one after the other
    "9b_modules": dict(B=16, T=8192, W=4096, H=16, mean_doc=None, seed=1009,
                       modules=True),
    # ... and one decoded token of it: every ring slot written
    "2b_attention_decode": dict(B=64, H=10, window=2048, seed=1008,
                                attention_step=True),
}

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs (scaled
# by a copy kernel of known size).  These are constants taken from the named
# summary file, not something a bench run measures: the JSON says so in
# `traffic_source`.  No entry = not measured for that workload (traffic null).
MEASURED_TRAFFIC_BYTES = {
    ("9b_prefill", "single"): (2.162e9, "profiles/hbm_traffic_9b_prefill.txt"),
    ("9b_prefill", "scan"): (4.345e9, "profiles/hbm_traffic_9b_prefill.txt"),
    ("2b_prefill", "single"): (0.474e9, "profiles/hbm_traffic_2b_prefill.txt"),
    ("2b_prefill", "scan"): (0.681e9, "profiles/hbm_traffic_2b_prefill.txt"),
}


def measured_traffic(workload, kernel):
  """(bytes, source) of the committed counter summary for a kernel, or
  (None, None)."""
  return MEASURED_TRAFFIC_BYTES.get((workload, kernel), (None, None))


METRIC = ("RG-LRU block tokens/s + scan HBM GB/s (% of roofline) at 2B and 9B "
          "widths")


def single_algorithmic_bytes(B, T, W, H, esize, seg_bytes, has_h0):
  n = B * T * W
  return (2 * esize * n            # x in, y out
          + B * T * seg_bytes      # segment positions
          + B * W * 4 * (int(has_h0) + 1)   # h0 in, h_last out (fp32)
          + B * 3 * W * esize      # conv state out
          + 2 * H * (W // H) ** 2 * esize   # both gate weight matrices
          + W * esize * 8)         # conv w (4), conv b, a_param, gate biases


def scan_algorithmic_bytes(B, T, W, esize, seg_bytes, has_h0):
  n = B * T * W
  return (4 * esize * n            # x, gx_pre, ga_pre in; y out
          + B * T * seg_bytes      # segment positions
          + B * W * 4 * (int(has_h0) + 1)   # h0 in, h_last out (fp32)
          + B * 3 * W * esize      # conv state out
          + W * esize * 8)         # conv w (4), conv b, a_param (+ gate biases)


def make_segment_pos(torch, B, T, mean_doc, seed):
  if mean_doc is None:
    return torch.arange(T).expand(B, T).contiguous()
  import numpy as np
  rng = np.random.default_rng(seed)
  out = np.zeros((B, T), np.int64)
  for b in range(B):
    t = 0
    while t < T:
      n = min(int(rng.geometric(1.0 / mean_doc)), T - t)
      out[b, t:t + n] = np.arange(n)
      t += n
  return torch.from_numpy(out)


def host_cores():
  """Threads for the CPU leg: the cores this process may use (an
  OMP_NUM_THREADS set by the environment is the share it was given)."""
  n = os.cpu_count() or 1
  try:
    n = min(n, len(os.sched_getaffinity(0)))
  except (AttributeError, OSError):
    pass
  env = os.environ.get("OMP_NUM_THREADS", "")
  if env.isdigit() and int(env) > 0:
    n = min(n, int(env))
  return n


def cpu_model():
  try:
    with open("/proc/cpuinfo") as f:
      for line in f:
        if line.startswith("model name"):
          return line.split(":", 1)[1].strip()
  except OSError:
    pass
  return "unknown"


def cpu_baseline(torch, R, wl, params, seconds_target=20.0):
  """Oracle (port of the reference torch path) on the host cores, on a slice
  of the workload: the first Bs batch rows at full sequence length (about
  10-30 s of CPU work in total)."""
  cores = host_cores()
  torch.set_num_threads(cores)
  Bs, Ts = min(wl["B"], 4), wl["T"]
  g = torch.Generator().manual_seed(wl["seed"])
  dt = torch.float32 if wl.get("dtype") == "f32" else torch.bfloat16
  x = torch.randn(Bs, Ts, wl["W"], generator=g).to(dt)
  seg = make_segment_pos(torch, Bs, Ts, wl["mean_doc"], wl["seed"])
  R.recurrent_core(x[:, :64], seg[:, :64], params)  # warm-up
  times = []
  t_all = time.perf_counter()
  while len(times) < 3 and (not times or
                            time.perf_counter() - t_all < seconds_target):
    t0 = time.perf_counter()
    R.recurrent_core(x, seg, params)
    times.append(time.perf_counter() - t0)
  best = sorted(times)[len(times) // 2]
  return {
      "value": Bs * Ts / best, "unit": "tokens/s", "cores": cores,
      "kind": "port", "cpu": cpu_model(),
      "sample": (f"oracle/torch_ref.recurrent_core, "
                 f"{'f32' if dt == torch.float32 else 'bf16'}, {Bs}x{Ts} tokens of "
                 f"the workload (W={wl['W']}, H={wl['H']}), median of "
                 f"{len(times)} runs, torch threads={torch.get_num_threads()}"),
  }


def shader_clock_ghz(torch, iters=2000):
  """Shader clock right now, from rg_clock_probe: one light wave per compute
  unit for about 0.2 ms, shader-clock cycles over the constant 100 MHz
  counter.  A light probe: under the matrix-instruction load of the prefill
  kernel the clock sits lower than what this reads."""
  import ctypes
  from recurrentgemma_amd import _lib
  out = torch.zeros(3, dtype=torch.int64, device="cuda:0")
  rc = _lib.lib().rg_clock_probe(
      ctypes.c_void_p(out.data_ptr()), iters,
      ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
  if rc != 0:
    return None
  torch.cuda.synchronize()
  cycles, ticks = (int(v) for v in out[:2].cpu())
  return cycles / (ticks * 10.0) if ticks > 0 else None


def prefill_clock_under_load(torch, fn):
  """Shader clock while the single prefill kernel runs, from the counters its
  workgroup (0, 0) keeps around its tile loop (rg_prefill_clock_probe): one
  extra launch of fn() after the timed region.  None if fn() did not take that
  kernel."""
  import ctypes
  from recurrentgemma_amd import _lib
  lib = _lib.lib()
  out = torch.zeros(2, dtype=torch.int64, device="cuda:0")
  torch.cuda.synchronize()
  lib.rg_prefill_clock_probe(ctypes.c_void_p(out.data_ptr()))
  try:
    fn()
    torch.cuda.synchronize()
  finally:
    lib.rg_prefill_clock_probe(None)
  cycles, ticks = (int(v) for v in out.cpu())
  return cycles / (ticks * 10.0) if ticks > 0 else None


def settle(torch, fn, cap_s=0.5, window=10, rel=0.01, min_launches=30):
  """Untimed launches of fn() until the GPU has left its idle clocks: stops
  when the median duration of the last `window` launches is within `rel` of
  the median of the `window` before them (at least `min_launches`), or after
  cap_s seconds.  A launch right after start-up runs up to 20 % longer than
  the sustained ones (clock ramp), for some tens of launches.  Returns the
  number of launches made."""
  e0 = torch.cuda.Event(enable_timing=True)
  e1 = torch.cuda.Event(enable_timing=True)
  ms = []
  t0 = time.perf_counter()
  med = lambda v: sorted(v)[len(v) // 2]
  while time.perf_counter() - t0 < cap_s:
    e0.record()
    fn()
    e1.record()
    e1.synchronize()
    ms.append(e0.elapsed_time(e1))
    if len(ms) >= max(min_launches, 2 * window) and len(ms) % window == 0:
      a, b = med(ms[-2 * window:-window]), med(ms[-window:])
      if abs(a - b) <= rel * b:
        break
  return len(ms)


def launch_stats(ms_list):
  v = sorted(ms_list)
  return {"min": v[0], "median": v[len(v) // 2], "max": v[-1]}


def decode_algorithmic_bytes(B, W, H, esize):
  """One decode step: x in, y out, fp32 state and conv state read and written,
  both gate weight matrices, the per-channel parameters."""
  return (2 * B * W * esize + 2 * B * W * 4 + 2 * B * 3 * W * esize
          + 2 * H * (W // H) ** 2 * esize + W * esize * 8 + B * 8)


def run_attention(args, torch, ops, wl):
  """rg_attention_prefill on one block's prompt pass (the transposed copy of
  the values included in a step), with the library attention (torch SDPA,
  causal) timed after it for comparison.  Flops counted: the visible
  (query, key) pairs only, 4 * head_dim each."""
  dev = torch.device("cuda:0")
  B, T, H, hd, window = wl["B"], wl["T"], wl["H"], 256, wl["window"]
  g = torch.Generator().manual_seed(wl["seed"])
  q = torch.randn(B, T, H, hd, generator=g).to(torch.bfloat16).to(dev)
  k = torch.randn(B, T, 1, hd, generator=g).to(torch.bfloat16).to(dev)
  v = torch.randn(B, T, 1, hd, generator=g).to(torch.bfloat16).to(dev)
  pos = torch.arange(T, device=dev)[None].expand(B, T)
  first = torch.clamp(pos - window, min=0).to(torch.int32).contiguous()
  pairs = float((pos - first + 1).sum().item()) * H
  flops = 4.0 * hd * pairs

  def timed(fn, steps, warmup):
    for _ in range(warmup):
      fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
      fn()
    e1.record()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps, e0.elapsed_time(e1) / steps

  wall, ms = timed(lambda: ops.attention_prefill(q, k, v, first, hd ** -0.5),
                   args.steps, args.warmup)

  def library():
    return torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2).expand(-1, H, -1, -1),
        v.transpose(1, 2).expand(-1, H, -1, -1), is_causal=True)
  _, lib_ms = timed(library, max(3, args.steps // 5), 2)
  achieved = flops / (ms * 1e-3) / 1e12
  print(json.dumps({
      "metric": "prompt-pass attention of one local-attention block, tokens/s",
      "value": B * T / wall, "unit": "tokens/s", "n_gpus": 1,
      "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall * 1e3,
      "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
      "dtype": "bf16", "data": "synthetic",
      "config": {"workload": args.workload, "batch": B, "seq_len": T,
                 "query_heads": H, "kv_heads": 1, "head_dim": hd,
                 "window": window,
                 "path": "rg_attention_prefill (+ the transposed copy of v)"},
      "roofline": {"kernel": "attn_prefill_bf16_kernel", "bound": "mfma",
                   "achieved": achieved, "peak": 2500.0, "unit": "TFLOP/s",
                   "frac": achieved / 2500.0, "traffic": None,
                   "algorithmic_flops": flops, "avg_launch_ms": ms},
      "library_attention": {"what": "torch SDPA, is_causal", "ms": lib_ms}}))


def run_training(args, torch, rg, ops, wl):
  """RecurrentBlock.forward and the backward pass through it inside
  training.differentiable(): conv, gate projections (bf16), RG-LRU gating and
  recurrence on kernels in both directions, the block's three linear layers
  as torch autograd.  A step = forward + loss + backward.  The backward
  kernels of the recurrent path are then timed alone on the same shapes."""
  from recurrentgemma_amd import training
  dev = torch.device("cuda:0")
  B, T, W, H = wl["B"], wl["T"], wl["W"], wl["H"]
  dtype = torch.bfloat16
  torch.manual_seed(wl["seed"])
  blk = rg.RecurrentBlock(width=W, num_heads=H, dtype=dtype).to(dev)
  g = torch.Generator().manual_seed(wl["seed"])
  x = torch.randn(B, T, W, generator=g).to(dtype).to(dev).requires_grad_(True)
  seg = make_segment_pos(torch, B, T, wl["mean_doc"], wl["seed"]).to(dev)

  def step():
    for p in blk.parameters():
      p.grad = None
    x.grad = None
    with training.differentiable():
      y, _ = blk(x, seg, return_cache=False)
      y.float().square().mean().backward()

  for _ in range(args.warmup):
    step()
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  for _ in range(args.steps):
    step()
  torch.cuda.synchronize()
  wall = (time.perf_counter() - t0) / args.steps
  with torch.no_grad():
    for _ in range(3):
      blk(x, seg, return_cache=False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
      blk(x, seg, return_cache=False)
    torch.cuda.synchronize()
    forward_only = (time.perf_counter() - t0) / args.steps

  def events(fn, steps=20, warmup=3):
    for _ in range(warmup):
      fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
      fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps

  n = B * T * W
  xc = torch.randn(B, T, W, generator=g).to(dtype).to(dev)
  gx = torch.randn(B, T, W, generator=g).to(dtype).to(dev)
  ga = torch.randn(B, T, W, generator=g).to(dtype).to(dev)
  dy = torch.randn(B, T, W, generator=g).to(dtype).to(dev)
  lru, conv = blk.rg_lru, blk.conv_1d
  with torch.no_grad():
    y, _, _ = ops.lru_scan_fused(xc, gx, ga, lru.a_param, seg)
    reset = seg == 0
    a = torch.rand(B, T, W, generator=g).to(dtype).to(dev)
    kernels = []
    for name, fn, per_element in (
        ("rg_rglru_backward", lambda: ops.rglru_backward(
            dy, xc, gx, ga, lru.a_param, reset, y, None, None), 8),
        ("rg_linear_scan_backward", lambda: ops.linear_scan_backward(
            dy, a, reset, y, None, None), 5),
        ("rg_conv1d_backward (+ the sum of its per-chunk planes)",
         lambda: ops.conv1d_backward(dy, xc, seg, conv.w), 3),
        ("rg_gates_gemm (forward of both gate projections)",
         lambda: ops.gates_gemm(xc, lru.input_gate.w, lru.input_gate.b,
                                lru.a_gate.w, lru.a_gate.b), 3),
        ("rg_gates_weight_grads (weight and bias gradients of both gate "
         "projections)",
         lambda: ops.gates_weight_grads(xc, dy, dy, lru.input_gate.w.shape[0]),
         3),
        ("rg_lru_scan_fused (forward of gating and recurrence)",
         lambda: ops.lru_scan_fused(xc, gx, ga, lru.a_param, seg), 4),
        ("rg_gelu_mul (the block's x * gelu(y) join)",
         lambda: ops.gelu_mul(xc, gx), 3),
        ("rg_gelu_mul_backward", lambda: ops.gelu_mul_backward(dy, xc, gx),
         5)):
      ms = events(fn)
      nbytes = per_element * n * 2
      gbs = nbytes / (ms * 1e-3) / 1e9
      kernels.append({"call": name, "ms": ms, "algorithmic_bytes": nbytes,
                      "achieved_gbs": gbs, "frac_of_hbm_peak": gbs / 8000.0})
  main = kernels[0]
  print(json.dumps({
      "metric": "RecurrentBlock forward + backward, tokens/s",
      "value": B * T / wall, "unit": "tokens/s", "n_gpus": 1,
      "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall * 1e3,
      "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
      "dtype": "bf16", "data": "synthetic",
      "config": {"workload": args.workload, "batch": B, "seq_len": T,
                 "width": W, "lru_width": W, "heads": H,
                 "documents": "geometric mean %d" % wl["mean_doc"],
                 "path": "training.differentiable(): kernels for conv, gate "
                         "projections, RG-LRU and the gelu join in both "
                         "directions; linear layers torch autograd"},
      "forward_only_ms": forward_only * 1e3,
      "roofline": {"kernel": "rglru_backward_kernel (rg_rglru_backward)",
                   "bound": "hbm", "achieved": main["achieved_gbs"],
                   "peak": 8000.0, "unit": "GB/s",
                   "frac": main["frac_of_hbm_peak"], "traffic": None,
                   "algorithmic_bytes": main["algorithmic_bytes"],
                   "avg_launch_ms": main["ms"]},
      "kernels": kernels}))


def run_modules(args, torch, rg, R, wl):
  """Conv1D.forward, BlockDiagonalLinear.forward and RGLRU.forward as a caller
  of the stand-alone modules runs them (recurrentgemma/torch/layers.py:
  447-529, 127-137, 313-365), one after the other on the same input shape.  A
  step = the three calls; each module is also timed by itself with HIP
  events."""
  dev = torch.device("cuda:0")
  B, T, W, H = wl["B"], wl["T"], wl["W"], wl["H"]
  dtype = torch.bfloat16
  params = R.make_params(W, H, dtype, seed=wl["seed"] + 100)
  conv = rg.Conv1D(W, 4, dtype=dtype)
  conv.load_state_dict({"w": params["conv_w"], "b": params["conv_b"]})
  lru = rg.RGLRU(W, H, dtype=dtype)
  lru.load_state_dict({"a_param": params["a_param"],
                       "input_gate.w": params["w_x"],
                       "input_gate.b": params["b_x"],
                       "a_gate.w": params["w_a"], "a_gate.b": params["b_a"]})
  conv, lru = conv.to(dev), lru.to(dev)
  g = torch.Generator().manual_seed(wl["seed"])
  x = torch.randn(B, T, W, generator=g).to(dtype).to(dev)
  seg = make_segment_pos(torch, B, T, wl["mean_doc"], wl["seed"]).to(dev)
  n = B * T * W
  calls = [
      ("Conv1D.forward", "conv1d_prefill_k4_kernel (rg_conv1d_prefill)",
       lambda: conv(x, seg), 2 * n * 2),
      ("BlockDiagonalLinear.forward",
       "gates_mfma_bf16_kernel, one matrix (rg_block_diag_linear)",
       lambda: lru.input_gate(x), 2 * n * 2),
      ("RGLRU.forward",
       "block_prefill_teams_bf16_kernel without conv weights (rg_recurrent_core)",
       lambda: lru(x, seg), 2 * n * 2),
  ]

  def events(fn, steps, warmup):
    for _ in range(warmup):
      fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
      fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps

  def step():
    for _, _, fn, _ in calls:
      fn()

  for _ in range(args.warmup):
    step()
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  for _ in range(args.steps):
    step()
  torch.cuda.synchronize()
  wall = (time.perf_counter() - t0) / args.steps
  modules = []
  for name, kernel, fn, nbytes in calls:
    ms = events(fn, max(5, args.steps // 2), 3)
    gbs = nbytes / (ms * 1e-3) / 1e9
    modules.append({"module": name, "kernel": kernel, "ms": ms,
                    "algorithmic_bytes": nbytes, "achieved_gbs": gbs,
                    "frac_of_hbm_peak": gbs / 8000.0})
  worst = max(modules, key=lambda m: m["ms"])
  print(json.dumps({
      "metric": "stand-alone Conv1D + BlockDiagonalLinear + RGLRU, tokens/s",
      "value": B * T / wall, "unit": "tokens/s", "n_gpus": 1,
      "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall * 1e3,
      "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
      "dtype": "bf16", "data": "synthetic",
      "config": {"workload": args.workload, "batch": B, "seq_len": T,
                 "lru_width": W, "heads": H,
                 "path": "the drop-in modules called one by one"},
      "roofline": {"kernel": worst["kernel"], "bound": "hbm",
                   "achieved": worst["achieved_gbs"], "peak": 8000.0,
                   "unit": "GB/s", "frac": worst["frac_of_hbm_peak"],
                   "traffic": None,
                   "algorithmic_bytes": worst["algorithmic_bytes"],
                   "avg_launch_ms": worst["ms"]},
      "modules": modules}))


def run_attention_step(args, torch, ops, wl):
  """rg_attention_decode_fused on one block's decode step (projections in,
  block output before proj_final out; ring and count updated in place), then
  the separate calls it replaces.  Algorithmic bytes: both rings once, the
  projections, the output, the written slot."""
  dev = torch.device("cuda:0")
  B, H, hd, window = wl["B"], wl["H"], 256, wl["window"]
  g = torch.Generator().manual_seed(wl["seed"])
  qkv = torch.randn(B, (H + 2) * hd, generator=g).to(torch.bfloat16).to(dev)
  ring_k = torch.randn(B, window, hd, generator=g).to(torch.bfloat16).to(dev)
  ring_v = torch.randn(B, window, hd, generator=g).to(torch.bfloat16).to(dev)
  nt = torch.full((B,), window + 17, dtype=torch.int32, device=dev)
  pos = nt.to(torch.int64)
  freq = torch.arange(hd // 4, device=dev)
  inv_freq = 1.0 / (10000 ** (2 * freq / (hd // 2)))
  scale = hd ** -0.5
  q, k, v = (qkv[:, :H * hd], qkv[:, H * hd:(H + 1) * hd],
             qkv[:, (H + 1) * hd:])

  def timed(fn, steps, warmup):
    for _ in range(warmup):
      fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
      fn()
    e1.record()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps, e0.elapsed_time(e1) / steps

  def fused():
    return ops.attention_decode_fused(q, k, v, pos, inv_freq, ring_k, ring_v,
                                      nt, scale)

  def separate():
    q4 = q.reshape(B, 1, H, hd).contiguous()
    k4 = k.reshape(B, 1, 1, hd).contiguous()
    qr, kr = ops.rope_pair(q4, k4, pos.reshape(B, 1), inv_freq)
    qh = qr[:, 0]
    scores = torch.bmm(qh, ring_k.transpose(1, 2))
    probs = ops.attention_decode_probs(scores, qh, kr[:, 0, 0], nt, scale)
    from_ring = torch.bmm(probs[..., :window], ring_v)
    return ops.attention_decode_finish(from_ring, probs, kr[:, 0, 0],
                                       v.contiguous(), ring_k, ring_v, nt,
                                       update_cache=True)

  wall, ms = timed(fused, args.steps, args.warmup)
  _, sep_ms = timed(separate, max(3, args.steps // 2), 2)
  nbytes = (2 * B * window * hd * 2 + B * (H + 2) * hd * 2 + B * H * hd * 2 +
            2 * B * hd * 2)
  achieved = nbytes / (ms * 1e-3) / 1e9
  print(json.dumps({
      "metric": "decode-step attention of one local-attention block, tokens/s",
      "value": B / wall, "unit": "tokens/s", "n_gpus": 1,
      "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall * 1e3,
      "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
      "dtype": "bf16", "data": "synthetic",
      "config": {"workload": args.workload, "batch": B, "query_heads": H,
                 "kv_heads": 1, "head_dim": hd, "window": window,
                 "path": "rg_attention_decode_fused, launched from Python "
                         "(two kernels per step)"},
      "roofline": {"kernel": "attn_decode_chunks_kernel + "
                             "attn_decode_combine_kernel (avg_launch_ms covers "
                             "both)",
                   "bound": "hbm", "achieved": achieved, "peak": 8000.0,
                   "unit": "GB/s", "frac": achieved / 8000.0, "traffic": None,
                   "algorithmic_bytes": nbytes, "avg_launch_ms": ms},
      "separate_calls": {"what": "rg_rope_pair, torch.bmm, "
                                 "rg_attention_decode_probs, torch.bmm, "
                                 "rg_attention_decode_finish", "ms": sep_ms}}))


def run_griffin(args, torch, rg, wl):
  """Greedy decoding with the whole 2B-shape model: the recurrent blocks on
  this package's kernels, the rest plain torch.  One step = one new token for
  every sequence of the batch (a cached single-token pass through the 26
  blocks); the prompt pass is timed separately."""
  from recurrentgemma_amd import griffin as G
  from recurrentgemma_amd import sampler as S
  dev = torch.device("cuda:0")
  B, T = wl["B"], wl["T"]
  new_tokens = args.steps + 1 if args.steps != 50 else wl["new_tokens"]
  cfg = G.GriffinConfig.from_preset(G.Preset.RECURRENT_GEMMA_2B_V1)
  torch.manual_seed(wl["seed"])
  model = G.Griffin(cfg, device=dev, dtype=torch.bfloat16).eval()
  n_params = sum(p.numel() for p in model.parameters())
  g = torch.Generator().manual_seed(wl["seed"])
  tokens = torch.randint(0, cfg.vocab_size, (B, T), generator=g).to(
      dev, torch.int32)
  lens = torch.full((B,), T, device=dev, dtype=torch.int32)
  smp = S.Sampler(model, greedy_sampling=True, use_graph=not args.eager)

  def generate(n):
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out, _ = smp.sample_tokens(tokens, lens, n)
    torch.cuda.synchronize()
    return time.perf_counter() - t0, out

  generate(min(args.warmup, 8) + 1)          # warm-up: prompt + a few steps
  t_prompt, _ = generate(1)                  # prompt pass + first token
  t_full, out = generate(new_tokens)
  steps = new_tokens - 1
  t_decode = t_full - t_prompt
  # every decode step reads every parameter once (bf16); the embedding table
  # only as the logits projection
  step_bytes = 2 * n_params
  achieved = step_bytes * steps / t_decode / 1e9
  result = {
      "metric": "greedy decoding tokens/s, 2B residual stack",
      "value": B * steps / t_decode, "unit": "tokens/s", "n_gpus": 1,
      "steps": steps, "warmup": min(args.warmup, 8),
      "ms_per_step": t_decode * 1e3 / steps, "higher_is_better": True,
      "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
      "data": "synthetic",
      "config": {"workload": args.workload, "batch": B, "prompt_len": T,
                 "new_tokens": new_tokens, "blocks": cfg.num_layers,
                 "width": cfg.width, "vocab": cfg.vocab_size,
                 "parameters": n_params,
                 "path": "Sampler.sample_tokens ("
                         + ("eager" if args.eager else "decode step replayed "
                            "as a captured HIP graph")
                         + "), recurrent blocks: "
                         "rg_recurrent_prefill_gelu_mul (prompt) + "
                         "rg_recurrent_step_gelu_mul (step); attention "
                         "blocks: rg_attention_prefill (prompt) + "
                         "rg_attention_decode_fused (step); linear "
                         "layers of a decode step: rg_linear_rows"},
      "prompt_pass": {"ms": t_prompt * 1e3,
                      "tokens_per_s": B * T / t_prompt},
      "whole_generation": {"ms": t_full * 1e3,
                           "new_tokens_per_s": B * new_tokens / t_full},
      "roofline": {"kernel": "one decode step (all kernels of the 26 blocks "
                             "and the logits projection)",
                   "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS,
                   "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                   "traffic": None, "algorithmic_bytes": step_bytes,
                   "avg_launch_ms": t_decode * 1e3 / steps},
      "checksum": int(out.sum().item()),
  }
  print(json.dumps(result))


def run_decode(args, torch, rg, R, ops, wl, cpu_leg=True, name=None):
  """Times rg_recurrent_step (conv step, both gate projections, gate
  activations, state update) on B rows with the caches updated in place.
  Returns the result line as a dict."""
  B, W, H = wl["B"], wl["W"], wl["H"]
  dev = torch.device("cuda:0")
  dtype = torch.bfloat16
  params = R.make_params(W, H, dtype, seed=wl["seed"] + 100)
  P = {k: v.to(dev) for k, v in params.items()}
  g = torch.Generator().manual_seed(wl["seed"])
  x = torch.randn(B, 1, W, generator=g).to(dtype).to(dev)
  conv_cache = torch.randn(B, 3, W, generator=g).to(dtype).to(dev)
  h = torch.randn(B, W, generator=g).to(dev)
  seg = torch.full((B, 1), 2048, dtype=torch.int64, device=dev)

  def step():
    return ops.recurrent_step(x, seg, conv_cache, h, P["conv_w"], P["conv_b"],
                              P["w_x"], P["b_x"], P["w_a"], P["b_a"],
                              P["a_param"], in_place=True)

  settle_launches = 0 if args.no_settle else settle(torch, step, cap_s=0.2)
  for _ in range(args.warmup):
    step()
  torch.cuda.synchronize()
  e0 = torch.cuda.Event(enable_timing=True)
  e1 = torch.cuda.Event(enable_timing=True)

  def eager_loop():
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
      step()
    e1.record()
    torch.cuda.synchronize()
    return time.perf_counter() - t0, e0.elapsed_time(e1) / args.steps

  eager_elapsed, eager_dev_ms = eager_loop()
  if args.eager:
    elapsed, dev_ms = eager_elapsed, eager_dev_ms
  else:
    # The K consecutive steps as one captured HIP graph (what the sampler does
    # with its decode step): the launches cost no host time, the device sees
    # the kernels back to back.
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
      for _ in range(args.steps):
        step()
    graph.replay()
    torch.cuda.synchronize()
    # the graph of K steps replayed a few times: the median replay counts
    reps = []
    for _ in range(5):
      t0 = time.perf_counter()
      e0.record()
      graph.replay()
      e1.record()
      torch.cuda.synchronize()
      reps.append((e0.elapsed_time(e1) / args.steps, time.perf_counter() - t0))
    reps.sort()
    dev_ms, elapsed = reps[len(reps) // 2]
  algo = decode_algorithmic_bytes(B, W, H, 2)
  achieved = algo / (dev_ms * 1e-3) / 1e9
  result = {
      "metric": METRIC,
      "value": B / (elapsed / args.steps), "unit": "tokens/s", "n_gpus": 1,
      "steps": args.steps, "warmup": args.warmup,
      "ms_per_step": elapsed * 1e3 / args.steps, "higher_is_better": True,
      "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
      "data": "synthetic",
      "config": {"workload": name or args.workload, "batch": B, "seq_len": 1,
                 "lru_width": W, "heads": H, "activations": "bf16",
                 "state": "f32",
                 "path": "rg_recurrent_step, caches in place, "
                         + ("launched from Python step by step" if args.eager
                            else "the steps captured as one HIP graph")},
      "eager_loop": {"ms_per_step": eager_elapsed * 1e3 / args.steps,
                     "device_ms_per_step": eager_dev_ms},
      "roofline": {"kernel": "rg_recurrent_step (all launches of one step)",
                   "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS,
                   "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                   "traffic": None, "algorithmic_bytes": algo,
                   "avg_launch_ms": dev_ms,
                   "settle_launches": settle_launches,
                   "shader_clock_ghz_after": shader_clock_ghz(torch)},
  }
  if cpu_leg and not args.no_cpu_baseline:
    cores = host_cores()
    torch.set_num_threads(cores)
    xc, cc, hc = x.cpu(), conv_cache.cpu(), h.cpu()
    segc = seg.cpu()
    cache = R.CoreCache(rg_lru_state=hc, conv1d_state=cc)
    R.recurrent_core(xc, segc, params, cache)
    n = 20
    t0 = time.perf_counter()
    for _ in range(n):
      _, cache = R.recurrent_core(xc, segc, params, cache)
    dt = (time.perf_counter() - t0) / n
    result["cpu_baseline"] = {
        "value": B / dt, "unit": "tokens/s", "cores": cores, "kind": "port",
        "cpu": cpu_model(),
        "sample": (f"oracle/torch_ref.recurrent_core with caches, bf16, {n} "
                   f"decode steps of {B} rows (W={W}, H={H}), mean, torch "
                   f"threads={torch.get_num_threads()}")}
  return result


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=50)
  ap.add_argument("--warmup", type=int, default=10)
  ap.add_argument("--workload", default="9b_prefill", choices=sorted(WORKLOADS))
  ap.add_argument("--path", default="auto", choices=["auto", "single", "split"])
  ap.add_argument("--no-cpu-baseline", action="store_true",
                  help="lean run for the profiler: no CPU leg and no "
                       "additional 2B-width measurement")
  ap.add_argument("--no-settle", action="store_true",
                  help="skip the untimed settle phase before the warm-up steps "
                       "(launches until their durations stop moving, at most "
                       "0.5 s)")
  ap.add_argument("--eager", action="store_true",
                  help="2b_griffin_decode, 9b_decode: launch every kernel of a "
                       "decode step from Python instead of replaying a "
                       "captured graph")
  ap.add_argument("--calibration-copy", action="store_true",
                  help="after the timed steps, run one plain device copy of x "
                       "(known size) so that a counter run of this command "
                       "holds a reference dispatch to scale FETCH_SIZE / "
                       "WRITE_SIZE by")
  args = ap.parse_args()
  if args.gpus != 1:
    sys.exit("bench.py measures one GPU: this build has no multi-GPU path "
             "(run with --gpus 1)")

  import torch

  import recurrentgemma_amd as rg
  from oracle import torch_ref as R
  from recurrentgemma_amd import ops

  wl = WORKLOADS[args.workload]
  if wl.get("griffin"):
    run_griffin(args, torch, rg, wl)
    return
  if wl.get("decode"):
    print(json.dumps(run_decode(args, torch, rg, R, ops, wl)))
    return
  if wl.get("attention"):
    run_attention(args, torch, ops, wl)
    return
  if wl.get("attention_step"):
    run_attention_step(args, torch, ops, wl)
    return
  if wl.get("modules"):
    run_modules(args, torch, rg, R, wl)
    return
  if wl.get("training"):
    run_training(args, torch, rg, ops, wl)
    return
  result = run_prefill(args, torch, rg, R, ops, args.workload, args.steps,
                       args.warmup, extras=True)
  if (args.workload == "9b_prefill" and args.path == "auto"
      and not args.no_cpu_baseline):
    # the metric names both widths: the 2B-shape prefill, same contract, after
    # the timed region of the headline workload
    r2 = run_prefill(args, torch, rg, R, ops, "2b_prefill",
                     max(10, args.steps // 2), 5, extras=False)
    result["at_2b_width"] = {
        k: r2[k] for k in ("value", "unit", "steps", "warmup", "ms_per_step",
                           "config", "roofline", "gate_gemm",
                           "two_kernel_path") if k in r2}
    # ... and the other single-block configurations, each a few seconds: the
    # decode step (steps as one captured graph) and the float32 case, whose
    # 21 MB stay in the caches (warm and cold figures)
    saved = args.steps, args.warmup
    args.steps, args.warmup = 64, 10
    rd = run_decode(args, torch, rg, R, ops, WORKLOADS["9b_decode"],
                    cpu_leg=False, name="9b_decode")
    args.steps, args.warmup = saved
    result["at_decode"] = {
        k: rd[k] for k in ("value", "unit", "steps", "warmup", "ms_per_step",
                           "config", "eager_loop", "roofline") if k in rd}
    rf = run_prefill(args, torch, rg, R, ops, "2b_f32", 50, 10, extras=False,
                     cold_too=True)
    result["at_f32"] = {
        k: rf[k] for k in ("value", "unit", "steps", "warmup", "ms_per_step",
                           "dtype", "config", "roofline", "gate_gemm",
                           "cold_caches") if k in rf}
  print(json.dumps(result))


def run_prefill(args, torch, rg, R, ops, workload, steps, warmup, extras,
                cold_too=False):
  """One prefill workload: `warmup` untimed steps, `steps` timed ones; returns
  the result line as a dict; with the default path also the two-kernel form
  of a single-kernel workload, after the timed region.  extras: the
  calibration copy and the CPU baseline too; cold_too: for a working set that
  fits the caches, also the figure with the caches flushed between steps."""
  wl = WORKLOADS[workload]
  B, T, W, H = wl["B"], wl["T"], wl["W"], wl["H"]
  dev = torch.device("cuda:0")
  dtype = torch.float32 if wl.get("dtype") == "f32" else torch.bfloat16
  esize = 4 if dtype == torch.float32 else 2

  params = R.make_params(W, H, dtype, seed=wl["seed"] + 100)
  g = torch.Generator().manual_seed(wl["seed"])
  x = torch.randn(B, T, W, generator=g).to(dtype).to(dev)
  seg = make_segment_pos(torch, B, T, wl["mean_doc"], wl["seed"]).to(dev)
  blk = rg.RecurrentBlock(width=W, num_heads=H, dtype=dtype)
  blk.conv_1d.load_state_dict({"w": params["conv_w"], "b": params["conv_b"]})
  blk.rg_lru.load_state_dict({
      "a_param": params["a_param"], "input_gate.w": params["w_x"],
      "input_gate.b": params["b_x"], "a_gate.w": params["w_a"],
      "a_gate.b": params["b_a"]})
  blk = blk.to(dev)
  conv, lru = blk.conv_1d, blk.rg_lru

  def step_split(events=None):
    if events:
      events[0].record()
    gx, ga = ops.gates_gemm(x, lru.input_gate.w, lru.input_gate.b,
                            lru.a_gate.w, lru.a_gate.b,
                            conv=(seg, conv.w, conv.b))
    if events:
      events[1].record()
    y, h, cache = ops.lru_scan_fused(x, gx, ga, lru.a_param, seg,
                                     conv=(conv.w, conv.b),
                                     return_conv_cache=True)
    if events:
      events[2].record()
    return y, h, cache

  def step_single(events=None):
    if events:
      events[0].record()
    out = ops.recurrent_prefill(x, seg, conv.w, conv.b, lru.input_gate.w,
                                lru.input_gate.b, lru.a_gate.w, lru.a_gate.b,
                                lru.a_param)
    if events:
      events[1].record()
      events[2].record()
    return out

  def step_core(events=None):
    # what RecurrentBlock calls: one library call that picks the kernels
    if events:
      events[0].record()
    out = ops.recurrent_core(x, seg, conv.w, conv.b, lru.input_gate.w,
                             lru.input_gate.b, lru.a_gate.w, lru.a_gate.b,
                             lru.a_param)
    if events:
      events[1].record()
      events[2].record()
    return out

  # the choice rg_recurrent_core makes: the single kernel where its workgroups
  # (one per row, head and time chunk) fill the GPU
  chunked = esize == 2 and ops.recurrent_prefill_chunked(B, T, W, H)
  path = args.path
  if path == "auto":
    many_short = (B * H > 512 and T <= 16) or (B * H > 1024 and T <= 32)
    path = ("single" if ops.recurrent_prefill_supported(x, H)
            and not many_short else "split")
  if args.path == "auto":
    step = step_core
  else:
    step = step_single if path == "single" else step_split
  # float32, 256-wide heads, at most 32 (row, head) pairs: the library's
  # one-launch float32 kernel (core_f32_small_serves in csrc/rg_core_f32.hip)
  f32_single = (args.path == "auto" and esize == 4 and W // H == 256
                and B * H <= 32)

  per_launch = {}

  def timed(fn, steps, warmup, key=None):
    for _ in range(warmup):
      fn()
    torch.cuda.synchronize()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)]
           for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
      fn(evs[i])
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    a = [e[0].elapsed_time(e[1]) for e in evs]
    b = [e[1].elapsed_time(e[2]) for e in evs]
    if key:
      per_launch[key] = (launch_stats(a), launch_stats(b))
    return elapsed, sum(a) / steps, sum(b) / steps

  # untimed: until the launch durations stop moving (the clock ramp after
  # start-up), before the --warmup steps
  settle_launches = 0 if args.no_settle else settle(torch, step)
  elapsed, first_ms, second_ms = timed(step, steps, warmup, key="main")
  clock_ghz = shader_clock_ghz(torch)
  clock_loaded = prefill_clock_under_load(torch, step) if esize == 2 else None

  tokens = B * T
  from recurrentgemma_amd import _lib
  in_chunks = _lib.lib().rg_scan_split_workspace_bytes(B, T, W) > 0
  seg_bytes = seg.element_size()
  scan_algo = scan_algorithmic_bytes(B, T, W, esize, seg_bytes, has_h0=False)
  gemm_flops = 1024.0 * W * tokens
  gemm_bytes = 3 * esize * B * T * W

  def split_figures(gemm_ms, scan_ms):
    achieved = scan_algo / (scan_ms * 1e-3) / 1e9
    traffic, source = measured_traffic(workload, "scan")
    return {
        "scan": {
            "kernel": "lru_scan_kernel (conv + gates + scan)",
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic, "traffic_source": source,
            "algorithmic_bytes": scan_algo, "avg_launch_ms": scan_ms},
        "gate_gemm": {
            "kernel": ("gates_mfma_bf16_kernel" if esize == 2
                       else "gates_mfma_f32_kernel (v_mfma_f32_32x32x2_f32)"),
            "avg_launch_ms": gemm_ms,
            "tflops": gemm_flops / (gemm_ms * 1e-3) / 1e12,
            "frac_of_mfma_peak": gemm_flops / (gemm_ms * 1e-3)
                                 / (2.5e15 if esize == 2 else 157.3e12),
            "gbs": gemm_bytes / (gemm_ms * 1e-3) / 1e9,
            "frac_of_hbm_peak": gemm_bytes / (gemm_ms * 1e-3) / 1e9
                                / HBM_PEAK_GBS}}

  if path == "single":
    algo = single_algorithmic_bytes(B, T, W, H, 2, seg_bytes, has_h0=False)
    achieved = algo / (first_ms * 1e-3) / 1e9
    traffic, source = measured_traffic(workload, "single")
    roofline = {
        "kernel": ("block_prefill_teams_bf16_kernel (conv + gate GEMMs + gates "
                   "+ scan, two waves per SIMD)"
                   + (": two launches (chunk 0 + summaries of the chunks "
                      "after it; replay of chunks 1..n-1); avg_launch_ms "
                      "covers both" if chunked else "")),
        "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS,
        "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
        "traffic": traffic, "traffic_source": source,
        "algorithmic_bytes": algo, "avg_launch_ms": first_ms,
        "launch_ms": per_launch["main"][0],
        "mfma_tflops": gemm_flops / (first_ms * 1e-3) / 1e12,
        "frac_of_bf16_mfma_peak": gemm_flops / (first_ms * 1e-3) / 2.5e15}
  elif f32_single:
    # float32 with few rows: rg_recurrent_core is ONE launch that does the
    # conv, both gate projections (true float32 products on the float32
    # matrix instruction), the gates and the recurrence
    algo = single_algorithmic_bytes(B, T, W, H, 4, seg_bytes, has_h0=False)
    tf = gemm_flops / (first_ms * 1e-3) / 1e12
    roofline = {
        "kernel": "core_f32_small_kernel (conv + gate GEMMs on "
                  "v_mfma_f32_16x16x4_f32 + gates + scan, one launch)",
        "bound": "mfma", "achieved": tf, "peak": 157.3, "unit": "TFLOP/s",
        "frac": tf / 157.3, "traffic": None, "algorithmic_bytes": algo,
        "avg_launch_ms": first_ms, "launch_ms": per_launch["main"][0],
        "gbs": algo / (first_ms * 1e-3) / 1e9}
  else:
    if args.path == "auto":
      # per-kernel durations: the same two launches called one by one, with
      # events between them, after the timed region
      _, first_ms, second_ms = timed(step_split, steps, warmup, key="main")
    figs = split_figures(first_ms, second_ms)
    figs["gate_gemm"]["launch_ms"] = per_launch["main"][0]
    figs["scan"]["launch_ms"] = per_launch["main"][1]
    roofline = figs["scan"]
  roofline["settle_launches"] = settle_launches
  roofline["shader_clock_ghz_after"] = clock_ghz
  if path == "single":
    roofline["shader_clock_ghz_under_load"] = clock_loaded

  cold = None
  if (extras or cold_too) and x.numel() * esize * 4 < (256 << 20):
    # The whole working set fits the caches (4 MB of L2 per XCD, 256 MB behind
    # them): the timed loop above is a warm-cache figure.  Cold: 1 GiB is
    # written between the steps and each step is timed on its own.
    flush = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    n_cold = min(steps, 20)
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)]
           for _ in range(n_cold)]
    for i in range(n_cold):
      flush.fill_(i & 1)
      step(evs[i])
    torch.cuda.synchronize()
    cold = {"ms_per_step": sum(e[0].elapsed_time(e[2]) for e in evs) / n_cold,
            "steps": n_cold,
            "how": "1 GiB written between steps; HIP events around each step"}
    del flush

  if extras and args.calibration_copy:
    torch.empty_like(x).copy_(x)  # reads and writes x.numel()*2 bytes
    torch.cuda.synchronize()

  result = {
      "metric": METRIC,
      "value": tokens / (elapsed / steps),
      "unit": "tokens/s",
      "n_gpus": 1,
      "steps": steps,
      "warmup": warmup,
      "ms_per_step": elapsed * 1e3 / steps,
      "higher_is_better": True,
      "scaling": "weak",
      "vs_baseline": None,
      "dtype": "bf16" if esize == 2 else "f32",
      "data": "synthetic",
      "config": {
          "workload": workload, "batch": B, "seq_len": T, "lru_width": W,
          "heads": H, "activations": "bf16" if esize == 2 else "f32",
          "state": "f32",
          "documents": ("one per row" if wl["mean_doc"] is None
                        else f"geometric mean {wl['mean_doc']}"),
          "path": ("rg_recurrent_prefill_split (single kernel, rows in time "
                   "chunks side by side)" if path == "single" and chunked
                   else "rg_recurrent_prefill (single launch)"
                   if path == "single"
                   else "rg_recurrent_core: one float32 launch (conv + gate "
                        "GEMMs + gates + scan)" if f32_single
                   else ("rg_recurrent_core: " if args.path == "auto" else "")
                        + "rg_gates_gemm(conv on load) + "
                        + ("rg_lru_scan_fused_split(conv): sequences in chunks "
                           "side by side" if in_chunks
                           else "rg_lru_scan_fused(conv)"))},
      "roofline": roofline,
  }
  if cold:
    result["cold_caches"] = cold
  if path == "split" and not f32_single:
    result["gate_gemm"] = figs["gate_gemm"]
  elif args.path == "auto":
    # the two-kernel form of the same step, measured after the timed region
    n2 = max(20, steps // 2)
    if not args.no_settle:
      settle(torch, step_split, cap_s=0.25)
    e2, g_ms, s_ms = timed(step_split, n2, 3, key="split")
    figs = split_figures(g_ms, s_ms)
    figs["gate_gemm"]["launch_ms"] = per_launch["split"][0]
    figs["scan"]["launch_ms"] = per_launch["split"][1]
    result["two_kernel_path"] = {
        "value": tokens / (e2 / n2), "unit": "tokens/s", "steps": n2,
        "scan": figs["scan"], "gate_gemm": figs["gate_gemm"]}
  if extras and not args.no_cpu_baseline:
    result["cpu_baseline"] = cpu_baseline(torch, R, wl, params)
  return result


if __name__ == "__main__":
  main()
