"""Writes tests/golden/griffin_golden.npz from the REAL reference model.

Run once, in the build container only (the reference does not exist on the GPU
box):  python tests/golden/make_griffin_golden.py

The reference's common.py and torch/{array_typing,layers,modules,griffin,
sampler}.py are loaded by file path (the package __init__ imports JAX, and
jaxtyping is not installed: sys.modules is pre-seeded with a stand-in for the
jaxtyping annotation classes and with empty parent packages).  No reference
file is modified, copied or written.

What is pinned (nothing but the reference fixes these: mask and ring-cache
arithmetic of the attention block, rotary embedding, residual wiring, logits
soft cap, the sampler's left padding and split prompt processing):
  * Griffin.forward on a left-padded batch: logits and every block's cache;
  * one cached decode step after it: logits and caches;
  * a prompt longer than the attention window (ring wrap-around) + 3 steps;
  * Sampler.__call__ (greedy) on prompts of different lengths, with logits.
All float32, tiny shapes.  The model's parameters are stored too, under the
reference's state-dict keys.

With --bf16 it writes tests/golden/griffin_bf16_golden.npz instead: the
reference model in bfloat16 with 256-wide RG-LRU heads (the shapes that take
this package's bf16 kernels), its parameters regenerated from a seed by
tests/helpers.seeded_state_dict instead of stored, and beside every bf16
result the same computation by the reference in float32 on the same
(bf16-valued) parameters: the distance between the two is the yardstick for a
third bf16 implementation.
"""

import importlib.util
import os
import sys
import types

import numpy as np
import torch

ROOT = "/root/reference/recurrentgemma"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)),
                   "griffin_golden.npz")


def load_reference():
  class _Ann:
    def __class_getitem__(cls, item):
      return cls

  jt = types.ModuleType("jaxtyping")
  for name in ("Float", "Integer", "Bool", "Int", "Array"):
    setattr(jt, name, type(name, (_Ann,), {}))
  sys.modules["jaxtyping"] = jt
  for pkg in ("recurrentgemma", "recurrentgemma.torch"):
    m = types.ModuleType(pkg)
    m.__path__ = []
    sys.modules[pkg] = m

  def load(name, path):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    setattr(sys.modules[name.rsplit(".", 1)[0]], name.rsplit(".", 1)[1], mod)
    spec.loader.exec_module(mod)
    return mod

  common = load("recurrentgemma.common", os.path.join(ROOT, "common.py"))
  for name in ("array_typing", "layers", "modules", "griffin", "sampler"):
    mod = load(f"recurrentgemma.torch.{name}",
               os.path.join(ROOT, "torch", f"{name}.py"))
  return common, sys.modules["recurrentgemma.torch.griffin"], mod


class ToyVocab:
  """Whitespace-separated integers as token ids."""

  def bos_id(self):
    return 2

  def eos_id(self):
    return 1

  def pad_id(self):
    return 0

  def EncodeAsIds(self, s):
    return [int(t) for t in s.split()]

  def DecodeIds(self, ids):
    return " ".join(str(i) for i in ids)


def flat_cache(prefix, cache, out):
  for name, c in cache.items():
    for field, value in c._asdict().items():
      out[f"{prefix}/{name}/{field}"] = value.detach().cpu().numpy().copy()


def main():
  common, griffin, sampler = load_reference()
  R, A = common.TemporalBlockType.RECURRENT, common.TemporalBlockType.ATTENTION
  config = common.GriffinConfig(
      vocab_size=48, width=32, mlp_expanded_width=40, num_heads=2,
      block_types=(R, A, R), embeddings_scale_by_sqrt_dim=True,
      attention_window_size=6, logits_soft_cap=30.0, lru_width=64)
  torch.manual_seed(4242)
  model = griffin.Griffin(config, gradient_checkpointing=False,
                          dtype=torch.float32)
  with torch.no_grad():
    # zero-initialised parameters would leave their paths untested
    for name, p in model.named_parameters():
      if name.endswith((".b", ".bias", ".scale")):
        p.normal_(0.0, 0.1)
  model.eval()
  out = {f"param/{k}": v.detach().numpy().copy()
         for k, v in model.state_dict().items()}

  gen = torch.Generator().manual_seed(7)
  with torch.no_grad():
    # ---- case 1: left-padded batch, then one cached step -------------------
    T = 5
    tokens = torch.randint(3, config.vocab_size, (2, T), generator=gen)
    pos = torch.stack([torch.arange(T), torch.tensor([-1, -1, 0, 1, 2])])
    logits, cache = model(tokens, pos, None, return_logits=True,
                          return_cache=True)
    out["c1/tokens"], out["c1/pos"] = tokens.numpy(), pos.numpy()
    out["c1/logits"] = logits.numpy().copy()
    flat_cache("c1/cache", cache, out)
    nxt = torch.randint(3, config.vocab_size, (2, 1), generator=gen)
    npos = pos[:, -1:] + 1
    # the reference's checkpoint-free branch drops return_cache: call blocks
    # through the same public forward, which returns the cache by default
    logits2, cache2 = model(nxt, npos, cache, return_logits=True,
                            return_cache=True)
    out["c1/next_tokens"], out["c1/next_pos"] = nxt.numpy(), npos.numpy()
    out["c1/next_logits"] = logits2.numpy().copy()
    flat_cache("c1/next_cache", cache2, out)

    # ---- case 2: prompt longer than the window, three cached steps ---------
    T = 9
    tokens = torch.randint(3, config.vocab_size, (2, T), generator=gen)
    pos = torch.stack([torch.arange(T),
                       torch.cat([torch.arange(4), torch.arange(5)])])
    logits, cache = model(tokens, pos, None, return_logits=True,
                          return_cache=True)
    out["c2/tokens"], out["c2/pos"] = tokens.numpy(), pos.numpy()
    out["c2/logits"] = logits.numpy().copy()
    flat_cache("c2/cache", cache, out)
    steps = torch.randint(3, config.vocab_size, (2, 3), generator=gen)
    out["c2/step_tokens"] = steps.numpy()
    p = pos[:, -1:] + 1
    for i in range(3):
      lg, cache = model(steps[:, i:i + 1], p, cache, return_logits=True,
                        return_cache=True)
      out[f"c2/step{i}_logits"] = lg.numpy().copy()
      p = p + 1
    flat_cache("c2/final_cache", cache, out)

    # ---- case 3: the sampler, greedy, prompts of different lengths ---------
    smp = sampler.Sampler(model, ToyVocab(), greedy_sampling=True)
    prompts = ["5 9 13 21 8 30 11", "7 40 3", "12"]
    for echo in (False, True):
      res = smp(prompts, total_generation_steps=6, echo=echo,
                return_logits=True, end_sampling_at_eos_token=False)
      tag = "c3/echo" if echo else "c3/plain"
      for i, (t, lg) in enumerate(zip(res.tokens, res.logits)):
        out[f"{tag}/tokens{i}"] = t.numpy().copy()
        out[f"{tag}/logits{i}"] = lg.numpy().copy()
      out[f"{tag}/text"] = np.array(res.text)
    out["c3/prompts"] = np.array(prompts)

  np.savez_compressed(OUT, **out)
  print("wrote", OUT, len(out), "arrays,", os.path.getsize(OUT), "bytes")


BF16_OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)),
                        "griffin_bf16_golden.npz")
BF16_SEED = 77


def bf16_config(common):
  R, A = common.TemporalBlockType.RECURRENT, common.TemporalBlockType.ATTENTION
  return common.GriffinConfig(
      vocab_size=512, width=512, mlp_expanded_width=768, num_heads=2,
      block_types=(R, R, A), embeddings_scale_by_sqrt_dim=True,
      attention_window_size=16, logits_soft_cap=30.0, lru_width=512)


def main_bf16():
  sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(
      os.path.abspath(__file__)))))
  from tests import helpers
  common, griffin, sampler = load_reference()
  config = bf16_config(common)
  models = {}
  for tag, dtype in (("bf16", torch.bfloat16), ("f32", torch.float32)):
    m = griffin.Griffin(config, gradient_checkpointing=False, dtype=dtype)
    shapes = {k: tuple(v.shape) for k, v in m.state_dict().items()}
    sd = helpers.seeded_state_dict(shapes, BF16_SEED, torch.bfloat16)
    m.load_state_dict({k: v.to(dtype) for k, v in sd.items()})
    models[tag] = m.eval()
  out = {"param_checksum": np.float64(helpers.state_dict_checksum(sd)),
         "param_seed": np.int64(BF16_SEED)}

  def f32(t):
    return t.detach().float().cpu().numpy().copy()

  gen = torch.Generator().manual_seed(9)
  with torch.no_grad():
    # ---- case 1: left-padded prompts longer than the window + 4 steps ------
    T, steps = 24, 4
    tokens = torch.randint(3, config.vocab_size, (2, T), generator=gen)
    pos = torch.stack([torch.arange(T),
                       torch.cat([torch.full((5,), -1), torch.arange(T - 5)])])
    step_tokens = torch.randint(3, config.vocab_size, (2, steps), generator=gen)
    out["c1/tokens"], out["c1/pos"] = tokens.numpy(), pos.numpy()
    out["c1/step_tokens"] = step_tokens.numpy()
    for tag, m in models.items():
      logits, cache = m(tokens, pos, None, return_logits=True,
                        return_cache=True)
      out[f"c1/{tag}/logits"] = f32(logits)
      for name, c in cache.items():
        for field, value in c._asdict().items():
          out[f"c1/{tag}/cache/{name}/{field}"] = f32(value) if (
              value.is_floating_point()) else value.numpy().copy()
      p = pos[:, -1:] + 1
      for i in range(steps):
        lg, cache = m(step_tokens[:, i:i + 1], p, cache, return_logits=True,
                      return_cache=True)
        out[f"c1/{tag}/step{i}_logits"] = f32(lg)
        p = p + 1
      for name, c in cache.items():
        for field, value in c._asdict().items():
          out[f"c1/{tag}/final_cache/{name}/{field}"] = f32(value) if (
              value.is_floating_point()) else value.numpy().copy()

    # ---- case 2: the sampler, greedy, prompts of different lengths ---------
    prompts = ["5 9 13 21 8 30 11 400 17 250 31 77 19 23 101 202 303 404 55",
               "7 40 3", "12 500 6 88 91"]
    out["c2/prompts"] = np.array(prompts)
    for tag, m in models.items():
      smp = sampler.Sampler(m, ToyVocab(), greedy_sampling=True)
      res = smp(prompts, total_generation_steps=12, echo=True,
                return_logits=True, end_sampling_at_eos_token=False)
      for i, (t, lg) in enumerate(zip(res.tokens, res.logits)):
        out[f"c2/{tag}/tokens{i}"] = t.numpy().copy()
        out[f"c2/{tag}/logits{i}"] = f32(lg)

  np.savez_compressed(BF16_OUT, **out)
  print("wrote", BF16_OUT, len(out), "arrays,", os.path.getsize(BF16_OUT),
        "bytes")
  for k in ("c1/%s/logits", "c1/%s/step3_logits", "c2/%s/logits0"):
    a, b = out[k % "bf16"], out[k % "f32"]
    print(k, "max |bf16 - f32| =", np.abs(a - b).max(), "rms",
          np.sqrt(np.mean((a - b) ** 2)), "max |f32| =", np.abs(b).max())


if __name__ == "__main__":
  if "--bf16" in sys.argv[1:]:
    main_bf16()
  else:
    main()
