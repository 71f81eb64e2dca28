"""The bf16 residual stack and sampler on the GPU against vectors written by
the reference model itself in bfloat16 (tests/golden/make_griffin_golden.py
--bf16: 256-wide RG-LRU heads, so the recurrent blocks take the bf16 kernels of
this package: single-launch prefill, packed decode step, few-row linear
layers).

Two bf16 implementations that round at different places cannot agree to the
1e-2 absolute / 1e-4 relative the reference uses between its own forward and
sampler passes (recurrentgemma/torch/sampler_test.py:217-222): the logits reach
14 and bf16 resolves 0.06 there.  The fixture therefore also holds the
reference's float32 results on the same bf16-valued parameters, and the bar is
the reference's own bf16 error against them:
  * max |ours - f32| <= 2 x max |reference bf16 - f32| and the same for the
    root mean square with factor 1.5, per tensor (logits, every cache field);
  * |ours - reference bf16| <= the sum of the two errors (triangle
    inequality, elementwise at the maximum);
  * greedy tokens equal the reference's until a step where the reference's own
    margin between the two candidates is below its bf16 error; the comparison
    of that row stops there.
The parameters are regenerated from the fixture's seed (helpers.
seeded_state_dict) and checked against its checksum."""

import os

import numpy as np
import pytest
import torch

from tests import helpers
from recurrentgemma_amd import griffin as G
from recurrentgemma_amd import sampler as S

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
GOLDEN = os.path.join(os.path.dirname(__file__), "golden",
                      "griffin_bf16_golden.npz")


@pytest.fixture(scope="module")
def golden():
  return np.load(GOLDEN)


@pytest.fixture(scope="module")
def model(golden):
  R, A = G.TemporalBlockType.RECURRENT, G.TemporalBlockType.ATTENTION
  cfg = G.GriffinConfig(
      vocab_size=512, width=512, mlp_expanded_width=768, num_heads=2,
      block_types=(R, R, A), embeddings_scale_by_sqrt_dim=True,
      attention_window_size=16, logits_soft_cap=30.0, lru_width=512)
  m = G.Griffin(cfg, dtype=torch.bfloat16)
  shapes = {k: tuple(v.shape) for k, v in m.state_dict().items()}
  sd = helpers.seeded_state_dict(shapes, int(golden["param_seed"]))
  assert helpers.state_dict_checksum(sd) == pytest.approx(
      float(golden["param_checksum"]), rel=1e-12)
  m.load_state_dict(sd)
  return m.to(DEV).eval()


def within_reference_error(got, ref_bf16, ref_f32, what):
  got = got.detach().float().cpu()
  ref_bf16 = torch.from_numpy(np.asarray(ref_bf16)).float()
  ref_f32 = torch.from_numpy(np.asarray(ref_f32)).float()
  assert got.shape == ref_f32.shape, (what, got.shape, ref_f32.shape)
  if got.numel() == 0:
    return
  scale = ref_f32.abs().max().item()
  floor = 2.0 ** -8 * scale  # one bf16 rounding of the largest value
  ref_err = (ref_bf16 - ref_f32).abs()
  our_err = (got - ref_f32).abs()
  assert our_err.max().item() <= 2.0 * ref_err.max().item() + floor, (
      what, "max", our_err.max().item(), ref_err.max().item(), scale)
  rms = lambda e: e.pow(2).mean().sqrt().item()
  assert rms(our_err) <= 1.5 * rms(ref_err) + floor / 8, (
      what, "rms", rms(our_err), rms(ref_err), scale)
  assert (got - ref_bf16).abs().max().item() <= (
      our_err.max().item() + ref_err.max().item()), what


def check_cache(cache, golden, prefix):
  names = [k for k in golden.files if k.startswith(f"{prefix % 'bf16'}/")]
  assert names
  for k in names:
    block, field = k[len(prefix % "bf16") + 1:].split("/")
    got = getattr(cache[block], field)
    k32 = (prefix % "f32") + k[len(prefix % "bf16"):]
    if not got.is_floating_point():
      assert torch.equal(got.cpu().long(),
                         torch.from_numpy(golden[k]).long()), k
    else:
      within_reference_error(got, golden[k], golden[k32], k)


def dev(a):
  return torch.from_numpy(np.asarray(a)).to(DEV)


def test_forward_and_steps_against_reference_bf16(model, golden):
  pos = dev(golden["c1/pos"])
  logits, cache = model(dev(golden["c1/tokens"]), pos)
  assert logits.dtype == torch.bfloat16
  within_reference_error(logits, golden["c1/bf16/logits"],
                         golden["c1/f32/logits"], "c1/logits")
  check_cache(cache, golden, "c1/%s/cache")
  steps = dev(golden["c1/step_tokens"])
  p = pos[:, -1:] + 1
  for i in range(steps.shape[1]):
    lg, cache = model(steps[:, i:i + 1], p, cache)
    within_reference_error(lg, golden[f"c1/bf16/step{i}_logits"],
                           golden[f"c1/f32/step{i}_logits"], f"c1/step{i}")
    p = p + 1
  check_cache(cache, golden, "c1/%s/final_cache")


class ToyVocab:
  def bos_id(self): return 2
  def eos_id(self): return 1
  def pad_id(self): return 0
  def EncodeAsIds(self, s): return [int(t) for t in s.split()]
  def DecodeIds(self, ids): return " ".join(str(i) for i in ids)


@pytest.mark.parametrize("use_graph", [True, False])
def test_sampler_against_reference_bf16(model, golden, use_graph):
  """Sampler.__call__ (echo, logits returned) with the decode step replayed as
  a captured graph, and launched eagerly."""
  smp = S.Sampler(model, ToyVocab(), greedy_sampling=True, use_graph=use_graph)
  prompts = [str(p) for p in golden["c2/prompts"]]
  res = smp(prompts, total_generation_steps=12, echo=True, return_logits=True,
            end_sampling_at_eos_token=False)
  for i, prompt in enumerate(prompts):
    want_t = torch.from_numpy(golden[f"c2/bf16/tokens{i}"]).long()
    ref_bf16 = torch.from_numpy(golden[f"c2/bf16/logits{i}"])
    ref_f32 = torch.from_numpy(golden[f"c2/f32/logits{i}"])
    got_t = res.tokens[i].cpu().long()
    got_l = res.logits[i].float().cpu()
    assert got_t.shape == want_t.shape and got_l.shape == ref_bf16.shape
    n_prompt = len(prompt.split()) + 1  # bos
    assert torch.equal(got_t[:n_prompt], want_t[:n_prompt])
    ref_err = (ref_bf16 - ref_f32).abs().max().item()
    same = n_prompt
    # logits row j predicts token j + 1
    for j in range(n_prompt, len(want_t)):
      if got_t[j] == want_t[j]:
        same = j + 1
        continue
      row = ref_bf16[j - 1]
      margin = (row[want_t[j]] - row[got_t[j]]).item()
      assert 0 <= margin <= 2 * ref_err, (i, j, margin, ref_err)
      break
    # until the sequences part, the logits are those of the same inputs
    within_reference_error(got_l[:same], ref_bf16[:same], ref_f32[:same],
                           f"c2/logits{i}[:{same}]")
    assert same >= n_prompt + 1, (i, same)


def test_config5_full_shape_graph_equals_eager():
  """Benchmark configuration 5 at its full shape: the 2B preset (26 blocks,
  width 2560, 10 heads of 256, window 2048, vocabulary 256000), random-init
  bf16, batch 64.  A short left-padded prompt, then a few greedy steps: the
  decode step replayed as a captured graph gives the tokens and logits of the
  eager loop bit for bit, every logit is finite and inside the soft cap, and
  a row's tokens do not depend on its neighbours.  (Reference-written vectors
  pin the same kernels at width 512: test_sampler_against_reference_bf16.)"""
  cfg = G.GriffinConfig.from_preset(G.Preset.RECURRENT_GEMMA_2B_V1)
  torch.manual_seed(1005)
  print("config5 full shape: model", flush=True)
  m = G.Griffin(cfg, device=DEV, dtype=torch.bfloat16).eval()
  B, L, steps = 64, 40, 6
  g = torch.Generator().manual_seed(1005)
  toks = torch.randint(3, cfg.vocab_size, (B, L), generator=g).to(
      DEV, torch.int32)
  lens = torch.full((B,), L, device=DEV, dtype=torch.int32)
  lens[1::2] = L - 7  # every second row left-padded
  for b in range(1, B, 2):
    toks[b, :7] = 0
  print("config5 full shape: eager", flush=True)
  want_t, want_l = S.Sampler(m).sample_tokens(toks, lens, steps,
                                              return_logits=True)
  print("config5 full shape: graph", flush=True)
  got_t, got_l = S.Sampler(m, use_graph=True).sample_tokens(
      toks, lens, steps, return_logits=True)
  torch.cuda.synchronize()
  assert torch.equal(got_t, want_t)
  assert torch.equal(got_l, want_l)
  assert torch.isfinite(got_l.float()).all()
  assert got_l.float().abs().max().item() <= cfg.logits_soft_cap
  print("config5 full shape: four rows alone", flush=True)
  alone_t, _ = S.Sampler(m).sample_tokens(toks[:4].contiguous(),
                                          lens[:4].contiguous(), steps)
  # (other batch sizes take other kernels for the linear layers: the logits
  # agree to rounding, the greedy tokens almost always)
  assert (alone_t == want_t[:4]).float().mean().item() >= 0.75
