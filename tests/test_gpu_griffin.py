"""The residual stack and the sampler around the recurrent block, on the GPU,
against vectors written by the reference model itself
(tests/golden/make_griffin_golden.py; float32, tiny shapes).  Tolerance: 2e-4
of the largest reference magnitude per tensor (GPU vs CPU float32 matmuls and
softmax); sampled tokens must be identical."""

import os

import numpy as np
import pytest
import torch

from recurrentgemma_amd import griffin as G
from recurrentgemma_amd import sampler as S

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "griffin_golden.npz")
TOL = 2e-4


@pytest.fixture(scope="module")
def golden():
  return np.load(GOLDEN)


@pytest.fixture(scope="module")
def model(golden):
  R, A = G.TemporalBlockType.RECURRENT, G.TemporalBlockType.ATTENTION
  cfg = G.GriffinConfig(
      vocab_size=48, width=32, mlp_expanded_width=40, num_heads=2,
      block_types=(R, A, R), embeddings_scale_by_sqrt_dim=True,
      attention_window_size=6, logits_soft_cap=30.0, lru_width=64)
  m = G.Griffin(cfg, dtype=torch.float32)
  sd = {k[len("param/"):]: torch.from_numpy(golden[k])
        for k in golden.files if k.startswith("param/")}
  assert set(sd) == set(m.state_dict()), set(sd) ^ set(m.state_dict())
  m.load_state_dict(sd)  # the reference's own keys and shapes
  return m.to(DEV).eval()


def close(got, want, what):
  want = torch.from_numpy(np.asarray(want))
  got = got.detach().cpu()
  assert got.shape == want.shape, (what, got.shape, want.shape)
  if want.numel() == 0:  # the reference cuts pad_length leading entries
    return
  if want.dtype in (torch.int32, torch.int64):
    assert torch.equal(got.to(want.dtype), want), what
    return
  err = (got.float() - want.float()).abs().max().item()
  scale = max(want.float().abs().max().item(), 1e-6)
  assert err <= TOL * scale, (what, err, scale)


def check_cache(cache, golden, prefix):
  names = [k for k in golden.files if k.startswith(prefix + "/")]
  assert names
  for k in names:
    block, field = k[len(prefix) + 1:].split("/")
    close(getattr(cache[block], field), golden[k], k)


def dev(a, dtype=None):
  t = torch.from_numpy(np.asarray(a)).to(DEV)
  return t if dtype is None else t.to(dtype)


def test_forward_left_padded_then_step(model, golden):
  logits, cache = model(dev(golden["c1/tokens"]), dev(golden["c1/pos"]))
  close(logits, golden["c1/logits"], "c1/logits")
  check_cache(cache, golden, "c1/cache")
  assert isinstance(cache["blocks.0"], G.modules.RecurrentBlockCache)
  assert isinstance(cache["blocks.1"], G.AttentionBlockCache)
  logits2, cache2 = model(dev(golden["c1/next_tokens"]),
                          dev(golden["c1/next_pos"]), cache)
  close(logits2, golden["c1/next_logits"], "c1/next_logits")
  check_cache(cache2, golden, "c1/next_cache")


def test_prompt_longer_than_window_then_steps(model, golden):
  pos = dev(golden["c2/pos"])
  logits, cache = model(dev(golden["c2/tokens"]), pos)
  close(logits, golden["c2/logits"], "c2/logits")
  check_cache(cache, golden, "c2/cache")
  steps = dev(golden["c2/step_tokens"])
  p = pos[:, -1:] + 1
  for i in range(3):
    lg, cache = model(steps[:, i:i + 1], p, cache)
    close(lg, golden[f"c2/step{i}_logits"], f"c2/step{i}")
    p = p + 1
  check_cache(cache, golden, "c2/final_cache")


def test_flags(model, golden):
  tokens, pos = dev(golden["c1/tokens"]), dev(golden["c1/pos"])
  assert model(tokens, pos, return_logits=False, return_cache=False) == (None,
                                                                         None)
  logits, cache = model(tokens, pos, return_cache=False)
  assert cache is None
  close(logits, golden["c1/logits"], "no-cache logits")
  none, cache = model(tokens, pos, return_logits=False)
  assert none is None
  check_cache(cache, golden, "c1/cache")
  empty = model.init_cache(2, torch.float32)
  assert set(empty) == {"blocks.0", "blocks.1", "blocks.2"}
  assert empty["blocks.1"].keys.shape == (2, 6, 1, 16)
  assert empty["blocks.0"].rg_lru_state.shape == (2, 64)


class ToyVocab:
  def bos_id(self): return 2
  def eos_id(self): return 1
  def pad_id(self): return 0
  def EncodeAsIds(self, s): return [int(t) for t in s.split()]
  def DecodeIds(self, ids): return " ".join(str(i) for i in ids)


@pytest.mark.parametrize("echo", [False, True])
def test_sampler_matches_reference(model, golden, echo):
  smp = S.Sampler(model, ToyVocab(), greedy_sampling=True)
  prompts = [str(p) for p in golden["c3/prompts"]]
  res = smp(prompts, total_generation_steps=6, echo=echo, return_logits=True,
            end_sampling_at_eos_token=False)
  tag = "c3/echo" if echo else "c3/plain"
  assert res.text == [str(t) for t in golden[f"{tag}/text"]]
  for i in range(len(prompts)):
    close(res.tokens[i], golden[f"{tag}/tokens{i}"], f"{tag}/tokens{i}")
    close(res.logits[i], golden[f"{tag}/logits{i}"], f"{tag}/logits{i}")


def test_sample_tokens_without_vocab(model, golden):
  smp = S.Sampler(model)
  toks = torch.tensor([[0, 0, 2, 7, 40, 3], [2, 5, 9, 13, 21, 8]], device=DEV,
                      dtype=torch.int32)
  lens = torch.tensor([4, 6], device=DEV, dtype=torch.int32)
  out, logits = smp.sample_tokens(toks, lens, 5)
  assert out.shape == (2, 5) and logits is None
  # the same prompts one at a time (no padding) give the same continuation
  for r in range(2):
    single, _ = smp.sample_tokens(toks[r:r + 1, 6 - int(lens[r]):],
                                  lens[r:r + 1], 5)
    assert torch.equal(single[0], out[r])


def test_sampling_from_the_distribution(model):
  """greedy_sampling=False draws from the categorical distribution of the
  logits (sampler.py:129-131): reproducible under a seed, tokens in range, and
  with one logit far above the rest the draw is that token."""
  smp = S.Sampler(model, greedy_sampling=False)
  toks = torch.tensor([[2, 7, 40, 3]], device=DEV, dtype=torch.int32)
  lens = torch.tensor([4], device=DEV, dtype=torch.int32)
  torch.manual_seed(123)
  a, _ = smp.sample_tokens(toks, lens, 6)
  torch.manual_seed(123)
  b, _ = smp.sample_tokens(toks, lens, 6)
  assert torch.equal(a, b)
  assert a.shape == (1, 6) and int(a.min()) >= 0 and int(a.max()) < 48
  peaked = torch.full((3, 48), -50.0, device=DEV)
  peaked[0, 5] = peaked[1, 47] = peaked[2, 0] = 50.0
  assert smp._pick(peaked).tolist() == [5, 47, 0]


def _bf16_model():
  """Three blocks with 256-wide heads in bf16: the shapes that take the
  single-launch decode kernel on packed weights."""
  R, A = G.TemporalBlockType.RECURRENT, G.TemporalBlockType.ATTENTION
  cfg = G.GriffinConfig(
      vocab_size=512, width=512, mlp_expanded_width=768, num_heads=2,
      block_types=(R, R, A), embeddings_scale_by_sqrt_dim=True,
      attention_window_size=16, logits_soft_cap=30.0, lru_width=512)
  torch.manual_seed(11)
  return G.Griffin(cfg, device=DEV, dtype=torch.bfloat16).eval()


@pytest.mark.parametrize("which", ["f32_tiny", "bf16_packed"])
def test_captured_decode_step_equals_eager(model, which):
  """Every replay of the captured step is compared with the eager loop: the
  same tokens and bit-identical logits, over enough steps for the attention
  ring to wrap, on two generations in a row (the second reuses the graph on
  new state), with eager work and synchronisations between replays."""
  m = model if which == "f32_tiny" else _bf16_model()
  vocab = m.config.vocab_size
  g = torch.Generator().manual_seed(3)
  eager, graphed = S.Sampler(m), S.Sampler(m, use_graph=True)
  for round_ in range(2):
    toks = torch.randint(3, vocab, (3, 9), generator=g).to(DEV, torch.int32)
    toks[1, :4] = 0
    lens = torch.tensor([9, 5, 9], device=DEV, dtype=torch.int32)
    want_t, want_l = eager.sample_tokens(toks, lens, 24, return_logits=True)
    got_t, got_l = graphed.sample_tokens(toks, lens, 24, return_logits=True)
    torch.cuda.synchronize()
    assert torch.equal(got_t, want_t), round_
    assert torch.equal(got_l, want_l), round_
  assert len(graphed._captured) == 1
  # the modules are back to returning new cache tensors
  assert not any(b.recurrent_block.decode_in_place for b in m.blocks
                 if hasattr(b, "recurrent_block"))


def test_captured_step_is_redone_after_a_weight_update():
  """A captured step reads re-laid-out copies of the weights taken at capture
  time: after the parameters are written in place the sampler must capture
  again, not replay a graph that mixes old packed and new plain weights."""
  m = _bf16_model()
  g = torch.Generator().manual_seed(5)
  toks = torch.randint(3, 512, (2, 7), generator=g).to(DEV, torch.int32)
  lens = torch.tensor([7, 7], device=DEV, dtype=torch.int32)
  graphed = S.Sampler(m, use_graph=True)
  _, before = graphed.sample_tokens(toks, lens, 10, return_logits=True)
  first = graphed._captured[2]
  with torch.no_grad():
    for p in m.parameters():
      if p.dim() >= 2:
        p.mul_(0.5)  # the logits change
  want_t, want_l = S.Sampler(m).sample_tokens(toks, lens, 10, return_logits=True)
  got_t, got_l = graphed.sample_tokens(toks, lens, 10, return_logits=True)
  assert graphed._captured[2] is not first
  assert torch.equal(got_t, want_t) and torch.equal(got_l, want_l)
  assert not torch.equal(got_l, before)
  # inference-mode tensors (no version counter) are accepted everywhere
  with torch.inference_mode():
    toks_i = toks.clone()
    out_i, _ = S.Sampler(m).sample_tokens(toks_i, lens.clone(), 4)
  assert torch.equal(out_i, want_t[:, :4])


def test_stack_refuses_to_run_where_gradients_are_expected():
  m = _bf16_model()
  toks = torch.randint(3, 512, (1, 4)).to(DEV, torch.int32)
  pos = torch.arange(4, device=DEV)[None]
  # the way the reference's own tests call a model: not switched to eval(),
  # gradients enabled -- computes, like under no_grad
  m.train()
  logits, _ = m(toks, pos)
  assert not logits.requires_grad
  with torch.no_grad():
    again, _ = m(toks, pos)
  assert torch.equal(logits, again)
  m.eval()
  # asked for gradients: an input that requires grad, or the differentiable
  # path switched on
  blk = m.blocks[0]
  x = torch.randn(1, 4, m.config.width, device=DEV,
                  dtype=torch.bfloat16).requires_grad_(True)
  with pytest.raises(NotImplementedError, match="forward only"):
    blk(x, pos)
  from recurrentgemma_amd import training
  with training.differentiable():
    with pytest.raises(NotImplementedError, match="forward only"):
      m(toks, pos)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hd", [16, 64, 256])
def test_rope_kernel(dtype, hd):
  """rg_rope against the reference's tensor expression (modules.py:52-83)
  evaluated by torch on the GPU in the same dtype: bit-identical (the same
  float32 table, sin/cos of the same angles, the same roundings)."""
  from recurrentgemma_amd import ops
  gen = torch.Generator().manual_seed(hd)
  x = torch.randn(3, 7, 2, hd, generator=gen).to(dtype).to(DEV)
  pos = torch.tensor([[-1, -1, 0, 1, 2, 3, 4], [0, 1, 2, 0, 1, 2, 3],
                      [2040, 2041, 2042, 2043, 2044, 2045, 2046]], device=DEV)
  inv = G._inv_frequencies(hd, DEV)
  half = hd // 2
  rot, keep = x[..., :half], x[..., half:]
  angle = pos.reshape(3, 7, 1, 1) * inv
  sin, cos = torch.sin(angle).type_as(x), torch.cos(angle).type_as(x)
  lo, hi = torch.chunk(rot, 2, dim=-1)
  want = torch.cat([lo * cos - hi * sin, hi * cos + lo * sin, keep], dim=-1)
  for p in (pos, pos.to(torch.int32)):
    got = ops.rope(x, p, inv)
    assert torch.equal(got, want), (got - want).abs().max()
  # queries and keys in one launch: each as on its own
  k = torch.randn(3, 7, 1, hd, generator=gen).to(dtype).to(DEV)
  q2, k2 = ops.rope_pair(x, k, pos, inv)
  assert torch.equal(q2, want) and torch.equal(k2, ops.rope(k, pos, inv))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,heads,hd,window", [(2, 2, 16, 6), (5, 10, 256, 64),
                                               (3, 4, 64, 300)])
def test_attention_decode_kernels(dtype, B, heads, hd, window):
  """The decode step of the attention block (scores product + the two
  kernels + values product) against the reference's formulation
  (modules.py:440-474: concatenate the ring and the new key/value, mask from
  the ring positions, float32 softmax) evaluated by torch on the GPU, for a
  ring that is empty, partly filled, exactly full and wrapped.  fp32: 1e-5 of
  the largest magnitude; bf16: 2e-2 (sum of the ring part and the new token's
  part rounded separately).  Ring and token count must be updated exactly."""
  from recurrentgemma_amd import ops
  gen = torch.Generator().manual_seed(B * 1000 + window)
  tol = 1e-5 if dtype == torch.float32 else 2e-2
  nts = torch.tensor(([0, 3, window, 2 * window + 5, window - 1] * B)[:B],
                     dtype=torch.int32, device=DEV)
  q = torch.randn(B, heads, hd, generator=gen).to(dtype).to(DEV)
  kn = torch.randn(B, hd, generator=gen).to(dtype).to(DEV)
  vn = torch.randn(B, hd, generator=gen).to(dtype).to(DEV)
  rk = torch.randn(B, window, hd, generator=gen).to(dtype).to(DEV)
  rv = torch.randn(B, window, hd, generator=gen).to(dtype).to(DEV)
  scale = hd ** -0.5
  # reference formulation
  n = nts[:, None].long()
  slot = torch.arange(window, device=DEV)[None]
  now = slot + (n // window) * window
  k_pos = torch.where(now < n, now, now - window)
  k_pos = torch.cat([k_pos, n], dim=-1)                       # [B, w+1]
  mask = (n >= k_pos) & (n <= k_pos + window) & (k_pos >= 0)
  keys = torch.cat([rk, kn[:, None]], dim=1)
  vals = torch.cat([rv, vn[:, None]], dim=1)
  logits = torch.einsum("bnh,bsh->bns", q, keys) * scale
  logits = torch.where(mask[:, None], logits, -2.3819763e38).float()
  p = torch.softmax(logits, dim=-1).type_as(q)
  want = torch.einsum("bns,bsh->bnh", p, vals)
  # kernels
  k2, v2, nt2 = rk.clone(), rv.clone(), nts.clone()
  scores = torch.bmm(q, k2.transpose(1, 2))
  probs = ops.attention_decode_probs(scores, q, kn, nt2, scale)
  assert helpers_max_rel(probs, p) < tol
  out = ops.attention_decode_finish(torch.bmm(probs[..., :window], v2), probs,
                                    kn, vn, k2, v2, nt2, update_cache=True)
  assert helpers_max_rel(out, want) < tol
  assert torch.equal(nt2, nts + 1)
  rows = torch.arange(B, device=DEV)
  exp_k, exp_v = rk.clone(), rv.clone()
  exp_k[rows, (nts % window).long()] = kn
  exp_v[rows, (nts % window).long()] = vn
  assert torch.equal(k2, exp_k) and torch.equal(v2, exp_v)
  # without the cache update nothing is written
  k3, v3, nt3 = rk.clone(), rv.clone(), nts.clone()
  out3 = ops.attention_decode_finish(torch.bmm(probs[..., :window], v3), probs,
                                     kn, vn, k3, v3, nt3, update_cache=False)
  assert torch.equal(out3, out) and torch.equal(k3, rk) and torch.equal(nt3, nts)


def helpers_max_rel(got, want):
  got, want = got.float(), want.float()
  return ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_soft_cap_kernel(dtype):
  """rg_soft_cap against torch's own three kernels on the GPU (quotient by a
  scalar, tanh, product): same roundings; one unit in the last place is left
  for the tanh of two builds of the device math library."""
  from recurrentgemma_amd import ops
  gen = torch.Generator().manual_seed(77)
  x = (torch.randn(3, 5, 1003, generator=gen) * 40).to(dtype).to(DEV)
  got = ops.soft_cap(x, 30.0)
  want = torch.tanh(x / 30.0) * 30.0
  assert got.dtype == dtype and got.shape == x.shape
  ulp = torch.finfo(dtype).eps * want.float().abs().clamp_min(1e-30)
  assert ((got.float() - want.float()).abs() <= ulp).all()
  assert (got.float().abs() <= 30.0).all()
  mism = (got != want).float().mean().item()
  assert mism < 0.02, mism


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_argmax_kernel(dtype):
  """rg_argmax_rows against torch.argmax: bf16 rows of a vocabulary's length
  are full of equal maxima (first index wins), plus rows with a NaN, a row
  whose maximum is its last element, negative rows."""
  from recurrentgemma_amd import ops
  gen = torch.Generator().manual_seed(78)
  x = torch.randn(9, 25601, generator=gen).to(dtype)
  x[1] = -x[1].abs() - 1.0
  x[2, -1] = 100.0
  x[3, 17] = float("nan")
  x[4, 5] = x[4, 20000] = 50.0
  x[5] = 0.0
  x = x.to(DEV)
  got = ops.argmax_last(x)
  assert got.dtype == torch.int64
  assert torch.equal(got, torch.argmax(x, dim=-1))
  assert got[2].item() == 25600 and got[3].item() == 17 and got[4].item() == 5
  x3 = x[:8].reshape(2, 4, -1)
  assert torch.equal(ops.argmax_last(x3), torch.argmax(x3, dim=-1))
  odd = x[:, 1:100]  # rows that are neither contiguous nor 16-byte aligned
  assert torch.equal(ops.argmax_last(odd), torch.argmax(odd, dim=-1))


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4),
                                       (torch.bfloat16, 3e-2)])
def test_prompt_attention_causal_shortcut(monkeypatch, dtype, tol):
  """Rows that are one document inside the window take the library's causal
  attention instead of the explicit mask: same logits and cache (to the
  tolerance of the dtype); a row with a second document start, or a prompt
  longer than the window, keeps the mask."""
  R, A = G.TemporalBlockType.RECURRENT, G.TemporalBlockType.ATTENTION
  cfg = G.GriffinConfig(
      vocab_size=64, width=64, mlp_expanded_width=96, num_heads=2,
      block_types=(A, R, A), embeddings_scale_by_sqrt_dim=True,
      attention_window_size=16, logits_soft_cap=30.0, lru_width=64)
  torch.manual_seed(9)
  m = G.Griffin(cfg, dtype=dtype).to(DEV).eval()
  gen = torch.Generator().manual_seed(10)
  B, T = 3, 12
  tokens = torch.randint(0, 64, (B, T), generator=gen).to(DEV)
  asked = []
  real = G._rows_are_one_document

  def spy(segment_pos):
    asked.append(real(segment_pos))
    return asked[-1]

  def forced_off(segment_pos):
    return False

  def run(pos, fn):
    monkeypatch.setattr(G, "_rows_are_one_document", fn)
    return m(tokens[:, :pos.shape[1]], pos, None, return_logits=True,
             return_cache=True)

  one_doc = torch.arange(T, device=DEV)[None].expand(B, -1).contiguous()
  one_doc[1] += 5  # a row that continues a document
  logits, cache = run(one_doc, spy)
  assert asked == [True, True]
  want, want_cache = run(one_doc, forced_off)
  scale = want.float().abs().max().item()
  assert (logits.float() - want.float()).abs().max().item() <= tol * scale
  for name in cache:
    for got_t, want_t in zip(cache[name], want_cache[name]):
      s = max(want_t.float().abs().max().item(), 1e-6)
      assert (got_t.float() - want_t.float()).abs().max().item() <= tol * s
  # a second document start in one row: the mask path, bit for bit
  two_docs = one_doc.clone()
  two_docs[2, 7:] = torch.arange(T - 7, device=DEV)
  asked.clear()
  got2, _ = run(two_docs, spy)
  assert asked == [False, False]
  assert torch.equal(got2, run(two_docs, forced_off)[0])
