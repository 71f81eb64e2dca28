"""Prompt-pass attention kernel (rg_attention_prefill) against the reference's
op sequence (recurrentgemma/torch/modules.py:444-476: scores in the activation
dtype, scaled, masked with the band of :86-127, softmax in float32,
probabilities back in the activation dtype, weighted sum of the values)
evaluated with float32 tensor ops on the same bf16-valued inputs, and against
the library's attention routine where the mask is one it can take."""

import pytest
import torch

from recurrentgemma_amd import ops
from tests import helpers

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def band(segment_pos, window):
  """first visible key per query, as LocalAttentionBlock computes it."""
  B, T = segment_pos.shape
  pos = torch.arange(T, device=segment_pos.device)[None].expand(B, T)
  start = torch.cummax(torch.where(segment_pos == 0, pos, 0), dim=-1).values
  return torch.maximum(start, pos - window).to(torch.int32)


def reference(q, k, v, segment_pos, window, scale):
  B, T, H, hd = q.shape
  qf, kf, vf = q.float(), k.float().reshape(B, T, hd), v.float().reshape(B, T, hd)
  logits = torch.einsum("bthd,bsd->bhts", qf, kf).to(q.dtype).float() * scale
  pos = torch.arange(T, device=q.device)
  doc = torch.cumsum(segment_pos == 0, dim=-1)
  mask = ((pos[:, None] >= pos[None, :]) &
          (pos[:, None] <= pos[None, :] + window))[None] & (
              doc[:, :, None] == doc[:, None, :])
  logits = torch.where(mask[:, None], logits, torch.finfo(torch.float32).min)
  probs = torch.softmax(logits, dim=-1).to(q.dtype).float()
  return torch.einsum("bhts,bsd->bthd", probs, vf).to(q.dtype)


@pytest.mark.parametrize("B,T,H,window,mean_doc", [
    (1, 1, 1, 2048, None),
    (2, 33, 2, 2048, None),
    (1, 127, 3, 2048, 40),
    (2, 130, 2, 16, None),
    (3, 300, 10, 64, 90),
    (1, 513, 2, 2048, None),
    (2, 1000, 4, 128, 300),
])
def test_attention_prefill_kernel(B, T, H, window, mean_doc):
  hd = 256
  g = torch.Generator().manual_seed(B * 1000 + T)
  q = (torch.randn(B, T, H, hd, generator=g) * 1.5).to(torch.bfloat16).to(DEV)
  k = (torch.randn(B, T, 1, hd, generator=g) * 1.5).to(torch.bfloat16).to(DEV)
  v = torch.randn(B, T, 1, hd, generator=g).to(torch.bfloat16).to(DEV)
  if mean_doc is None:
    seg = torch.arange(T).expand(B, T).clone()
  else:
    seg = helpers.document_positions(B, T, mean_doc, seed=T)
  if T > 2:
    seg[0, 0] = 3  # a row that continues a document
  seg = seg.to(DEV)
  scale = hd ** -0.5
  got = ops.attention_prefill(q, k, v, band(seg, window), scale)
  want = reference(q, k, v, seg, window, scale)
  assert got.shape == want.shape and got.dtype == torch.bfloat16
  helpers.assert_close_elementwise(got, want, rtol=2e-2, atol_of_max=2e-2,
                                   what="attention")


def test_attention_prefill_left_padded_rows():
  """Rows padded on the left with position -1, as the sampler lays out
  prompts of different lengths (sampler.py:234-238): the first real token
  starts the document, the pads before it only see each other."""
  B, T, H, hd, window = 3, 200, 2, 256, 2048
  g = torch.Generator().manual_seed(5)
  q = torch.randn(B, T, H, hd, generator=g).to(torch.bfloat16).to(DEV)
  k = torch.randn(B, T, 1, hd, generator=g).to(torch.bfloat16).to(DEV)
  v = torch.randn(B, T, 1, hd, generator=g).to(torch.bfloat16).to(DEV)
  seg = torch.arange(T).expand(B, T).clone()
  for b, pad in enumerate((0, 37, 150)):
    seg[b] = torch.cat([torch.full((pad,), -1), torch.arange(T - pad)])
  seg = seg.to(DEV)
  got = ops.attention_prefill(q, k, v, band(seg, window), hd ** -0.5)
  want = reference(q, k, v, seg, window, hd ** -0.5)
  for b, pad in enumerate((0, 37, 150)):  # the real tokens
    helpers.assert_close_elementwise(got[b, pad:], want[b, pad:], rtol=2e-2,
                                     atol_of_max=2e-2, what=f"row {b}")


@pytest.mark.parametrize("B,T,H,window", [(2, 257, 10, 2048), (1, 700, 3, 2048),
                                          (2, 400, 4, 96), (1, 1500, 2, 300)])
def test_attention_prefill_against_library_attention(B, T, H, window):
  """The same kernel against the library's own attention routine
  (torch.nn.functional.scaled_dot_product_attention, float32 on the same
  bf16-valued inputs): one document per row; a prompt no longer than the
  window is plain causal attention (is_causal=True, no mask written here),
  a longer one the band `t - window <= s <= t` of modules.py:86-127 as a
  boolean mask.  Tolerance: the bf16 roundings of scores and probabilities
  that the kernel keeps from the reference's op sequence and float32
  attention does not have (2e-2 of the value plus 2e-2 of the largest)."""
  hd = 256
  g = torch.Generator().manual_seed(T + window)
  q = torch.randn(B, T, H, hd, generator=g).to(torch.bfloat16).to(DEV)
  k = torch.randn(B, T, 1, hd, generator=g).to(torch.bfloat16).to(DEV)
  v = torch.randn(B, T, 1, hd, generator=g).to(torch.bfloat16).to(DEV)
  seg = torch.arange(T).expand(B, T).contiguous().to(DEV)
  got = ops.attention_prefill(q, k, v, band(seg, window), hd ** -0.5)
  qf = q.float().transpose(1, 2)                       # [B, H, T, hd]
  kf = k.float().transpose(1, 2).expand(-1, H, -1, -1)
  vf = v.float().transpose(1, 2).expand(-1, H, -1, -1)
  if T <= window + 1:
    want = torch.nn.functional.scaled_dot_product_attention(
        qf, kf, vf, is_causal=True, scale=hd ** -0.5)
  else:
    t = torch.arange(T, device=DEV)
    visible = (t[None, :] <= t[:, None]) & (t[None, :] >= t[:, None] - window)
    want = torch.nn.functional.scaled_dot_product_attention(
        qf, kf, vf, attn_mask=visible, scale=hd ** -0.5)
  want = want.transpose(1, 2)
  helpers.assert_close_elementwise(got, want, rtol=2e-2, atol_of_max=2e-2,
                                   what="attention vs library")


def test_attention_prefill_refuses_other_shapes():
  q = torch.zeros(1, 8, 2, 128, dtype=torch.bfloat16, device=DEV)
  assert not ops.attention_prefill_supported(q)
  assert not ops.attention_prefill_supported(
      torch.zeros(1, 8, 2, 256, device=DEV))
  with pytest.raises(Exception):
    ops.attention_prefill(q, q[:, :, :1], q[:, :, :1],
                          torch.zeros(1, 8, dtype=torch.int32, device=DEV), 1.0)


# ------------------------------------------------ one decoded token --------


def _decode_case(B, heads, window, tokens_seen, seed, ld=None):
  hd = 256
  g = torch.Generator().manual_seed(seed)
  width = (heads + 2) * hd if ld is None else ld
  qkv = (torch.randn(B, width, generator=g) * 1.2).to(torch.bfloat16).to(DEV)
  ring_k = (torch.randn(B, window, hd, generator=g) * 1.2).to(torch.bfloat16)
  ring_v = torch.randn(B, window, hd, generator=g).to(torch.bfloat16)
  nt = torch.tensor(tokens_seen, dtype=torch.int32)
  assert nt.shape == (B,)
  pos = (nt + 3).to(torch.int64)
  return qkv, ring_k.to(DEV), ring_v.to(DEV), nt.to(DEV), pos.to(DEV)


def _decode_separate_calls(qkv, heads, ring_k, ring_v, nt, pos, inv_freq, scale):
  """The same step as the block ran it before: rotary embedding, a batched
  product, the softmax kernel, a second product, the finishing kernel."""
  B, hd = qkv.shape[0], 256
  window = ring_k.shape[1]
  q = qkv[:, :heads * hd].reshape(B, 1, heads, hd).contiguous()
  k = qkv[:, heads * hd:(heads + 1) * hd].reshape(B, 1, 1, hd).contiguous()
  v = qkv[:, (heads + 1) * hd:(heads + 2) * hd].contiguous()
  q, k = ops.rope_pair(q, k, pos.reshape(B, 1), inv_freq)
  qh = q[:, 0]
  scores = torch.bmm(qh, ring_k.transpose(1, 2))
  probs = ops.attention_decode_probs(scores, qh, k[:, 0, 0], nt, scale)
  from_ring = torch.bmm(probs[..., :window], ring_v)
  return ops.attention_decode_finish(from_ring, probs, k[:, 0, 0], v, ring_k,
                                     ring_v, nt, update_cache=True)


@pytest.mark.parametrize("B,heads,window,tokens_seen", [
    (4, 10, 2048, [2048, 5000, 2047, 300]),  # the usual window: wrapped or not
    (5, 10, 512, [0, 1, 15, 16, 17]),        # an empty ring, first passes
    (3, 16, 256, [255, 256, 257]),           # one chunk, sixteen heads
    (2, 1, 300, [299, 301]),                 # a window that is no multiple
    (3, 3, 1024, [64, 65, 700]),             # waves and chunks without a slot
    (2, 2, 16, [3, 40]),                     # a window shorter than a pass
])
def test_attention_decode_fused(B, heads, window, tokens_seen):
  """rg_attention_decode_fused against the separate calls (same roundings up
  to the unnormalised probabilities of a streaming softmax) and against the
  reference's op sequence in float32 tensor ops."""
  hd = 256
  scale = hd ** -0.5
  qkv, ring_k, ring_v, nt, pos = _decode_case(B, heads, window, tokens_seen,
                                              seed=B * 100 + window)
  freq = torch.arange(hd // 4, device=DEV)
  inv_freq = 1.0 / (10000 ** (2 * freq / (hd // 2)))
  assert ops.attention_decode_fused_supported(qkv, heads, hd, window)
  rk1, rv1, nt1 = ring_k.clone(), ring_v.clone(), nt.clone()
  want = _decode_separate_calls(qkv, heads, rk1, rv1, nt1, pos, inv_freq, scale)
  rk2, rv2, nt2 = ring_k.clone(), ring_v.clone(), nt.clone()
  print("[case] decode attention", B, heads, window, tokens_seen, flush=True)
  got = ops.attention_decode_fused(
      qkv[:, :heads * hd], qkv[:, heads * hd:(heads + 1) * hd],
      qkv[:, (heads + 1) * hd:], pos, inv_freq, rk2, rv2, nt2, scale)
  torch.cuda.synchronize()
  assert got.shape == (B, heads, hd) and got.dtype == torch.bfloat16
  # the ring and the count: bit for bit
  assert torch.equal(nt2, nt1) and torch.equal(nt2, nt + 1)
  assert torch.equal(rk2, rk1) and torch.equal(rv2, rv1)
  helpers.assert_close_elementwise(got, want, what="out", rtol=2e-2,
                                   atol_of_max=1e-2)
  # float32 tensor ops on the same values (the rotated q and k of the
  # separate calls; scores rounded as the reference's bf16 product is)
  q = qkv[:, :heads * hd].reshape(B, 1, heads, hd).contiguous()
  k = qkv[:, heads * hd:(heads + 1) * hd].reshape(B, 1, 1, hd).contiguous()
  v = qkv[:, (heads + 1) * hd:].float()
  q, k = ops.rope_pair(q, k, pos.reshape(B, 1), inv_freq)
  keys = torch.cat([ring_k.float(), k[:, 0].float()], dim=1)     # [B, w+1, hd]
  vals = torch.cat([ring_v.float(), v[:, None]], dim=1)
  logits = torch.einsum("bhd,bsd->bhs", q[:, 0].float(), keys)
  logits = (logits.bfloat16().float() * scale).bfloat16().float()
  slot = torch.arange(window, device=DEV)[None]
  seen = (nt[:, None] >= window) | (slot < nt[:, None])
  seen = torch.cat([seen, torch.ones_like(seen[:, :1])], dim=1)
  logits = torch.where(seen[:, None], logits, float("-inf"))
  ref = torch.einsum("bhs,bsd->bhd", torch.softmax(logits, dim=-1), vals)
  helpers.assert_close_elementwise(got, ref, what="out vs float32", rtol=2e-2,
                                   atol_of_max=1e-2)
  # without the update nothing but the output is written
  rk3, rv3, nt3 = ring_k.clone(), ring_v.clone(), nt.clone()
  again = ops.attention_decode_fused(
      qkv[:, :heads * hd].contiguous(),
      qkv[:, heads * hd:(heads + 1) * hd].contiguous(),
      qkv[:, (heads + 1) * hd:].contiguous(), pos.to(torch.int32), inv_freq,
      rk3, rv3, nt3, scale, update_cache=False)
  assert torch.equal(again, got)
  assert torch.equal(rk3, ring_k) and torch.equal(rv3, ring_v)
  assert torch.equal(nt3, nt)


def test_attention_decode_fused_shape_sweep():
  """Seeded random shapes (heads, window, batch, fill of the ring, row
  strides) against the separate calls: output within the bf16 bar, ring and
  count bit for bit."""
  import random
  rnd = random.Random(20240917)
  hd, scale = 256, 256 ** -0.5
  freq = torch.arange(hd // 4, device=DEV)
  inv_freq = 1.0 / (10000 ** (2 * freq / (hd // 2)))
  for case in range(24):
    heads = rnd.choice([1, 2, 4, 7, 10, 16])
    window = rnd.choice([8, 40, 256, 257, 600, 1024, 2048, 4096])
    B = rnd.randint(1, 9)
    seen = [rnd.choice([0, 1, rnd.randint(0, window), window,
                        window + rnd.randint(1, 3 * window)]) for _ in range(B)]
    ld = (heads + 2) * hd + 8 * rnd.randint(0, 5)
    print("[case] decode attention sweep", case, heads, window, B, seen, ld,
          flush=True)
    qkv, ring_k, ring_v, nt, pos = _decode_case(B, heads, window, seen,
                                                seed=1000 + case, ld=ld)
    rk1, rv1, nt1 = ring_k.clone(), ring_v.clone(), nt.clone()
    want = _decode_separate_calls(qkv, heads, rk1, rv1, nt1, pos, inv_freq,
                                  scale)
    rk2, rv2, nt2 = ring_k.clone(), ring_v.clone(), nt.clone()
    got = ops.attention_decode_fused(
        qkv[:, :heads * hd], qkv[:, heads * hd:(heads + 1) * hd],
        qkv[:, (heads + 1) * hd:(heads + 2) * hd], pos, inv_freq, rk2, rv2, nt2,
        scale)
    torch.cuda.synchronize()
    assert torch.equal(nt2, nt1) and torch.equal(rk2, rk1)
    assert torch.equal(rv2, rv1)
    helpers.assert_close_elementwise(got, want, what=f"out, case {case}",
                                     rtol=2e-2, atol_of_max=1e-2)


def test_attention_decode_fused_refuses_what_it_cannot_run():
  x = torch.zeros(2, 12 * 256, dtype=torch.bfloat16, device=DEV)
  assert not ops.attention_decode_fused_supported(x, 17, 256, 2048)
  assert not ops.attention_decode_fused_supported(x, 10, 128, 2048)
  assert not ops.attention_decode_fused_supported(x, 10, 256, 16385)
  assert not ops.attention_decode_fused_supported(x.float(), 10, 256, 2048)
