"""Prompt-pass attention kernel (rg_attention_prefill) against the reference's
op sequence (recurrentgemma/torch/modules.py:444-476: scores in the activation
dtype, scaled, masked with the band of :86-127, softmax in float32,
probabilities back in the activation dtype, weighted sum of the values)
evaluated with float32 tensor ops on the same bf16-valued inputs."""

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


def test_attention_prefill_refuses_other_shapes():
  q = torch.zeros(1, 8, 2, 128, dtype=torch.bfloat16, device=DEV)
  assert not ops.attention_prefill_supported(q)
  assert not ops.attention_prefill_supported(
      torch.zeros(1, 8, 2, 256, device=DEV))
  with pytest.raises(Exception):
    ops.attention_prefill(q, q[:, :, :1], q[:, :, :1],
                          torch.zeros(1, 8, dtype=torch.int32, device=DEV), 1.0)
