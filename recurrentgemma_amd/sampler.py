"""Autoregressive sampling from a Griffin model.

Follows recurrentgemma/torch/sampler.py:70-434: prompts are left-padded to a
common length, pad positions are -1 (not a document boundary, so the first
real token, position 0, resets the recurrent state and cuts the conv), the
prompt is processed as T-1 tokens without logits plus one cached step for the
last token, then one cached step per generated token with positions
last+1, last+2, ...  `Sampler.__call__` keeps the reference's string interface
(any vocabulary object with EncodeAsIds / DecodeIds / bos_id / eos_id /
pad_id); `sample_tokens` is the same loop on token ids for callers that have
no vocabulary (benchmarks, tests).
"""

from __future__ import annotations

from collections.abc import Sequence
from typing import NamedTuple

import torch

from recurrentgemma_amd import griffin as griffin_lib


class SamplerOutput(NamedTuple):
  text: list[str]
  logits: list[torch.Tensor]
  tokens: list[torch.Tensor]


class Sampler:
  """Sampler for a Griffin model (greedy, or from the categorical
  distribution of the logits)."""

  def __init__(self, model: griffin_lib.Griffin, vocab=None,
               greedy_sampling: bool = True, is_it_model: bool = False):
    self.model = model
    self.vocab = vocab
    self.greedy_sampling = greedy_sampling
    self._is_it_model = is_it_model
    self._eos_token = (None if vocab is None else torch.tensor(
        [vocab.eos_id()], device=self.device))

  @property
  def dtype(self) -> torch.dtype:
    return next(self.model.parameters()).dtype

  @property
  def device(self) -> torch.device:
    return next(self.model.parameters()).device

  @property
  def vocab_size(self) -> int:
    return self.model.config.vocab_size

  def _pick(self, logits):
    if self.greedy_sampling:
      return torch.argmax(logits, dim=-1)
    return torch.distributions.Categorical(logits=logits).sample()

  @torch.no_grad()
  def sample_tokens(self, padded_tokens, input_lengths,
                    total_generation_steps: int, echo: bool = False,
                    return_logits: bool = False, eos_token=None,
                    pad_id: int = 0):
    """The sampling loop on token ids.

    padded_tokens [B, L] int, left-padded; input_lengths [B] real lengths.
    Returns (tokens_buffer [B, steps (+L with echo)], logits_buffer | None).
    Stops early only when `eos_token` (a 1-element tensor) is given and a step
    produces exactly that tensor for the whole batch, like the reference
    (sampler.py:176-179 compares with torch.equal).
    """
    dev = self.device
    ints = dict(device=dev, dtype=torch.int32)
    bsz, plen = padded_tokens.shape
    positions = torch.arange(plen, **ints)[None].expand(bsz, plen)
    positions = positions - plen + input_lengths[:, None].to(**ints)
    positions = torch.clip(positions, min=-1)
    model = self.model

    prev_logits = logits = cache = None
    if total_generation_steps == 0:
      prev_logits, _ = model(padded_tokens, positions, None,
                             return_logits=return_logits and echo,
                             return_cache=False)
    elif plen == 1:
      logits, cache = model(padded_tokens, positions, None,
                            return_logits=True, return_cache=True)
      prev_logits = logits[:, :0]
    else:
      # the logits of the first L-1 prompt tokens are never formed unless
      # they are asked for
      prev_logits, cache = model(padded_tokens[:, :-1], positions[:, :-1],
                                 None, return_logits=return_logits and echo,
                                 return_cache=True)
      logits, cache = model(padded_tokens[:, -1:], positions[:, -1:], cache,
                            return_logits=True,
                            return_cache=total_generation_steps > 1)

    tokens_buffer = torch.full((bsz, total_generation_steps), pad_id, **ints)
    logits_buffer = None
    if logits is not None:
      tokens_buffer[:, 0] = self._pick(logits[:, 0])
    if return_logits:
      logits_buffer = torch.zeros(
          (bsz, total_generation_steps, self.vocab_size), dtype=self.dtype,
          device=dev)
      if logits is not None:
        logits_buffer[:, 0] = logits[:, 0]
    step, total = 0, total_generation_steps
    if echo:
      tokens_buffer = torch.cat([padded_tokens.to(**ints), tokens_buffer], 1)
      if return_logits:
        logits_buffer = (prev_logits if logits is None else torch.cat(
            [prev_logits, logits, logits_buffer], dim=1))
      step, total = step + plen, total + plen

    pos = positions[:, -1:] + 1
    done = False
    while total_generation_steps > 1 and step < total - 1 and not done:
      logits, cache = model(tokens_buffer[:, step][:, None], pos, cache,
                            return_logits=True, return_cache=True)
      nxt = self._pick(logits[:, 0])
      tokens_buffer[:, step + 1] = nxt
      if logits_buffer is not None:
        logits_buffer[:, step + 1] = logits[:, 0]
      if eos_token is not None:
        done = torch.equal(nxt, eos_token)
      step, pos = step + 1, pos + 1
    return tokens_buffer, logits_buffer

  def tokenize(self, input_string: str) -> torch.Tensor:
    if self._is_it_model:
      input_string = (f"<start_of_turn>user\n{input_string}<end_of_turn>\n"
                      "<start_of_turn>model\n")
    ids = [self.vocab.bos_id()] + self.vocab.EncodeAsIds(input_string)
    return torch.tensor(ids, dtype=torch.int32, device=self.device)

  @torch.no_grad()
  def __call__(self, input_strings: Sequence[str], total_generation_steps: int,
               echo: bool = False, return_logits: bool = False,
               end_sampling_at_eos_token: bool = True) -> SamplerOutput:
    if total_generation_steps < 0:
      raise ValueError("total_generation_steps must be at least 0.")
    ids = [self.tokenize(s) for s in input_strings]
    lengths = torch.tensor([len(t) for t in ids], device=self.device,
                           dtype=torch.int32)
    longest = int(lengths.max())
    pad = self.vocab.pad_id()
    padded = torch.stack([
        torch.cat([t.new_full([longest - len(t)], pad), t]) for t in ids])
    tokens, logits = self.sample_tokens(
        padded, lengths, total_generation_steps, echo=echo,
        return_logits=return_logits,
        eos_token=self._eos_token if end_sampling_at_eos_token else None,
        pad_id=pad)
    pads = (longest - lengths).tolist()
    tokens = [row[p:] for row, p in zip(tokens, pads)]
    logits = ([row[p:] for row, p in zip(logits, pads)]
              if return_logits else [])
    return SamplerOutput(
        text=[self.vocab.DecodeIds(t.tolist()) for t in tokens],
        tokens=tokens, logits=logits)
