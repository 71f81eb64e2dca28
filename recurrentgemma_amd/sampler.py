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
from recurrentgemma_amd import ops


class SamplerOutput(NamedTuple):
  text: list[str]
  logits: list[torch.Tensor]
  tokens: list[torch.Tensor]


def _parameter_stamp(model):
  """Address, version counter and dtype of every parameter: a captured step
  reads re-laid-out copies of the weights made when it was captured, so it is
  only good for as long as this stays the same (no load_state_dict, optimizer
  step, .to() since)."""
  return tuple(ops.tensor_stamp(p) + (p.dtype,) for p in model.parameters())


class _CapturedStep:
  """One cached single-token pass through the model, captured once as a HIP
  graph on fixed buffers (token ids, positions, every block's cache, logits)
  and replayed per generated token: the ~1300 kernel launches of a step cost
  one graph launch.  The caches are updated in place inside the graph, the
  positions advance inside it too.  Token selection stays outside (a reduction
  over the whole vocabulary may clear its scratch with a memset node, which
  must not be recorded into a graph on this platform)."""

  def __init__(self, model, batch_size, dtype, device):
    self.model = model
    self.stamp = _parameter_stamp(model)
    ints = dict(device=device, dtype=torch.int32)
    self.tokens = torch.zeros((batch_size, 1), **ints)
    self.pos = torch.ones((batch_size, 1), **ints)
    self.cache = model.init_cache(batch_size, dtype, device=device)
    self._recurrent = [b.recurrent_block for b in model.blocks
                       if hasattr(b, "recurrent_block")]
    with self._in_place():
      side = torch.cuda.Stream(device=device)
      side.wait_stream(torch.cuda.current_stream(device))
      with torch.cuda.stream(side):
        for _ in range(2):  # library handles, packed weights, allocator pools
          model(self.tokens, self.pos, self.cache)
      torch.cuda.current_stream(device).wait_stream(side)
      self.graph = torch.cuda.CUDAGraph()
      with torch.cuda.graph(self.graph):
        self.logits, _ = model(self.tokens, self.pos, self.cache)
        self.pos.add_(1)

  def _in_place(self):
    blocks = self._recurrent

    class _Ctx:
      def __enter__(self):
        self.old = [b.decode_in_place for b in blocks]
        for b in blocks:
          b.decode_in_place = True

      def __exit__(self, *exc):
        for b, o in zip(blocks, self.old):
          b.decode_in_place = o

    return _Ctx()

  def load(self, cache, pos):
    """Takes over the state a prompt pass left behind."""
    for name, c in cache.items():
      for dst, src in zip(self.cache[name], c):
        dst.copy_(src)
    self.pos.copy_(pos)

  def step(self, tokens):
    self.tokens.copy_(tokens)
    self.graph.replay()
    return self.logits


class Sampler:
  """Sampler for a Griffin model (greedy, or from the categorical
  distribution of the logits).  use_graph: decode steps replay a captured HIP
  graph (same kernels, same results as the eager loop)."""

  def __init__(self, model: griffin_lib.Griffin, vocab=None,
               greedy_sampling: bool = True, is_it_model: bool = False,
               use_graph: bool = False):
    self.model = model
    self.vocab = vocab
    self.greedy_sampling = greedy_sampling
    self.use_graph = use_graph
    self._captured = {}
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
      return ops.argmax_last(logits)
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
    captured = None
    if self.use_graph and total_generation_steps > 2:
      captured = self._captured.get(bsz)
      stamp = _parameter_stamp(model)
      if (captured is None or captured.stamp != stamp or
          any(s[1] is None for s in stamp)):  # (no version counter: recapture)
        captured = self._captured[bsz] = _CapturedStep(model, bsz, self.dtype,
                                                       dev)
      captured.load(cache, pos)
    while total_generation_steps > 1 and step < total - 1 and not done:
      if captured is not None:
        logits = captured.step(tokens_buffer[:, step][:, None])
      else:
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
