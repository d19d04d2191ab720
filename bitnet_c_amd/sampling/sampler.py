"""Sampling: per-sequence state on the host, the arithmetic over the vocabulary on the GPU.

Options and their meaning are the reference's (src/sampler.c:137-172, src/main.c:224-233):
temperature 0 is argmax; otherwise logits / T, softmax, and a draw with one uniform
number from the sequence's own xorshift64* generator (src/sampler.c:6-15; seed 0 means
42, src/sampler.c:22); top_p in (0, 1) restricts the draw to the nucleus, any other value
draws from the whole vocabulary; a repetition penalty != 1 divides (logit > 0) or
multiplies the logits of the distinct tokens among the last `repeat_window` ones, prompt
tokens included (src/main.c:1648-1650), before the temperature.  Every sequence has its
own generator and ring, so what it samples does not depend on its batch.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence

import torch

from .. import ops

_MASK = (1 << 64) - 1


class XorShift64Star:
    def __init__(self, seed: int):
        self.state = (int(seed) & _MASK) or 42

    def next_u32(self) -> int:
        s = self.state
        s ^= s >> 12
        s ^= (s << 25) & _MASK
        s ^= s >> 27
        self.state = s
        return ((s * 0x2545F4914F6CDD1D) & _MASK) >> 32

    def next_float(self) -> float:
        return (self.next_u32() >> 8) / 16777216.0


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_p: float = 0.9
    seed: int = 42
    repeat_penalty: float = 1.0      # the library default; the command line's default is 1.1
    repeat_window: int = 64

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if self.repeat_penalty <= 0 or self.repeat_window <= 0:
            raise ValueError("repeat_penalty and repeat_window must be positive")


class SequenceSampler:
    """Sampling state of one sequence: its generator and its ring of recent tokens."""

    def __init__(self, params: SamplingParams, prompt: Sequence[int] = ()):
        self.params = params
        self.rng = XorShift64Star(params.seed)
        self.recent: List[int] = []
        if params.repeat_penalty != 1.0:
            for t in prompt:
                self.accept(t)

    def accept(self, token: int) -> None:
        if self.params.repeat_penalty != 1.0:
            self.recent.append(int(token))
            if len(self.recent) > self.params.repeat_window:
                del self.recent[0]


def _sample_rows(logits: torch.Tensor, samplers: Sequence[SequenceSampler]) -> torch.Tensor:
    """One token per row of `logits`, left on the GPU (int32 [B]).  Rows are grouped by their parameters; each group
    is one launch."""
    if logits.shape[0] != len(samplers):
        raise ValueError("one sampler per row of logits")
    groups = {}
    for i, s in enumerate(samplers):
        p = s.params
        groups.setdefault((p.temperature, p.top_p, p.repeat_penalty, p.repeat_window), []).append(i)
    whole = len(groups) == 1
    out = None if whole else torch.empty((len(samplers),), dtype=torch.int32, device=logits.device)
    for (temp, top_p, penalty, window), rows in groups.items():
        sub = logits if whole else logits[rows].contiguous()
        if penalty != 1.0 and any(samplers[i].recent for i in rows):
            # one host tensor for all rows (-1 = empty place), one upload
            rec = torch.tensor([list(samplers[i].recent)[:window] + [-1] * (window - min(window, len(samplers[i].recent)))
                                for i in rows], dtype=torch.int32)
            ops.repeat_penalty_(sub, rec.to(sub.device), penalty)
        uniforms = None
        if temp != 0.0:
            # from pinned memory, so that the upload does not make the host wait for the device
            uniforms = torch.tensor([samplers[i].rng.next_float() for i in rows], dtype=torch.float32)
            uniforms = (uniforms.pin_memory() if sub.is_cuda else uniforms).to(sub.device, non_blocking=True)
        toks = ops.sample(sub, temp, top_p, uniforms)
        if whole:
            return toks
        out[torch.tensor(rows, dtype=torch.long).to(out.device)] = toks
    return out


def sample_batch(logits: torch.Tensor, samplers: Sequence[SequenceSampler]) -> List[int]:
    """One token per row of `logits` ([B, vocab] float32 on the GPU; changed in place when a
    penalty applies)."""
    return [int(t) for t in _sample_rows(logits, samplers).tolist()]


class PendingTokens:
    """Tokens that a sampling launch has left on the device and that are on their way to the host."""

    def __init__(self, device_tokens: torch.Tensor):
        self.device_tokens = device_tokens
        self._host = torch.empty(device_tokens.shape, dtype=device_tokens.dtype, pin_memory=device_tokens.is_cuda)
        self._host.copy_(device_tokens, non_blocking=True)
        self._arrived = torch.cuda.Event() if device_tokens.is_cuda else None
        if self._arrived is not None:
            self._arrived.record()

    def rows(self, indices: Sequence[int]) -> torch.Tensor:
        """device_tokens of the given rows, still on the device."""
        idx = torch.tensor(list(indices), dtype=torch.long)
        return self.device_tokens[(idx.pin_memory() if self.device_tokens.is_cuda else idx).to(self.device_tokens.device,
                                                                                           non_blocking=True)]

    def tokens(self) -> List[int]:
        """Waits for the copy (not for anything queued after it)."""
        if self._arrived is not None:
            self._arrived.synchronize()
        return [int(t) for t in self._host.tolist()]


def start_sampling(logits: torch.Tensor, samplers: Sequence[SequenceSampler]):
    """sample_batch without the wait: queues the sampling and the tokens' copy to the host and returns PendingTokens,
    whose device_tokens a decode step can consume (Engine.step(..., device_tokens=...)) before the host has seen them.
    None when a sequence's penalty needs the host's list of recent tokens first: then sample_batch is the way."""
    if any(s.params.repeat_penalty != 1.0 for s in samplers):
        return None
    return PendingTokens(_sample_rows(logits, samplers))


sample_batch.start = start_sampling
