"""The Python entry point: load a model folder, generate."""
from __future__ import annotations

from typing import Callable, Optional, Sequence

import torch

from .engine import Engine, Request, generate
from .sampling import SamplingParams, sample_batch

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


class LLM:
    def __init__(self, engine: Engine):
        self.engine = engine

    @property
    def config(self):
        return getattr(self.engine, "config", None)

    # the step function under the loop, for callers that bring their own: logits [wanted, vocab] (float32) at the
    # places that the entries (engine.StepEntry(slot, tokens, want)) ask for
    def new_sequence(self) -> int:
        return self.engine.new_sequence()

    def step(self, entries, device_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        return self.engine.step(entries, device_tokens)

    def release(self, slot: int) -> None:
        self.engine.release(slot)

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 256, temperature: float = 0.0,
                 top_p: float = 0.9, seed: int = 42, repeat_penalty: float = 1.0, stop_ids: Optional[Sequence[int]] = None,
                 batch_size: int = 8, on_token: Optional[Callable[[int, int], bool]] = None,
                 return_results: bool = False):
        """Token ids generated for every prompt (lists of token ids).  The options have the
        reference's meaning (-n, --temp, --topp, --seed, --repeat-penalty); every prompt gets
        its own generator seeded with `seed`.  stop_ids None: the configuration's eos ids."""
        if stop_ids is None:
            stop_ids = tuple(self.engine.model.plan.stop_ids)
        params = SamplingParams(temperature=temperature, top_p=top_p, seed=seed, repeat_penalty=repeat_penalty)
        reqs = [Request(list(p), max_new_tokens, params, tuple(stop_ids)) for p in prompts]
        results = generate(self.engine, reqs, sample_batch, batch_size=batch_size, on_token=on_token)
        for r in results:
            if r.finish.startswith("error"):
                raise ValueError(r.finish)
        return results if return_results else [r.tokens for r in results]


def load(folder: str, dtype="bfloat16", max_tokens: int = 8192, device: str = "cuda:0", max_seq_len: int = 0,
         use_graphs: bool = True, n_seqs: int = 1, streamed_weights=None) -> LLM:
    """max_tokens: cached positions of all live sequences together (sizes the cache); 0: room for n_seqs sequences
    of the longest length there can be, or what fits into the device's free memory if that is less.
    max_seq_len: the longest sequence (the reference's --maxseq), 0 = the model's limit.
    streamed_weights: keep every weight matrix a second time in the order the decode kernels read it (faster decode
    steps for the matrices' memory once more); None: as many as fit into what the cache leaves free."""
    if dtype not in _DTYPES:
        raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}")
    return LLM(Engine.from_folder(folder, _DTYPES[dtype], max_tokens, device, max_seq_len, 0, use_graphs, n_seqs,
                                  streamed_weights))
