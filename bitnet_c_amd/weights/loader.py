"""Weights of a model folder, read by tensor name against what the plan expects.

The plan names every tensor it needs with its shape.  Loading compares that list with
what the files hold and raises ONE error that lists every missing tensor, every
unexpected tensor and every wrong shape (the reference stops at the first missing
tensor, src/model.c:137-140, 541-544, and trusts the file's shapes).  Tensors keep
their stored type on the host: bfloat16 stays bfloat16, a tensor stored in 32 bits stays
so, float16 is widened to float32 losslessly, integer tables become int32.  The parts
cast to their compute types when they upload.  The host copy is immutable after load,
as the reference's BnModel is (include/model.h).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Tuple

import torch

from .safetensors_io import SafetensorsError, open_model_files


class WeightError(ValueError):
    """Missing / unexpected tensors and wrong shapes of a model folder, all in one message."""

    def __init__(self, folder, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shape = sorted(wrong_shape)
        self.wrong_dtype = sorted(wrong_dtype)
        lines = [f"{folder}: the tensors do not match the configuration"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, expected {list(want)}" for n, got, want in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  wrong type ({len(self.wrong_dtype)}): " + ", ".join(
                f"{n} is {dt}" for n, dt in self.wrong_dtype))
        super().__init__("\n".join(lines))


@dataclass(frozen=True)
class TensorSpec:
    """One tensor the plan expects.  `init`: how the random-weights mode fills it."""
    name: str
    shape: Tuple[int, ...]
    init: str = "normal"          # "normal" | "ones" | "zeros"
    optional: bool = False


_FLOATS = (torch.float32, torch.bfloat16, torch.float16, torch.float64)
_INTS = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8)


def _host_dtype(t: torch.Tensor) -> torch.Tensor:
    if t.dtype in (torch.float16, torch.float64):
        return t.to(torch.float32)
    if t.dtype in _INTS and t.dtype != torch.int32:
        return t.to(torch.int32)
    return t


def load_tensors(folder: str, expected: Dict[str, TensorSpec]) -> Dict[str, torch.Tensor]:
    """name -> host tensor for every expected tensor that the folder holds."""
    try:
        files = open_model_files(folder)
    except SafetensorsError as e:
        raise WeightError(folder, [f"(no readable weights: {e})"], [], []) from None
    try:
        where = {}
        for f in files:
            for name in f.names():
                where[name] = f
        missing = [n for n, s in expected.items() if n not in where and not s.optional]
        unexpected = [n for n in where if n not in expected]
        wrong_shape, wrong_dtype = [], []
        for n, s in expected.items():
            if n in where:
                dt, shape = where[n].entries[n]
                if tuple(shape) != tuple(s.shape):
                    wrong_shape.append((n, tuple(shape), tuple(s.shape)))
                if dt not in _FLOATS + _INTS:
                    wrong_dtype.append((n, str(dt)))
        if missing or unexpected or wrong_shape or wrong_dtype:
            raise WeightError(folder, missing, unexpected, wrong_shape, wrong_dtype)
        return {n: _host_dtype(where[n].read(n)) for n in expected if n in where}
    finally:
        for f in files:
            f.close()
