"""Weights of a model folder, read by tensor name against what the plan expects.

The plan names every tensor it needs with its shape.  Loading compares that list with
what the files hold and raises ONE error that lists every missing tensor, every
unexpected tensor and every wrong shape (the reference stops at the first missing
tensor, src/model.c:137-140, 541-544, and trusts the file's shapes).  Tensors keep
their stored type on the host: bfloat16 stays bfloat16, a tensor stored in 32 bits stays
so, float16 is widened to float32 losslessly, integer tables become int32.  The parts
cast to their compute types after they upload.  The file is mapped, not read: a tensor on
the host is a view of the map (the reference's BnModel points into its mapped file the same
way and is immutable after load, include/model.h), and a model is uploaded tensor by tensor
without the host ever holding more than what is on its way.
"""
from __future__ import annotations

from collections.abc import Mapping
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


class TensorSource(Mapping):
    """name -> host tensor, for every expected tensor that the folder holds, without holding them: a tensor is
    a view of the mapped file (no copy; float16 and the integer types are converted when they are asked for, one
    tensor at a time), and release(names) lets the pages of tensors that have been uploaded go.  A model is
    loaded tensor by tensor this way and the host never holds more than what is being uploaded (the reference
    maps the file and uploads from the map, src/model.c:147, src/gpu_cuda.cu:11571).  Use as a context manager,
    or close() it; tensors taken from it must not be used after that."""

    def __init__(self, folder: str, files, where):
        self.folder, self._files, self._where = folder, files, where

    def __getitem__(self, name: str) -> torch.Tensor:
        return _host_dtype(self._where[name].view(name))

    def __iter__(self):
        return iter(self._where)

    def __len__(self) -> int:
        return len(self._where)

    def __contains__(self, name) -> bool:
        return name in self._where

    def release(self, names) -> None:
        for n in names:
            f = self._where.get(n)
            if f is not None:
                f.release(n)

    def close(self) -> None:
        for f in self._files:
            f.close()
        self._files, self._where = [], {}

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def open_tensors(folder: str, expected: Dict[str, TensorSpec]) -> TensorSource:
    """Checks what the folder holds against what the plan expects (one WeightError for everything that is missing,
    unexpected, mis-shaped or of a type that no part takes) and returns the tensors as a TensorSource."""
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
        return TensorSource(folder, files, {n: where[n] for n in expected if n in where})
    except BaseException:
        for f in files:
            f.close()
        raise


def load_tensors(folder: str, expected: Dict[str, TensorSpec]) -> Dict[str, torch.Tensor]:
    """name -> host tensor that owns its memory, for every expected tensor that the folder holds: the whole model
    on the host.  For small models and for callers that keep the tensors; a model is loaded through open_tensors."""
    with open_tensors(folder, expected) as src:
        return {n: src[n].clone() for n in src}
