"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.  The reference has no such mode (its tests need real model
files); the distribution is the one its benchmark configurations name: every matrix
N(0, 0.02), every norm weight 1.

Each tensor is drawn from its own generator, seeded by (seed, tensor name), so a tensor's
values depend on nothing but the seed, its name and its shape.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict

import torch

from .loader import TensorSpec
from .safetensors_io import write_file

STD = 0.02


def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & ((1 << 63) - 1)


def random_tensors(expected: Dict[str, TensorSpec], seed: int, dtype=torch.bfloat16, device="cpu",
                   include_optional: bool = False) -> Dict[str, torch.Tensor]:
    """Tensors for every spec.  Matrices are drawn in float32 and rounded once to `dtype`;
    norm weights are float32 ones."""
    out = {}
    for name, spec in expected.items():
        if spec.optional and not include_optional:
            continue
        if spec.init == "ones":
            out[name] = torch.ones(spec.shape, dtype=torch.float32, device=device)
        elif spec.init == "zeros":
            out[name] = torch.zeros(spec.shape, dtype=torch.float32, device=device)
        elif spec.init == "normal":
            g = torch.Generator(device=device)
            g.manual_seed(_tensor_seed(seed, name))
            t = torch.empty(spec.shape, dtype=torch.float32, device=device)
            t.normal_(0.0, STD, generator=g)
            out[name] = t.to(dtype)
        else:
            raise ValueError(f"tensor {name}: unknown init {spec.init!r}")
    return out


def write_model_folder(folder: str, config, seed: int, dtype=torch.bfloat16) -> str:
    """config: a typed configuration of a registered architecture."""
    from ..config.base import architecture_for
    if isinstance(dtype, str):
        dtype = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32,
                 "fp32": torch.float32}[dtype]
    raw = config.to_dict()
    arch = architecture_for(raw)
    plan = arch.build_plan(config)
    os.makedirs(folder, exist_ok=True)
    raw["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32"}.get(dtype, str(dtype))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f, indent=1)
    tensors = random_tensors(plan.expected_tensors(), seed, dtype)
    write_file(os.path.join(folder, "model.safetensors"), tensors,
               metadata={"format": "pt", "seed": seed, "init": f"normal(0,{STD}); norms 1"})
    return folder
