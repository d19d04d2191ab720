"""RMSNorm: out = x * 1/sqrt(mean(x^2) + eps) * w, eps inside the root
(src/transformer/rmsnorm_scalar.c:4-13).  Computed in float32 whatever the activation
type; the weight is kept in float32."""
from __future__ import annotations

import torch

from .. import ops
from .base import NORMS, ParamSpec, Part
from .linear import upload


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone
    deferrable = True        # a product may fold this norm around itself (weight and eps are all it needs)
    takes_partial_sums = True    # apply() accepts ops.PartialSums as the delta

    def __init__(self, dim: int, eps: float):
        self.dim, self.eps = int(dim), float(eps)
        self.weight = None

    def tensors(self):
        return {"weight": ParamSpec((self.dim,), init="ones")}

    def load(self, tensors, device, dtype):
        self.weight = upload(tensors["weight"], device, torch.float32)

    def apply(self, x, delta, out_dtype, rows=None):
        return ops.add_rmsnorm(x, delta, self.weight, self.eps, out_dtype, rows)
