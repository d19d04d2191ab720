"""A weight matrix [out, in] with an optional bias, applied through ops.linear.  Shared by
the mixers and feed-forwards; not a registered part by itself."""
from __future__ import annotations

import torch

from .. import ops


class Linear:
    def __init__(self):
        self.weight = None
        self.bias = None

    def load(self, weight: torch.Tensor, bias, device, dtype):
        self.weight = weight.to(dtype).to(device).contiguous()
        self.bias = bias.to(torch.float32).to(device).contiguous() if bias is not None else None

    def __call__(self, x: torch.Tensor, out_dtype=None, rows: slice | None = None) -> torch.Tensor:
        w = self.weight if rows is None else self.weight[rows]
        y = ops.linear(x, w, out_dtype)
        if self.bias is not None:
            ops.bias_add(y, self.bias if rows is None else self.bias[rows].contiguous())
        return y
