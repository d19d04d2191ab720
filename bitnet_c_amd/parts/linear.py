"""A weight matrix [out, in] with an optional bias, applied through ops.linear.  Shared by
the mixers and feed-forwards; not a registered part by itself."""
from __future__ import annotations

import torch

from .. import ops


def upload(t: torch.Tensor, device, dtype) -> torch.Tensor:
    """A tensor on the device in the compute type: copied up in the type it has (a host tensor may be a view of
    the mapped model file, which is neither converted nor copied on the host) and converted there."""
    return t.to(device).to(dtype).contiguous()      # a tensor that is there already in that type is taken as it is


class Linear:
    def __init__(self):
        self.weight = None
        self.bias = None
        self.streamed = None     # ops.StreamedWeight: the weight once more, in the order the decode kernels read it
        self.stream_tile_rows = None     # rows per tile of that copy; None: what suits the matrix (ops.stream_tile_rows)

    def load(self, weight: torch.Tensor, bias, device, dtype):
        self.weight = upload(weight, device, dtype)
        self.bias = upload(bias, device, torch.float32) if bias is not None else None
        self.streamed = None

    def stream_bytes(self) -> int:
        """Bytes that keep_streamed() would add (0 where the kernels that read a streamed copy do not apply)."""
        w = self.weight
        if w is None or w.dtype != torch.bfloat16 or w.dim() != 2 or not w.is_cuda or w.shape[1] % 8:
            return 0
        R, C = self.stream_tile_rows or ops.stream_tile_rows(w.shape[0]), ops.STREAM_TILE_COLS
        return -(-w.shape[0] // R) * R * -(-w.shape[1] // C) * C * 2

    def keep_streamed(self, keep: bool = True) -> None:
        """Makes (or drops) the streamed copy of the weight, which every product of up to 128 rows then reads."""
        self.streamed = ops.stream_copy(self.weight, self.stream_tile_rows) if keep and self.stream_bytes() else None

    def __call__(self, x, out_dtype=None, rows: slice | None = None) -> torch.Tensor:
        """x: activations, or an ops.DeferredNorm whose norm this product applies itself when it can."""
        w = self.weight if rows is None else self.weight[rows]
        streamed = self.streamed if rows is None else None
        if isinstance(x, ops.DeferredNorm):
            M, (N, K) = x.shape[0], w.shape
            if (self.bias is None and out_dtype in (None, torch.bfloat16) and w.dtype == torch.bfloat16
                    and ops.can_fuse_norm(M, N, K, w.dtype) and w.data_ptr() % 16 == 0):
                return ops.linear_prenorm(x, w, streamed)
            x = x.materialize()
        y = ops.linear(x, w, out_dtype, streamed=streamed)
        if self.bias is not None:
            ops.bias_add(y, self.bias if rows is None else self.bias[rows].contiguous())
        return y

    def lazy(self, x: torch.Tensor):
        """The product in the form in which it reaches a residual stream cheapest (bf16, no bias): a LazyDelta at
        decode sizes, where it can add itself to the stream; partial sums over ranges of K (ops.PartialSums), which the
        kernel of the next norm adds up, where ops.can_split_sums says so; else its result."""
        from .base import LazyDelta
        M, (N, K) = x.shape[0], self.weight.shape
        plain = (self.bias is None and x.dim() == 2 and x.dtype == torch.bfloat16 and self.weight.dtype == torch.bfloat16
                 and x.data_ptr() % 16 == 0 and self.weight.data_ptr() % 16 == 0)
        if plain and ops.can_defer_norm(M, N, K, x.dtype):
            return LazyDelta(x, self)
        if plain and ops.can_split_sums(M, N, K, x.dtype) and x.stride(1) == 1 and x.stride(0) % 8 == 0:
            return ops.linear_partial_sums(x, self.weight, self.streamed)
        return self(x)

    def into_stream(self, x: torch.Tensor, stream: torch.Tensor, norm_weight: torch.Tensor, eps: float):
        """stream += self(x) in one kernel that leaves the next norm deferred; None if the stream does not fit."""
        if tuple(stream.shape) != (x.shape[0], self.weight.shape[0]) or not stream.is_contiguous():
            return None
        return ops.linear_into_stream(x, self.weight, stream, norm_weight, eps, self.streamed)
