"""Position encodings.  The attention mixer hands its projected Q, K, V to the encoding,
which encodes Q and K and stores K and V in the cache (the cache holds encoded keys, as
the reference's does: src/transformer/cpu.c:893-898).

"rope": split-half rotary pairs (i, i + rope_dims/2), angle = pos * f_i with
f_i = theta^(-2i/rope_dims) (src/transformer/cpu_backend.c:283-296,
src/model_arch.c:322-338); the f_i are computed once in double and rounded to float32,
and the kernel forms angle, cos and sin in float32.  The reference rescales no
frequencies on this path; the "llama3" rescaling is written from its definition:
wavelengths below orig/high_freq_factor stay, those above orig/low_freq_factor are
divided by `factor`, those between are interpolated linearly in orig/wavelength.

"none": no encoding; K and V are stored as they are.
"""
from __future__ import annotations

import math

import torch

from .. import ops
from .base import POSITION_ENCODINGS, Part


def rope_frequencies(rope_dims: int, theta: float, scaling: dict | None = None) -> torch.Tensor:
    i = torch.arange(rope_dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * i / rope_dims)
    if scaling:
        kind = scaling.get("rope_type")
        if kind == "llama3":
            factor = float(scaling["factor"])
            low, high = float(scaling["low_freq_factor"]), float(scaling["high_freq_factor"])
            orig = float(scaling["original_max_position_embeddings"])
            wavelen = 2.0 * math.pi / f
            smooth = (orig / wavelen - low) / (high - low)
            mid = (1.0 - smooth) * f / factor + smooth * f
            f = torch.where(wavelen < orig / high, f, torch.where(wavelen > orig / low, f / factor, mid))
        elif kind not in (None, "default"):
            raise ValueError(f"position encoding: unknown frequency scaling {kind!r}")
    return f.to(torch.float32)


class PositionEncoding(Part):
    rope_dims = 0
    inv_freq = None

    def prepare(self, device) -> None:
        pass

    def fusable(self, hs: int):
        """(ok, inv_freq or None): whether a decode attention kernel may do this encoding and the
        cache write itself: a rotation of the whole head with these frequencies, or none."""
        if self.rope_dims == 0:
            return True, None
        return self.rope_dims == hs, self.inv_freq

    def encode_and_store(self, qkv, ctx, H, Hkv, hs, kv) -> None:
        ops.rope_kv_write(qkv, ctx.positions, H, Hkv, hs, inv_freq=self.inv_freq, rope_dims=self.rope_dims,
                          seq_index=ctx.seq_index if kv.writes else None,
                          block_table=kv.block_table if kv.writes else None,
                          k_pages=kv.k_pages if kv.writes else None,
                          v_pages=kv.v_pages if kv.writes else None,
                          page_tiles=ctx.page_tiles() if kv.writes and not ctx.is_decode else None,
                          v_transposed=kv.v_transposed, blocked=bool(kv.blocked))


@POSITION_ENCODINGS.register("rope")
class RotaryEncoding(PositionEncoding):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone
    def __init__(self, head_dim: int, theta: float, rope_dims: int = 0, scaling=None):
        self.head_dim = int(head_dim)
        self.rope_dims = int(rope_dims) or self.head_dim
        if self.rope_dims % 2 or self.rope_dims > self.head_dim:
            raise ValueError(f"rope: rope_dims {self.rope_dims} must be even and at most head_dim {head_dim}")
        self.theta = float(theta)
        self.scaling = dict(scaling) if scaling else None
        self._host = rope_frequencies(self.rope_dims, self.theta, self.scaling)
        self.inv_freq = None

    def prepare(self, device):
        self.inv_freq = self._host.to(device).contiguous()


@POSITION_ENCODINGS.register("none")
class NoEncoding(PositionEncoding):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone
    def __init__(self, head_dim: int = 0):
        self.rope_dims = 0
