"""Dense gated feed-forward: down(act(gate(x)) * up(x)); act is a parameter, silu(g) = g / (1 + exp(-g)) for this
architecture (src/transformer/cpu.c:1270-1303, src/transformer/cpu_backend.c:385-391; the reference's other kinds,
tanh-gelu and relu^2, cpu_backend.c:343-417, are the kernels' other values).  Gate and up
are stored stacked (as the reference's GPU upload stacks them, include/backend_model.h:22)
so that one product computes both, with gate and up rows alternating in blocks of 8 when the
width allows it, so that the decode kernel finds both halves of a result column in one tile;
at decode sizes the activation is part of that kernel."""
from __future__ import annotations

import torch

from .. import ops
from .base import FEED_FORWARDS, ParamSpec, Part
from .linear import Linear, upload


@FEED_FORWARDS.register("gated")
@FEED_FORWARDS.register("swiglu")
class SwiGLU(Part):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone
    takes_deferred_norm = True      # forward accepts an ops.DeferredNorm for h
    gives_lazy_delta = True         # forward(..., lazy_ok=True) may return a LazyDelta

    def __init__(self, hidden: int, intermediate: int, bias: bool = False, activation: str = "silu"):
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"feed-forward: unknown activation {activation!r}; known: {sorted(ops.ACTIVATIONS)}")
        self.hidden, self.F, self.has_bias, self.activation = int(hidden), int(intermediate), bool(bias), activation
        self.gate_up, self.down = Linear(), Linear()
        self.gate_up.stream_tile_rows = ops.STREAM_TILE_ROWS     # gate and up interleaved in blocks of 8: a tile holds both

    def tensors(self):
        t = {"w_gate": ParamSpec((self.F, self.hidden)), "w_up": ParamSpec((self.F, self.hidden)),
             "w_down": ParamSpec((self.hidden, self.F))}
        if self.has_bias:
            t.update({"b_gate": ParamSpec((self.F,), "normal"), "b_up": ParamSpec((self.F,), "normal"),
                      "b_down": ParamSpec((self.hidden,), "normal")})
        return t

    def load(self, tensors, device, dtype):
        self.interleaved = self.F % 8 == 0
        wg, wu = upload(tensors["w_gate"], device, dtype), upload(tensors["w_up"], device, dtype)
        w = ops.interleave_gate_up(wg, wu) if self.interleaved else torch.cat([wg, wu], dim=0)     # on the device
        del wg, wu
        b = None
        if self.has_bias:
            bg, bu = upload(tensors["b_gate"], device, torch.float32), upload(tensors["b_up"], device, torch.float32)
            b = (torch.stack([bg.reshape(-1, 8), bu.reshape(-1, 8)], dim=1).reshape(-1) if self.interleaved
                 else torch.cat([bg, bu]))
        self.gate_up.load(w, b, device, dtype)
        self.down.load(tensors["w_down"], tensors.get("b_down") if self.has_bias else None, device, dtype)

    def linears(self):
        return [self.gate_up, self.down]

    def forward(self, h, ctx, lazy_ok: bool = False):
        if isinstance(h, ops.DeferredNorm):
            w = self.gate_up.weight
            M = h.shape[0]
            if (not self.has_bias and self.interleaved and w.dtype == torch.bfloat16
                    and (ops.can_fuse_norm(M, self.F, self.hidden, w.dtype)
                         or (M > ops.FUSED_ROWS and ops.LIBRARY_PRODUCTS and w.data_ptr() % 16 == 0))):
                act = ops.linear_swiglu_prenorm(h, w, self.activation, self.gate_up.streamed)
                return self.down.lazy(act) if lazy_ok else self.down(act)
            h = h.materialize()
        if self.has_bias:
            act = ops.swiglu(self.gate_up(h), self.interleaved, self.activation)
        else:
            act = ops.linear_swiglu(h, self.gate_up.weight, self.interleaved, activation=self.activation,
                                    streamed=self.gate_up.streamed)
        return self.down.lazy(act) if lazy_ok else self.down(act)
