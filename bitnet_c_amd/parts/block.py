"""Arrangement of the parts of one layer.

"prenorm": x += mixer(norm(x)); x += ffn(norm(x)) -- the order of the reference's layer
(src/transformer/cpu.c:536-939 and :1247-1303): norm, mixer, add, norm, feed-forward, add."""
from __future__ import annotations

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Part, PartSpec


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    def __init__(self, mixer: PartSpec, ffn: PartSpec, mixer_norm: PartSpec, ffn_norm: PartSpec):
        self.mixer = MIXERS.build(mixer)
        self.ffn = FEED_FORWARDS.build(ffn)
        self.mixer_norm = NORMS.build(mixer_norm)
        self.ffn_norm = NORMS.build(ffn_norm)

    @property
    def prompt_capturable(self) -> bool:
        return all(getattr(c, "prompt_capturable", False) for c in self.children().values())

    def children(self):
        return {"mixer": self.mixer, "ffn": self.ffn, "mixer_norm": self.mixer_norm, "ffn_norm": self.ffn_norm}

    def linears(self):
        return [l for part in self.children().values() for l in getattr(part, "linears", list)()]

    def tensors(self):
        return {f"{cn}.{tn}": spec for cn, c in self.children().items() for tn, spec in c.tensors().items()}

    def load(self, tensors, device, dtype):
        for cn, c in self.children().items():
            c.load({k[len(cn) + 1:]: v for k, v in tensors.items() if k.startswith(cn + ".")}, device, dtype)

    def cache_need(self):
        return self.mixer.cache_need()

    def forward(self, stream, ctx, kv):
        # A part that says so may get its norm undone (it applies it inside its first product) and may hand
        # its last product in undone (it then adds itself to the stream): see ResidualStream.
        tap = getattr(ctx, "tap", None)        # diagnostics (StepContext.tap): the stream at the reference's three dump points
        if tap is not None:
            tap("layer_in", ctx.entry, stream, ctx)
        h = stream.normed(self.mixer_norm, ctx.act_dtype, consumer=self.mixer, ctx=ctx)
        if getattr(self.mixer, "gives_lazy_delta", False):
            stream.add(self.mixer.forward(h, ctx, kv, lazy_ok=True))
        else:
            stream.add(self.mixer.forward(h, ctx, kv))
        if tap is not None:
            tap("ffn_in", ctx.entry, stream, ctx)
        h = stream.normed(self.ffn_norm, ctx.act_dtype, consumer=self.ffn, ctx=ctx)
        if getattr(self.ffn, "gives_lazy_delta", False):
            stream.add(self.ffn.forward(h, ctx, lazy_ok=True))
        else:
            stream.add(self.ffn.forward(h, ctx))
        if tap is not None:
            tap("layer_out", ctx.entry, stream, ctx)
