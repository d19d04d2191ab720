"""The model: parts built from a plan, weights loaded into them, one forward over the
tokens of a step.  It owns the uploaded device tensors (the reference's backend model
holds them apart from the immutable host weights, include/backend_model.h:14-108).
"""
from __future__ import annotations

import os
from typing import Dict, List

import torch

from .. import ops
from ..parts import BLOCKS, NORMS, CacheNeed, ResidualStream
from ..parts.linear import upload
from .plan import ModelPlan


# Of the device's memory, the share that has to stay free after the streamed copies for a model to keep them unasked.
STREAMED_FREE_SHARE = 0.5


def streamed_by_default(copy_bytes: int, free_bytes: int, total_bytes: int) -> bool:
    """Whether a model keeps streamed copies of its weight matrices when nobody says: they cost the matrices' size once
    more and make every decode step and short prompt step 5 to 12 % faster, so they are kept where memory is plentiful
    (half of the device still free afterwards: on 288 GB every model up to some 70 GB of weights) and left out where the
    cache needs the room."""
    return copy_bytes > 0 and free_bytes - copy_bytes >= STREAMED_FREE_SHARE * total_bytes


class DecoderModel:
    def __init__(self, plan: ModelPlan, dtype=torch.bfloat16, device="cuda:0", streamed_weights=None):
        """streamed_weights: keep a second copy of every weight matrix in the order in which the kernels of up to 128
        rows read it (ops.StreamedWeight); None: streamed_by_default decides after the weights are loaded
        (BITNET_STREAMED_WEIGHTS=0 or 1 decides instead, for measurements)."""
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"compute dtype must be bfloat16 or float32, got {dtype}")
        plan.validate()
        self.plan, self.dtype, self.device = plan, dtype, torch.device(device)
        env = os.environ.get("BITNET_STREAMED_WEIGHTS", "")
        self.streamed_weights = streamed_weights if streamed_weights is not None or env == "" else env != "0"
        self.lm_head_streamed = None     # ops.StreamedWeight of the output matrix
        self.has_streamed = False
        self.blocks = [BLOCKS.build(lp.block) for lp in plan.layers]
        self.final_norm = NORMS.build(plan.final_norm) if plan.final_norm is not None else None
        self.lm_head_bias = None         # [V] float32, when the plan names one
        self.embedding = None            # [V, D] in the compute dtype
        self.lm_head = None              # [V, D]; the embedding itself when tied

    # ---- weights --------------------------------------------------------------------
    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        """tensors: folder name -> host (or device) tensor for every name of plan.expected_tensors(): a dict, or a
        weights.TensorSource, whose tensors are views of the mapped file; then every layer's tensors are let go
        (release) as soon as the layer has uploaded them, so the host never holds the model."""
        p = self.plan
        done = getattr(tensors, "release", lambda names: None)
        for lp, blk in zip(p.layers, self.blocks):
            local = {ln: tensors[fn] for ln, fn in lp.names.items() if fn in tensors and ln in blk.tensors()}
            blk.load(local, self.device, self.dtype)
            del local
            done(lp.names.values())
        if self.final_norm is not None:
            self.final_norm.load({ln: tensors[fn] for ln, fn in p.final_norm_names.items()}, self.device, self.dtype)
        if p.lm_head_bias_name is not None:
            self.lm_head_bias = upload(tensors[p.lm_head_bias_name], self.device, torch.float32)
            done([p.lm_head_bias_name])
        self.embedding = upload(tensors[p.embedding_name], self.device, self.dtype)
        done([p.embedding_name])
        if p.lm_head_name is None:
            self.lm_head = self.embedding
        else:
            self.lm_head = upload(tensors[p.lm_head_name], self.device, self.dtype)
            done([p.lm_head_name])
        keep = self.streamed_weights
        if keep is None:
            free, total = torch.cuda.mem_get_info(self.device) if self.device.type == "cuda" else (0, 0)
            keep = streamed_by_default(self.streamed_bytes(), free, total)
        self.keep_streamed(bool(keep))

    # ---- streamed copies ---------------------------------------------------------------
    def linears(self) -> list:
        return [l for blk in self.blocks for l in getattr(blk, "linears", list)()]

    def streamed_bytes(self) -> int:
        """Bytes that the streamed copies of all weight matrices take (taken or not)."""
        if self.dtype != torch.bfloat16 or self.device.type != "cuda":
            return 0
        head = 0
        if self.lm_head is not None and self.lm_head.shape[1] % 8 == 0:
            R, C = ops.stream_tile_rows(self.lm_head.shape[0]), ops.STREAM_TILE_COLS
            head = -(-self.lm_head.shape[0] // R) * R * -(-self.lm_head.shape[1] // C) * C * 2
        return head + sum(l.stream_bytes() for l in self.linears())

    def keep_streamed(self, keep: bool = True) -> None:
        """Makes (or drops) the streamed copy of every weight matrix of the parts and of the output matrix."""
        keep = keep and self.streamed_bytes() > 0
        for l in self.linears():
            l.keep_streamed(keep)
        head = keep and self.lm_head is not None and self.lm_head.shape[1] % 8 == 0
        self.lm_head_streamed = ops.stream_copy(self.lm_head) if head else None
        self.has_streamed = bool(keep)

    def weight_bytes(self) -> int:
        """Bytes of every weight a decode step reads once (the embedding table only when it is
        also the output matrix)."""
        seen, total = set(), 0

        def add(t):
            nonlocal total
            if t is not None and t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()

        def walk(obj, depth=0):
            if isinstance(obj, torch.Tensor):
                add(obj)
            elif depth < 4 and hasattr(obj, "__dict__"):
                for k, v in vars(obj).items():
                    if k != "streamed":                # a second copy of a matrix: a step reads one of the two
                        walk(v, depth + 1)

        for blk in self.blocks:
            walk(blk)
        walk(self.final_norm)
        add(self.lm_head)
        add(self.lm_head_bias)
        return total

    # ---- cache needs -------------------------------------------------------------------
    def cache_needs(self):
        needs: List[CacheNeed] = [self.blocks[e.layer].cache_need() for e in self.plan.schedule]
        return needs, [e.kv_from for e in self.plan.schedule]

    # ---- forward -----------------------------------------------------------------------
    def forward(self, ctx, views) -> torch.Tensor:
        """ctx: the step's StepContext; views[i]: the KVView of schedule entry i.
        Returns float32 logits [len(ctx.want_rows), vocab]."""
        x = ops.embed_gather(self.embedding, ctx.tokens, self.plan.embedding_multiplier)    # src/model_embed.c:6-28
        stream = ResidualStream(x)
        for i, e in enumerate(self.plan.schedule):
            ctx.entry = i
            self.blocks[e.layer].forward(stream, ctx, views[i])
        # final norm on the wanted rows only, then the output matrix (src/transformer/logits.c:249-314)
        if self.final_norm is not None:
            h = stream.normed(self.final_norm, self.dtype, rows=ctx.want_rows)
        else:
            h = ops.gather_rows(stream.flush(), ctx.want_rows, self.dtype)
        logits = ops.linear(h, self.lm_head, torch.float32, streamed=self.lm_head_streamed)
        if self.lm_head_bias is not None and logits.shape[0]:
            ops.bias_add(logits, self.lm_head_bias)
        if self.plan.logit_softcap > 0:                            # src/transformer/logits.c:325-333
            ops.softcap_(logits, self.plan.logit_softcap)
        return logits
