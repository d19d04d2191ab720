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
from ..parts.linear import Linear, upload
from .plan import ModelPlan


# Of the device's memory, the share that stays free when a model takes streamed copies unasked: activations of long
# prompts, captured graphs and the libraries' work buffers live there.
STREAMED_RESERVE_SHARE = 0.1


def streamed_budget(free_bytes: int, total_bytes: int) -> int:
    """Bytes that a model's streamed copies may take when nobody says: what is free once the weights and the cache are in
    place, but for a tenth of the device's memory.  The copies cost a matrix's size once more and make every decode step
    and short prompt step 5 to 12 % faster, so what the cache does not ask for is spent on them, the largest matrices
    first (a model of 16 GB on 288 GB keeps them all; one of 140 GB keeps those of its feed-forwards' first products as
    far as the room goes)."""
    return max(0, int(free_bytes - STREAMED_RESERVE_SHARE * total_bytes))


class DecoderModel:
    def __init__(self, plan: ModelPlan, dtype=torch.bfloat16, device="cuda:0", streamed_weights=None):
        """streamed_weights: keep a second copy of every weight matrix in the order in which the kernels of up to 128
        rows read it (ops.StreamedWeight): True at load, False never; None: the engine that takes the model decides once
        its cache is allocated (settle_streamed: as many copies as streamed_budget allows, the largest matrices first).
        BITNET_STREAMED_WEIGHTS=0 or 1 decides instead, for measurements."""
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"compute dtype must be bfloat16 or float32, got {dtype}")
        plan.validate()
        self.plan, self.dtype, self.device = plan, dtype, torch.device(device)
        env = os.environ.get("BITNET_STREAMED_WEIGHTS", "")
        self.streamed_weights = streamed_weights if streamed_weights is not None or env == "" else env != "0"
        self.head = Linear()             # the output matrix as the parts hold theirs (weight = lm_head; its streamed copy)
        self.has_streamed = False        # whether any matrix has a streamed copy
        self.streamed_settled = False    # whether the copies have been decided (at load, or by settle_streamed)
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
        self.head.weight = self.lm_head
        if self.streamed_weights is not None:
            self.keep_streamed(bool(self.streamed_weights))
        else:
            self.keep_streamed(False)
            self.streamed_settled = False          # an engine decides, with its cache in place

    # ---- streamed copies ---------------------------------------------------------------
    def linears(self) -> list:
        """Every weight matrix that a product of few rows reads once: the parts' own and the output matrix."""
        return [l for blk in self.blocks for l in getattr(blk, "linears", list)()] + [self.head]

    def streamed_bytes(self) -> int:
        """Bytes that the streamed copies of all weight matrices take (taken or not)."""
        if self.dtype != torch.bfloat16 or self.device.type != "cuda":
            return 0
        return sum(l.stream_bytes() for l in self.linears())

    def keep_streamed(self, keep: bool = True, budget: int = None, keep_free: int = 0) -> int:
        """Makes (or drops) the streamed copies of the parts' weight matrices and of the output matrix; with a budget (in
        bytes) only as many as fit into it, the largest matrices first.  keep_free: bytes of the device's memory that
        must stay free; a copy that cuts into them (the allocator could not place it in what it holds) is dropped again
        and no other of its size or larger is tried, and so is a copy that the device has no room for.  Returns the bytes that the copies
        take."""
        matrices = self.linears()
        applies = self.dtype == torch.bfloat16 and self.device.type == "cuda"
        sizes = [l.stream_bytes() if applies else 0 for l in matrices]
        used, too_large = 0, None                # too_large: the size of a copy that found no place (smaller ones still may)
        for i in sorted(range(len(matrices)), key=lambda i: -sizes[i]):      # a stable order: equal sizes in model order
            fits = bool(keep and sizes[i] > 0 and (too_large is None or sizes[i] < too_large)
                        and (budget is None or used + sizes[i] <= budget))
            free_before = torch.cuda.mem_get_info(self.device)[0] if fits and keep_free else 0
            try:
                matrices[i].keep_streamed(fits)
            except torch.cuda.OutOfMemoryError:
                matrices[i].keep_streamed(False)
                fits, too_large = False, sizes[i]
            if fits and keep_free and torch.cuda.mem_get_info(self.device)[0] < min(keep_free, free_before):
                matrices[i].keep_streamed(False)         # it was placed in memory that is to stay free
                torch.cuda.empty_cache()
                fits, too_large = False, sizes[i]
            used += sizes[i] if fits else 0
        self.has_streamed = used > 0
        self.streamed_settled = True
        return used

    def settle_streamed(self) -> None:
        """Called by an engine once its cache is allocated: a model that was not told whether to keep streamed copies
        takes as many as streamed_budget allows now.  What the allocator holds without using it counts as free (after
        loading a model of 140 GB that is tens of GB, in pieces: a copy that finds no piece large enough is placed in the
        device's free memory, of which a tenth of the device is kept back)."""
        if self.streamed_settled:
            return
        free, total, held = 0, 0, 0
        if self.device.type == "cuda":
            torch.cuda.empty_cache()
            free, total = torch.cuda.mem_get_info(self.device)
            held = max(0, torch.cuda.memory_reserved(self.device) - torch.cuda.memory_allocated(self.device))
        self.keep_streamed(True, streamed_budget(free + held, total), keep_free=int(STREAMED_RESERVE_SHARE * total))

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
        logits = ops.linear(h, self.lm_head, torch.float32, streamed=self.head.streamed)
        if self.lm_head_bias is not None and logits.shape[0]:
            ops.bias_add(logits, self.lm_head_bias)
        if self.plan.logit_softcap > 0:                            # src/transformer/logits.c:325-333
            ops.softcap_(logits, self.plan.logit_softcap)
        return logits
