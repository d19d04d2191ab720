"""The plan of a model: data from which the model is built.

A plan lists the layers (each a block of parts, named by registry key and constants),
the order in which they run, and the tensor name of every parameter.  The order is data
too: `schedule` is a list of entries, each naming a layer; a layer may be named twice
(its weights are shared, each entry has cache storage of its own), and an entry may read
the cache of an earlier entry instead of writing its own (`kv_from`).  The reference
holds the same decisions in per-layer plan structs that it recomputes on every call
(src/transformer/plan.c:315-342, 705-863; shared KV: plan.c:18-25).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

from ..parts.base import PartSpec
from ..weights.loader import TensorSpec


@dataclass(frozen=True)
class LayerPlan:
    block: PartSpec                      # a registered block with its parts as parameters
    names: Dict[str, str]                # the block's local tensor name -> name in the model folder


@dataclass(frozen=True)
class ScheduleEntry:
    layer: int
    kv_from: Optional[int] = None        # index of an earlier schedule entry whose cache is read


@dataclass(frozen=True)
class ModelPlan:
    vocab_size: int
    hidden_size: int
    layers: List[LayerPlan]
    schedule: List[ScheduleEntry]
    final_norm: Optional[PartSpec]       # the norm in front of the output matrix; None: the architecture has none
    embedding_name: str
    final_norm_names: Dict[str, str]
    lm_head_name: Optional[str]          # None: the output matrix is the embedding matrix (tied)
    max_positions: int = 0               # 0: no limit from the architecture
    stop_ids: tuple = ()
    # What some architectures put around the blocks (the reference: src/model_embed.c:23-27 scales the embedding
    # row, src/transformer/logits.c:325-333 bounds the logits); 1 and 0 leave this architecture's values as they are.
    embedding_multiplier: float = 1.0    # the embedding row times this before the first block
    logit_softcap: float = 0.0           # > 0: logits = cap * tanh(logits / cap)
    lm_head_bias_name: Optional[str] = None   # a bias [vocab] added to the logits (before the soft-cap); None: none

    def validate(self) -> None:
        if not self.embedding_multiplier > 0 or self.logit_softcap < 0:
            raise ValueError("the embedding multiplier must be positive and the logit soft-cap 0 (none) or positive")
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"schedule entry {i} names layer {e.layer}; there are {len(self.layers)}")
            if e.kv_from is not None:
                if not 0 <= e.kv_from < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.kv_from}, "
                                     f"which does not run before it")
                if self.schedule[e.kv_from].kv_from is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.kv_from}, "
                                     f"which has no cache of its own")

    def expected_tensors(self) -> Dict[str, TensorSpec]:
        """Every tensor of the model folder, by name, with its shape."""
        from ..parts import BLOCKS, NORMS
        out: Dict[str, TensorSpec] = {}

        def put(name, shape, init, optional=False):
            if name in out and tuple(out[name].shape) != tuple(shape):
                raise ValueError(f"tensor {name} is expected with two shapes: {out[name].shape} and {shape}")
            out[name] = TensorSpec(name, tuple(shape), init, optional)

        put(self.embedding_name, (self.vocab_size, self.hidden_size), "normal")
        for lp in self.layers:
            blk = BLOCKS.build(lp.block)
            for local, spec in blk.tensors().items():
                if local not in lp.names:
                    raise ValueError(f"the plan gives no tensor name for {local!r}")
                put(lp.names[local], spec.shape, spec.init, spec.optional)
        if self.final_norm is not None:
            norm = NORMS.build(self.final_norm)
            for local, spec in norm.tensors().items():
                put(self.final_norm_names[local], spec.shape, spec.init, spec.optional)
        if self.lm_head_name is not None:
            put(self.lm_head_name, (self.vocab_size, self.hidden_size), "normal")
        if self.lm_head_bias_name is not None:
            put(self.lm_head_bias_name, (self.vocab_size,), "normal")
        return out
