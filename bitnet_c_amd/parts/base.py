"""What a layer is put together from: a mixer (attention here), a feed-forward, norms, a
position encoding, and the arrangement of these in a block.  Each kind of part has its
own registry from a name to a class; a plan names parts by (kind, params) and a layer is
built from the plan alone, so one model can hold different mixers and feed-forwards in
different layers.  No part knows which model it is in: sizes and constants arrive as
parameters, tensors under local names ("wq", "weight"), and the architecture maps the
local names to the names of the model folder.

Interfaces (a new part implements the one of its kind and registers itself):

  every part     tensors() -> {local name: TensorSpec-like (shape, init, optional)}
                 load(tensors: {local name: host tensor}, device, dtype) -> None
                 linears() -> [parts.linear.Linear] (optional: the weight matrices that the model may keep a
                 second time in the order the decode kernels read them)

  norm           apply(x_f32 [T, D], delta or None, out_dtype, rows=None) -> [T or len(rows), D]
                 (adds delta into x in place when rows is None, then norms)

  position       prepare(device) -> None
                 encode_and_store(qkv, ctx, H, Hkv, hs, kv) -> None
                 (encodes Q in place, encodes K and stores K, V into kv when kv.writes)

  mixer          cache_need() -> CacheNeed (what it keeps per sequence: keys/values and/or a
                 state of fixed size)
                 forward(h [T, D], ctx, kv) -> delta [T, D]

  feed-forward   forward(h [T, D], ctx) -> delta [T, D]

  block          forward(stream: ResidualStream, ctx, kv) -> None

The reference decides the same things per call with per-layer plan structs
(include/transformer_plan_internal.h:12-185, src/transformer/plan.c:315-342, 705-863);
here the decision is made once, when the model is built.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch


@dataclass(frozen=True)
class PartSpec:
    """A part named by its registry key and its constants."""
    kind: str
    params: Tuple[Tuple[str, object], ...] = ()

    @staticmethod
    def of(kind: str, **params) -> "PartSpec":
        return PartSpec(kind, tuple(sorted(params.items())))

    def kwargs(self) -> dict:
        return dict(self.params)


@dataclass(frozen=True)
class ParamSpec:
    shape: Tuple[int, ...]
    init: str = "normal"        # how the random-weights mode fills it: normal | ones | zeros
    optional: bool = False


@dataclass(frozen=True)
class KVNeed:
    """Keys and values of every position (window 0) or of the last `window` positions, and how a page of the
    cache holds them.  A page keeps PAGE positions of every kv head: the keys as [kv head, PAGE, head_dim]; the
    values, v_head_dim wide (0: as wide as the keys), either the same way (v_layout "rows") or turned,
    [kv head, v_head_dim, PAGE] ("transposed": 8 consecutive positions of one value column lie together).  "blocked"
    (bf16, values as wide as keys, a head size that is a multiple of 32) keeps the sizes of "transposed" but orders
    the keys and the values inside a (page, kv head) as this library's matrix-core attention kernels load them
    (ops.blocked_page_index); nothing else reads such pages.  v_layout None asks for the layout
    that this library's attention kernels read at the cache's type and head size (ops.kernel_v_layout); a mixer with
    kernels or torch code of its own names the layout it wants ("rows" or "transposed")."""
    n_kv_heads: int
    head_dim: int
    window: int = 0
    v_head_dim: int = 0
    v_layout: Optional[str] = None

    V_LAYOUTS = ("rows", "transposed", "blocked")

    def __post_init__(self):
        if self.v_layout is not None and self.v_layout not in self.V_LAYOUTS:
            raise ValueError(f"KVNeed: v_layout {self.v_layout!r} is not one of {self.V_LAYOUTS}")
        if self.n_kv_heads < 1 or self.head_dim < 1 or self.v_head_dim < 0 or self.window < 0:
            raise ValueError(f"KVNeed: sizes must be positive, got {self}")
        if self.v_layout == "blocked" and (self.head_dim % 32 or self.v_head_dim not in (0, self.head_dim)):
            raise ValueError(f"KVNeed: blocked pages need values as wide as keys and a head size that is a multiple of 32, got {self}")

    @property
    def v_dim(self) -> int:
        return self.v_head_dim or self.head_dim


@dataclass(frozen=True)
class StateNeed:
    """A state of fixed size per sequence, zero when the sequence starts.  device_addressed: the mixer reads
    and writes it through the step's device-side slot ids only (ctx.slot_ids; padding rows carry the id of a
    row that no sequence owns), never through the host's slot list, so its decode steps can be replayed from
    a captured graph."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
    device_addressed: bool = False


@dataclass(frozen=True)
class CacheNeed:
    kv: Optional[KVNeed] = None
    state: Optional[StateNeed] = None


class Registry:
    def __init__(self, what: str):
        self.what = what
        self._items: Dict[str, type] = {}

    def register(self, name: str, cls: type = None, *, replace: bool = False):
        def put(c):
            if name in self._items and not replace:
                raise ValueError(f"{self.what} {name!r} is already registered")
            self._items[name] = c
            return c
        return put(cls) if cls is not None else put

    def build(self, spec: PartSpec, **extra):
        if spec.kind not in self._items:
            raise KeyError(f"unknown {self.what} {spec.kind!r}; registered: {sorted(self._items)}")
        return self._items[spec.kind](**spec.kwargs(), **extra)

    def names(self):
        return sorted(self._items)

    def __contains__(self, name):
        return name in self._items


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block")


class Part:
    """Base of all parts: no tensors, nothing to load."""

    # Whether the part's work on a prompt step can be recorded into a graph and replayed for other sequences: it reads
    # the step from the device tensors of its context alone (tokens, positions, seq_index, seq_lens, slot_ids, tiles(),
    # page_tiles(), the block tables), never from the host lists (slots, n_new, pos0, row_ranges()), and never waits for
    # the device.  The parts of this library say True; a part that does not say so keeps its model's prompt steps eager.
    prompt_capturable = False

    def tensors(self) -> Dict[str, ParamSpec]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        pass

    def linears(self) -> list:
        """The part's weight matrices (parts.linear.Linear) that are read once per product: a model may ask each of them
        to keep a streamed copy of its weight.  A part with kernels of its own returns none."""
        return []


@dataclass
class KVView:
    """What a mixer sees of the cache for one entry of the schedule in one step."""
    k_pages: Optional[torch.Tensor] = None      # [pages, Hkv, PAGE, head_dim]
    v_pages: Optional[torch.Tensor] = None      # [pages, Hkv, PAGE, v_dim], or [pages, Hkv, v_dim, PAGE] when v_transposed
    v_transposed: Optional[bool] = None         # the layout of v_pages (KVNeed.v_layout as the cache resolved it)
    blocked: bool = False                       # keys and values in the matrix-core kernels' own order (v_layout "blocked")
    block_table: Optional[torch.Tensor] = None  # [B, W] int32, this step's sequences
    writes: bool = True                         # False: the entry reads another entry's cache
    state: Optional[torch.Tensor] = None        # [max_slots + 1, *shape] fixed-size state, by slot
    max_len: int = 0                            # bound of the key count in this step (sizes the splits)


class LazyDelta:
    """A part's output that is still a product to be done: activations and the Linear that ends the
    part.  The stream either lets the product add itself to the stream and leave the next norm
    deferred (one kernel, ops.linear_into_stream), or computes it the plain way."""

    def __init__(self, act: torch.Tensor, linear):
        self.act, self.linear = act, linear

    def compute(self) -> torch.Tensor:
        return self.linear(self.act)


class ResidualStream:
    """The float32 residual stream of a step.  A part's output is held back as `pending` and
    is added by the kernel of the next norm, so the sum is formed once, in float32, without a
    pass of its own.  At decode sizes a part may hand in its last product undone (LazyDelta) and a
    consumer may take the norm undone (ops.DeferredNorm): the product then adds itself to the stream
    and the consumer's first product applies the norm, and neither the sum nor the norm is a kernel."""

    def __init__(self, x: torch.Tensor):
        self.x = x
        self.pending = None                      # a tensor, a LazyDelta, ops.PartialSums or None

    def add(self, delta) -> None:
        if self.pending is not None:
            self.flush()
        self.pending = delta

    def _pending_tensor(self):
        if isinstance(self.pending, LazyDelta):
            self.pending = self.pending.compute()
        return self.pending

    def flush(self) -> torch.Tensor:
        if self.pending is not None:
            from .. import ops
            ops.residual_add(self.x, self._pending_tensor())
            self.pending = None
        return self.x

    def normed(self, norm, out_dtype, rows=None, consumer=None, ctx=None):
        """The normed stream for the next part.  `consumer`: the part that will read it; when it
        declares `takes_deferred_norm` and the pending output is a LazyDelta that the norm can be
        folded around, the result is an ops.DeferredNorm instead of a tensor.  With more rows than the fused
        products take, a consumer that has a method wants_deferred_norm(ctx, rows) is asked first (ctx: the step's
        context): one that would only apply the norm the plain way gets the plain norm, in one kernel instead of two."""
        if (rows is None and isinstance(self.pending, LazyDelta) and getattr(consumer, "takes_deferred_norm", False)
                and getattr(norm, "deferrable", False)):
            deferred = self.pending.linear.into_stream(self.pending.act, self.x, norm.weight, norm.eps)
            if deferred is not None:
                self.pending = None
                return deferred
        if (rows is None and getattr(consumer, "takes_deferred_norm", False) and getattr(norm, "deferrable", False)
                and not isinstance(self.pending, LazyDelta)):
            from .. import ops
            wants = getattr(consumer, "wants_deferred_norm", None)
            if (ops.can_sum_deferred(self.x.shape[0], self.x.shape[1], out_dtype) and self.x.is_contiguous()
                    and (wants is None or ctx is None or wants(ctx, self.x.shape[0]))):
                # more rows than the fused products take: one kernel adds the pending output (a tensor or partial sums)
                # and leaves the norm's factor to the consumer's own kernels
                deferred = ops.sum_deferred(self.x, self.pending, norm.weight, norm.eps)
                self.pending = None
                return deferred
        delta = self._pending_tensor()
        if delta is not None and not isinstance(delta, torch.Tensor) and not getattr(norm, "takes_partial_sums", False):
            self.flush()                         # partial sums, and a norm that only knows tensors: add them up first
            delta = None
        h = norm.apply(self.x, delta, out_dtype, rows)
        if rows is None:
            self.pending = None
        return h
