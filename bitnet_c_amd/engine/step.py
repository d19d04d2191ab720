"""The step function and what it needs: the description of a step's batch and the engine
that runs it against the cache.

One step takes a batch of sequences that start together, with unequal lengths: their
prompts in one step, then one token each.  It runs only the tokens it is given, all
sequences as one flattened batch without padding between them, reads everything earlier
from the cache, and returns the float32 logits at the wanted places.  The reference has
five single-sequence entry points for this (include/transformer.h:9-30: one token with or
without logits; n tokens with last, no or all logits) and validates tokens and positions
before it touches state (src/transformer/prefill.c:1228-1237, src/transformer.c:60-70);
all new keys and values are in the cache before any new token attends
(src/transformer/prefill.c:1836-1875 before :1962).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Sequence

import torch

from .. import ops
from ..cache import PAGE, CacheError, CacheFull, PagedCache
from ..config import load_config
from ..weights import open_tensors
from .model import DecoderModel


class StepError(ValueError):
    """A step that cannot run; nothing was changed."""


@dataclass
class StepEntry:
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()          # places among `tokens` whose logits are wanted


class StepContext:
    """Device-side description of one step, shared by all parts."""

    def __init__(self, device, act_dtype, tokens, positions, seq_index, seq_lens, want_rows, slots_dev,
                 is_decode, slots, n_new, pos0, by_length=None, max_len_dev=None, captured=False):
        self.device, self.act_dtype = device, act_dtype
        # captured: the step is being recorded into a HIP graph and will be replayed with other sequences: only
        # the device tensors (tokens, positions, seq_lens, slot_ids, ...) are valid then, the host lists are not.
        # max_len_dev: in a captured step, a device int32 with the longest sequence's key count of each replay
        self.captured, self.max_len_dev = captured, max_len_dev
        # decode steps: the rows ordered by sequence length, longest first (a hint for kernels that
        # balance their workgroups by it; None = no hint)
        self.by_length = by_length
        self.tokens, self.positions, self.seq_index = tokens, positions, seq_index
        self.seq_lens, self.want_rows, self.slot_ids = seq_lens, want_rows, slots_dev
        self.is_decode = is_decode
        self.slots, self.n_new, self.pos0 = list(slots), list(n_new), list(pos0)   # host copies
        self.n_rows = int(tokens.numel())
        self.n_seqs = len(self.slots)
        # diagnostics: a callable (point, schedule entry, ResidualStream, ctx) that blocks call at "layer_in",
        # "ffn_in" and "layer_out" (the reference's bitnet_inp / bitnet_ffn_inp / bitnet_lout dumps,
        # src/transformer/cpu.c:401, :951, :981); `entry` is the schedule entry that is running
        self.tap = None
        self.entry = -1
        self._tiles: Dict[int, torch.Tensor] = {}
        self._page_tiles = None

    def row_ranges(self):
        """(first row, rows) of every sequence in the flattened batch."""
        out, r = [], 0
        for n in self.n_new:
            out.append((r, n))
            r += n
        return out

    def page_tiles(self) -> torch.Tensor:
        """[n, 4] int32: the new tokens cut at page boundaries (sequence, first row, rows, position of
        the first), for kernels that store a page's positions together.  A list may end in tiles of no rows."""
        if self._page_tiles is None:
            if self.captured:
                raise StepError("this captured step was recorded without a list of page tiles")
            self._page_tiles = torch.tensor(_page_tiles(self.n_new, self.pos0),
                                            dtype=torch.int32).reshape(-1, 4).to(self.device)
        return self._page_tiles

    def tiles(self, qt: int) -> torch.Tensor:
        """[n, 4] int32: (sequence, first row, rows <= qt, position of the first) covering all new
        tokens, for the prompt form of the attention kernel, in the order that gives its workgroups
        equal work (ops.pair_tiles).  A list may end in tiles of no rows."""
        t = self._tiles.get(qt)
        if t is None:
            if self.captured:
                raise StepError(f"this captured step was recorded without a list of tiles of {qt} tokens")
            t = torch.tensor(_query_tiles(self.n_new, self.pos0, qt), dtype=torch.int32).reshape(-1, 4).to(self.device)
            self._tiles[qt] = t
        return t


def _page_tiles(n_new, pos0) -> List[tuple]:
    """(sequence, first row, rows, position of the first) for every run of a sequence's new tokens
    inside one page."""
    rows, r = [], 0
    for s, (n, p0) in enumerate(zip(n_new, pos0)):
        i = 0
        while i < n:
            m = min(n - i, PAGE - (p0 + i) % PAGE)
            rows.append((s, r + i, m, p0 + i))
            i += m
        r += n
    return rows


def _query_tiles(n_new, pos0, qt: int) -> List[tuple]:
    """(sequence, first row, rows <= qt, position of the first) covering every sequence's new tokens, in the order
    in which the prompt form of attention wants them (ops.pair_tiles)."""
    rows, r = [], 0
    for s, (n, p0) in enumerate(zip(n_new, pos0)):
        for i in range(0, n, qt):
            rows.append((s, r + i, min(qt, n - i), p0 + i))
        r += n
    return ops.pair_tiles(rows)


def _by_length(lens) -> List[int]:
    """The rows ordered by length, longest first (ties by row)."""
    return sorted(range(len(lens)), key=lambda i: (-lens[i], i))


MAX_GRAPH_ROWS = 256      # rows of the largest captured decode step; a step of more sequences is replayed in pieces of this size


# Rows of the captured decode steps: the powers of two, and between them the counts at which the kernels' work takes a
# step (twelve rows of the sixteen of a matrix-core tile, three and six tiles of rows), so that a batch that has shrunk
# to 40 sequences does not pay for 64.
DECODE_BUCKETS = (1, 2, 4, 8, 12, 16, 32, 48, 64, 96, 128, 192, 256)


def _bucket(n: int) -> int:
    for b in DECODE_BUCKETS:
        if b >= n:
            return b
    return DECODE_BUCKETS[-1]


class _DecodeGraph:
    """A captured decode step for up to `rows` sequences.  The block tables are as wide as the engine's longest
    sequence and the split plan of attention follows the longest sequence of each replay through a device-side
    integer, so a graph is made for a number of rows and nothing else: no step of a generation waits for a
    capture because a sequence has grown.  The step's integers live in pinned buffers that are refilled
    before every replay; a row of the block tables is rewritten only when its sequence's pages have changed."""

    N_FIELDS = 7            # tokens, positions, sequence index, lengths, wanted rows, order by length, slot ids

    def __init__(self, engine: "Engine", rows: int):
        self.rows, self.width = rows, engine.max_pages
        dev, cache = engine.device, engine.cache
        n_groups = len(cache.groups)
        self.host = torch.zeros(self.N_FIELDS * rows + 1, dtype=torch.int32).pin_memory()
        self.host_np = self.host.numpy()                      # the same memory
        self.host_np[2 * rows:3 * rows] = range(rows)         # row b is sequence b
        self.host_np[4 * rows:5 * rows] = range(rows)         # wanted rows: all
        self.dev = torch.zeros(self.host.numel(), dtype=torch.int32, device=dev)
        self.host_tables = torch.zeros((max(n_groups, 1), rows, self.width), dtype=torch.int32).pin_memory()
        self.tables_np = self.host_tables.numpy()
        self.dev_tables = torch.zeros(self.host_tables.shape, dtype=torch.int32, device=dev)
        self.row_keys = [None] * rows                         # (slot, version of its pages) that a table row holds
        self.tables_dirty = True
        self.copied = torch.cuda.Event()
        self.copied.record()
        f = [self.dev[k * rows:(k + 1) * rows] for k in range(self.N_FIELDS)]
        self.tokens, self.positions, self.seq_index, self.seq_lens, self.want, self.by_length, self.slot_ids = f
        self.max_len = self.dev[self.N_FIELDS * rows:self.N_FIELDS * rows + 1]
        self.tables = {g: self.dev_tables[g] for g in range(n_groups)}
        views = [cache.view(i, self.tables, self.width * PAGE) for i in range(len(engine.model.plan.schedule))]
        self.ctx = StepContext(dev, engine.model.dtype, self.tokens, self.positions, self.seq_index, self.seq_lens,
                               self.want, self.slot_ids, True, [-1] * rows, [1] * rows, [0] * rows,
                               by_length=self.by_length, max_len_dev=self.max_len, captured=True)
        # padding rows everywhere: the warm-up and the capture run touch no sequence's pages or state
        self.fill([], [], [], engine)
        self.upload()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            engine.model.forward(self.ctx, views)              # loads every kernel before the capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, pool=engine.graph_pool):
            self.logits = engine.model.forward(self.ctx, views)

    def fill(self, slots, tokens, lens_after, engine):
        """Writes the step's integers into the pinned buffers."""
        rows, h, cache = self.rows, self.host_np, engine.cache
        self.copied.synchronize()
        n = len(slots)
        h[0:rows] = 0
        h[0:n] = tokens
        h[rows:2 * rows] = -1                                         # padding rows: position -1
        h[rows:rows + n] = [l - 1 for l in lens_after]
        h[3 * rows:4 * rows] = 0                                      # and no keys
        h[3 * rows:3 * rows + n] = lens_after
        h[5 * rows:6 * rows] = _by_length(list(lens_after) + [0] * (rows - n))
        h[6 * rows:7 * rows] = cache.padding_slot                     # their state is the row that no sequence owns
        h[6 * rows:6 * rows + n] = slots
        h[7 * rows] = max(lens_after) if n else 0
        for r, s in enumerate(slots):
            key = (s, cache.slot_version(s))
            if key != self.row_keys[r]:
                for g in range(len(cache.groups)):
                    pl = cache.pages_of(g, s)
                    self.tables_np[g, r, :len(pl)] = [max(p, 0) for p in pl]     # a page given back: as block_table
                    self.tables_np[g, r, len(pl):] = 0       # and nothing of the row's former owner stays behind it
                self.row_keys[r] = key
                self.tables_dirty = True
        for r in range(n, rows):                             # rows that have become padding: the table block_table() gives
            if self.row_keys[r] is not None:
                self.tables_np[:, r, :] = 0
                self.row_keys[r] = None
                self.tables_dirty = True

    def upload(self):
        self.dev.copy_(self.host, non_blocking=True)
        if self.tables_dirty:
            self.dev_tables.copy_(self.host_tables, non_blocking=True)
            self.tables_dirty = False
        self.copied.record()

    def run(self):
        self.graph.replay()
        return self.logits


MAX_PROMPT_GRAPH_ROWS = 8192      # prompt steps of more tokens than this run eagerly: their launches are a small part of them
MAX_PROMPT_GRAPHS = 12            # captured prompt steps that an engine keeps; the one unused for longest goes first


def _row_bucket(n: int) -> int:
    """Token rows of the captured step that serves a prompt step of n tokens: 16 and 32 (up to 16 rows the products are
    the fused ones of a decode step, and rows cost time there), then multiples of 64 up to 512, of 128 up to 2,048, of
    512 beyond: from 64 tokens on the padding is at most an eighth."""
    if n <= 32:
        return 16 if n <= 16 else 32
    unit = 64 if n <= 512 else 128 if n <= 2048 else 512
    return -(-n // unit) * unit


class _PromptGraph:
    """A captured prompt step (or a mixed one: some sequences with many tokens, some with one) for up to `rows`
    tokens of up to `seqs` sequences with up to `wants` wanted places.  Everything that differs between the steps it
    serves is device memory that is filled before a replay: tokens, positions (-1 for the padding rows, which write
    nothing), the sequence of every row, lengths, wanted rows, slot ids, the block tables at the engine's full
    width, and the tile lists of the attention kernels and of the cache write, padded with tiles of no rows.  So a
    prompt step costs the host one copy and one launch instead of some hundred launches (the reference runs its
    batched prompt pass from one call as well, src/transformer/prefill.c:1228-1962)."""

    def __init__(self, engine: "Engine", rows: int, seqs: int, wants: int, qts: Sequence[int], page_tiles: bool):
        self.rows, self.seqs, self.wants, self.width = rows, seqs, wants, engine.max_pages
        dev, cache = engine.device, engine.cache
        n_groups = len(cache.groups)
        self.n_tiles = {qt: -(-rows // qt) + seqs for qt in qts}         # every sequence may end in a tile that is not full
        self.n_page_tiles = -(-rows // PAGE) + 2 * seqs if page_tiles else 0
        sizes = [rows, rows, rows, seqs, wants, seqs] + [4 * self.n_tiles[qt] for qt in qts] + [4 * self.n_page_tiles]
        self.offsets = [0]
        for n in sizes:
            self.offsets.append(self.offsets[-1] + n)
        self.host = torch.zeros(max(self.offsets[-1], 1), dtype=torch.int32).pin_memory()
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(self.host.numel(), dtype=torch.int32, device=dev)
        f = [self.dev[a:b] for a, b in zip(self.offsets[:-1], self.offsets[1:])]
        self.tokens, self.positions, self.seq_index, self.seq_lens, self.want, self.slot_ids = f[:6]
        self.host_tables = torch.zeros((max(n_groups, 1), seqs, self.width), dtype=torch.int32).pin_memory()
        self.tables_np = self.host_tables.numpy()
        self.dev_tables = torch.zeros(self.host_tables.shape, dtype=torch.int32, device=dev)
        self.row_keys = [None] * seqs
        self.tables_dirty = True
        self.copied = torch.cuda.Event()
        self.copied.record()
        self.tables = {g: self.dev_tables[g] for g in range(n_groups)}
        views = [cache.view(i, self.tables, self.width * PAGE) for i in range(len(engine.model.plan.schedule))]
        self.ctx = StepContext(dev, engine.model.dtype, self.tokens, self.positions, self.seq_index, self.seq_lens,
                               self.want, self.slot_ids, False, [-1] * seqs, [0] * seqs, [0] * seqs, captured=True)
        self.qts = tuple(qts)
        for k, qt in enumerate(self.qts):
            self.ctx._tiles[qt] = f[6 + k].view(-1, 4)
        if page_tiles:
            self.ctx._page_tiles = f[6 + len(self.qts)].view(-1, 4)
        self.fill([], [], [], [], [], engine)                  # padding everywhere: the two runs below touch no sequence
        self.upload()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            engine.model.forward(self.ctx, views)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, pool=engine.graph_pool):
            self.logits = engine.model.forward(self.ctx, views)

    def fill(self, slots, tokens, n_new, pos0, want, engine):
        """tokens: the flattened new tokens; want: rows of the flattened batch."""
        h, o, cache = self.host_np, self.offsets, engine.cache
        self.copied.synchronize()
        T, B = len(tokens), len(slots)
        h[o[0]:o[1]] = 0
        h[o[0]:o[0] + T] = tokens
        h[o[1]:o[2]] = -1
        h[o[2]:o[3]] = 0
        r = 0
        for b, (n, p0) in enumerate(zip(n_new, pos0)):
            h[o[1] + r:o[1] + r + n] = range(p0, p0 + n)
            h[o[2] + r:o[2] + r + n] = b
            r += n
        h[o[3]:o[4]] = 0
        h[o[3]:o[3] + B] = [p + n for p, n in zip(pos0, n_new)]
        h[o[4]:o[5]] = 0
        h[o[4]:o[4] + len(want)] = want
        h[o[5]:o[6]] = cache.padding_slot
        h[o[5]:o[5] + B] = slots
        for k, qt in enumerate(self.qts):
            flat = [v for t in _query_tiles(n_new, pos0, qt) for v in t]
            h[o[6 + k]:o[7 + k]] = 0
            h[o[6 + k]:o[6 + k] + len(flat)] = flat
        if self.n_page_tiles:
            k = 6 + len(self.qts)
            flat = [v for t in _page_tiles(n_new, pos0) for v in t]
            h[o[k]:o[k + 1]] = 0
            h[o[k]:o[k] + len(flat)] = flat
        for r, s in enumerate(slots):
            key = (s, cache.slot_version(s))
            if key != self.row_keys[r]:
                for g in range(len(cache.groups)):
                    pl = cache.pages_of(g, s)
                    self.tables_np[g, r, :len(pl)] = [max(p, 0) for p in pl]
                    self.tables_np[g, r, len(pl):] = 0
                self.row_keys[r] = key
                self.tables_dirty = True
        for r in range(B, self.seqs):
            if self.row_keys[r] is not None:
                self.tables_np[:, r, :] = 0
                self.row_keys[r] = None
                self.tables_dirty = True

    def upload(self):
        self.dev.copy_(self.host, non_blocking=True)
        if self.tables_dirty:
            self.dev_tables.copy_(self.host_tables, non_blocking=True)
            self.tables_dirty = False
        self.copied.record()

    def run(self):
        self.graph.replay()
        return self.logits


class Engine:
    """A model, its cache and the step function over both."""

    def __init__(self, model: DecoderModel, max_tokens: int, max_seq_len: int = 0, max_slots: int = 0,
                 use_graphs: bool = True):
        ops.require_gpu()
        self.model, self.device = model, model.device
        needs, kv_from = model.cache_needs()
        self.cache = PagedCache(needs, kv_from, max_tokens, dtype=model.dtype, device=self.device,
                                max_slots=max_slots or None)
        model.settle_streamed()             # the cache has its memory: what is left may go to streamed copies of the weights
        limit = self.cache.n_pages * PAGE
        if model.plan.max_positions:
            limit = min(limit, model.plan.max_positions)
        self.max_seq_len = min(limit, max_seq_len) if max_seq_len else limit
        self.max_pages = (self.max_seq_len + PAGE - 1) // PAGE
        self.vocab_size = model.plan.vocab_size
        # A replayed graph sees device memory only.  A mixer that keeps a state can decode under graphs when it
        # addresses the state by the step's device-side slot ids (StateNeed.device_addressed); one that walks the
        # host's slot list cannot, and a model with such a mixer runs its decode steps eagerly.
        self.use_graphs = use_graphs and all(n.state is None or n.state.device_addressed for n in needs)
        self.tap = None                     # see StepContext.tap; while it is set, steps run without graphs
        # One captured step per number of rows (DECODE_BUCKETS, up to MAX_GRAPH_ROWS): at most thirteen, made at a batch's
        # start (prepare_decode) or at first use.  They share one memory pool: what a capture frees, the next
        # reuses, and each keeps only its own inputs and logits ([rows, vocab] float32).
        self._graphs: Dict[int, _DecodeGraph] = {}
        self.graph_pool = torch.cuda.graph_pool_handle() if self.use_graphs else None
        # Prompt steps are captured too, per (token rows, sequences, wanted places) rounded up to buckets: the first
        # step of a bucket runs eagerly (and shows which tile lists the model's parts ask for), the second is recorded,
        # every later one is a replay.  Only when every part of the model says that its prompt work can be recorded
        # (Part.prompt_capturable); prompt_graphs False keeps prompt steps eager.
        self.prompt_graphs = (all(getattr(b, "prompt_capturable", False) for b in model.blocks)
                              and (model.final_norm is None or getattr(model.final_norm, "prompt_capturable", False)))
        self._prompt_graphs: Dict[tuple, _PromptGraph] = {}     # in order of last use
        self._prompt_seen: Dict[tuple, int] = {}
        self._prompt_lists = None                                # (tile sizes asked for, page tiles asked for) of an eager prompt step
        self.graphs_built = 0
        self.steps_run = 0

    # ---- construction ---------------------------------------------------------------
    @staticmethod
    def cache_bytes_per_token(model: DecoderModel) -> int:
        """Bytes of keys and values that one cached position takes over all entries of the schedule."""
        needs, kv_from = model.cache_needs()
        size = torch.empty((), dtype=model.dtype).element_size()
        return sum(n.kv.n_kv_heads * (n.kv.head_dim + n.kv.v_dim) * size
                   for n, src in zip(needs, kv_from) if n.kv is not None and src is None)

    @staticmethod
    def tokens_that_fit(model: DecoderModel, wanted: int, share: float = 0.8) -> int:
        """`wanted` cached positions, or as many whole pages as fit into `share` of the device memory that is free
        now (the model is loaded already), whichever is less; at least one page."""
        per_token = Engine.cache_bytes_per_token(model)
        if per_token == 0:
            return max(PAGE, wanted)
        free, _ = torch.cuda.mem_get_info(model.device)
        fit = int(free * share) // per_token // PAGE * PAGE
        return max(PAGE, min(wanted, fit))

    @staticmethod
    def from_folder(folder: str, dtype=torch.bfloat16, max_tokens: int = 4096, device="cuda:0",
                    max_seq_len: int = 0, max_slots: int = 0, use_graphs: bool = True, n_seqs: int = 1,
                    streamed_weights=None) -> "Engine":
        """max_tokens: positions that the cache holds; 0: n_seqs sequences of the longest length there can be
        (the model's max_positions, or max_seq_len when that is less: the reference sizes its cache by
        min(context length, --maxseq), src/model.c:256-257), or as many as fit into the free device memory.
        streamed_weights: as DecoderModel's."""
        ops.require_gpu()
        arch, config = load_config(folder)
        plan = arch.build_plan(config)
        model = DecoderModel(plan, dtype, device, streamed_weights)
        with open_tensors(folder, plan.expected_tensors()) as tensors:      # views of the mapped file, uploaded one by one
            model.load(tensors)
        if max_tokens <= 0:
            longest = min(v for v in (plan.max_positions, max_seq_len) if v > 0) if (plan.max_positions or max_seq_len) else 4096
            per_seq = (longest + PAGE - 1) // PAGE * PAGE
            max_tokens = Engine.tokens_that_fit(model, per_seq * max(1, n_seqs))
        eng = Engine(model, max_tokens, max_seq_len, max_slots, use_graphs)
        eng.config = config
        return eng

    # ---- sequences ------------------------------------------------------------------
    def new_sequence(self) -> int:
        return self.cache.alloc_slot()

    def release(self, slot: int) -> None:
        self.cache.free_slot(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    # ---- the step -------------------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]):
        if not entries:
            raise StepError("a step needs at least one sequence")
        seen = set()
        for e in entries:
            if e.slot in seen:
                raise StepError(f"slot {e.slot} appears twice in one step")
            seen.add(e.slot)
            try:
                have = self.cache.length(e.slot)
            except CacheError as err:
                raise StepError(str(err)) from None
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"slot {e.slot}: no tokens in this step")
            for t in e.tokens:
                if not (0 <= int(t) < self.vocab_size):
                    raise StepError(f"slot {e.slot}: token {t} is outside [0, {self.vocab_size})")
            if have + n > self.max_seq_len:
                raise StepError(f"slot {e.slot}: {have} + {n} tokens exceed the sequence limit {self.max_seq_len}")
            for w in e.want:
                if not (0 <= int(w) < n):
                    raise StepError(f"slot {e.slot}: wanted place {w} is outside its {n} tokens")

    takes_device_tokens = True        # step(..., device_tokens=...) is there

    def step(self, entries: Sequence[StepEntry], device_tokens: torch.Tensor = None) -> torch.Tensor:
        """Runs the entries' tokens as one batch; returns float32 logits [wanted, vocab] in the
        order of the entries and of each entry's `want`.  On an error nothing has changed.

        device_tokens: for a step of one token a sequence, an int32 tensor [len(entries)] on the engine's device that
        holds the tokens (what a sampling kernel has just written); the entries' own tokens are placeholders then.
        The step is queued behind whatever writes that tensor, so the host can queue a decode step before it has
        seen the tokens that the step consumes."""
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        self._validate(entries)
        slots = [e.slot for e in entries]
        n_new = [len(e.tokens) for e in entries]
        if device_tokens is not None:
            if any(n != 1 for n in n_new):
                raise StepError("tokens on the device are taken by steps of one token a sequence only")
            dev = torch.device(self.device)
            there = device_tokens.device.type == dev.type and dev.index in (None, device_tokens.device.index)
            if device_tokens.dtype != torch.int32 or not there or tuple(device_tokens.shape) != (len(entries),):
                raise StepError(f"device_tokens must be int32 [{len(entries)}] on {self.device}, got "
                                f"{device_tokens.dtype} {tuple(device_tokens.shape)} on {device_tokens.device}")
        pos0 = [self.cache.length(s) for s in slots]
        try:
            self.cache.reserve(slots, n_new)
        except CacheFull as err:
            raise StepError(str(err)) from None
        is_decode = all(n == 1 for n in n_new)
        graphs = self.use_graphs and self.tap is None
        try:
            if is_decode and graphs:
                # the sequences of a decode step do not depend on each other: more of them than the largest captured
                # step holds are replayed in pieces
                pieces = [self._step_graph(entries[i:i + MAX_GRAPH_ROWS], slots[i:i + MAX_GRAPH_ROWS], pos0[i:i + MAX_GRAPH_ROWS],
                                           None if device_tokens is None else device_tokens[i:i + MAX_GRAPH_ROWS])
                          for i in range(0, len(entries), MAX_GRAPH_ROWS)]
                logits = pieces[0] if len(pieces) == 1 else torch.cat(pieces)
            elif not is_decode and graphs and self.prompt_graphs and self._prompt_bucket_ready(entries, n_new):
                logits = self._step_prompt_graph(entries, slots, n_new, pos0)
            else:
                logits = self._step_eager(entries, slots, n_new, pos0, is_decode, device_tokens)
        except BaseException:
            self.cache.unreserve(slots)          # the step did not happen: its pages go back
            raise
        self.cache.commit(slots, n_new)
        self.steps_run += 1
        return logits

    def _step_eager(self, entries, slots, n_new, pos0, is_decode, device_tokens=None):
        dev = self.device
        tokens, positions, seq_index, want = [], [], [], []
        row = 0
        for s, e in enumerate(entries):
            tokens += [int(t) for t in e.tokens]
            positions += list(range(pos0[s], pos0[s] + n_new[s]))
            seq_index += [s] * n_new[s]
            want += [row + int(w) for w in e.want]
            row += n_new[s]
        T, B = row, len(entries)
        lens_after = [p + n for p, n in zip(pos0, n_new)]
        tables = {g: self.cache.block_table(g, slots) for g in range(len(self.cache.groups))}
        # one upload for all integer inputs of the step
        order = _by_length(lens_after) if is_decode else []
        parts = [tokens, positions, seq_index, lens_after, want, slots, order] + [tables[g].reshape(-1).tolist()
                                                                                   for g in sorted(tables)]
        flat = torch.tensor([v for p in parts for v in p], dtype=torch.int32)
        devbuf = flat.to(dev)
        o = 0

        def take(n):
            nonlocal o
            v = devbuf[o:o + n]
            o += n
            return v

        d_tokens, d_pos, d_seq, d_lens, d_want, d_slots = take(T), take(T), take(T), take(B), take(len(want)), take(B)
        if device_tokens is not None:
            d_tokens.copy_(device_tokens)
        d_order = take(len(order)) if is_decode else None
        d_tables = {g: take(tables[g].numel()).view(tables[g].shape) for g in sorted(tables)}
        ctx = StepContext(dev, self.model.dtype, d_tokens, d_pos, d_seq, d_lens, d_want, d_slots, is_decode,
                          slots, n_new, pos0, by_length=d_order)
        ctx.tap = self.tap
        max_len = max(lens_after)
        views = [self.cache.view(i, d_tables, max_len) for i in range(len(self.model.plan.schedule))]
        logits = self.model.forward(ctx, views)
        if not is_decode:
            self._prompt_lists = (tuple(sorted(ctx._tiles)), ctx._page_tiles is not None)
        return logits

    # ---- captured prompt steps ----------------------------------------------------------
    @staticmethod
    def _prompt_key(entries, n_new):
        wants = sum(len(e.want) for e in entries)
        return _row_bucket(sum(n_new)), _bucket(len(entries)), _bucket(wants) if wants else 0

    def _prompt_bucket_ready(self, entries, n_new) -> bool:
        """Whether this prompt step is replayed from a graph: its bucket has been seen before (the first step of a
        bucket runs eagerly: one-off prompts never pay for a capture)."""
        if sum(n_new) > MAX_PROMPT_GRAPH_ROWS:
            return False
        key = self._prompt_key(entries, n_new)
        if key in self._prompt_graphs:
            return True
        seen = self._prompt_seen.get(key, 0)
        self._prompt_seen[key] = seen + 1
        return seen >= 1 and self._prompt_lists is not None

    def prepare_prompt(self, n_tokens: int, n_seqs: int = 1, n_wanted: int = 1) -> None:
        """Captures, now, the graph that prompt steps of this size replay (a server does it for the sizes it
        expects, a benchmark before its clock starts).  Needs one eager prompt step to have run before."""
        if not (self.use_graphs and self.prompt_graphs and self.tap is None) or n_tokens > MAX_PROMPT_GRAPH_ROWS:
            return
        if self._prompt_lists is None:
            raise StepError("prepare_prompt: run one prompt step first (it shows which tile lists the model's parts use)")
        self._prompt_graph_for((_row_bucket(n_tokens), _bucket(n_seqs), _bucket(n_wanted) if n_wanted else 0))

    def _prompt_graph_for(self, key) -> _PromptGraph:
        g = self._prompt_graphs.pop(key, None)
        if g is None:
            while len(self._prompt_graphs) >= MAX_PROMPT_GRAPHS:
                self._prompt_graphs.pop(next(iter(self._prompt_graphs)))        # the one unused for longest
            qts, page_tiles = self._prompt_lists
            g = _PromptGraph(self, key[0], key[1], key[2], qts, page_tiles)
            self.graphs_built += 1
        self._prompt_graphs[key] = g                                            # most recently used last
        return g

    def _step_prompt_graph(self, entries, slots, n_new, pos0):
        g = self._prompt_graph_for(self._prompt_key(entries, n_new))
        tokens = [int(t) for e in entries for t in e.tokens]
        want, row = [], 0
        for e, n in zip(entries, n_new):
            want += [row + int(w) for w in e.want]
            row += n
        g.fill(slots, tokens, n_new, pos0, want, self)
        g.upload()
        logits = g.run()
        return logits[:len(want)].clone()

    def prepare_decode(self, n_seqs: int) -> None:
        """Captures, now, every graph that decode steps of up to n_seqs sequences will replay (the batch
        shrinks as sequences end), so that no later step waits for a capture.  Does nothing for what is there."""
        if not self.use_graphs or self.tap is not None:
            return
        top = _bucket(min(max(n_seqs, 1), MAX_GRAPH_ROWS))
        for rows in reversed([b for b in DECODE_BUCKETS if b <= top]):
            self._graph_for(rows)

    def _graph_for(self, rows: int) -> _DecodeGraph:
        g = self._graphs.get(rows)
        if g is None:
            g = _DecodeGraph(self, rows)
            self._graphs[rows] = g
            self.graphs_built += 1
        return g

    def _step_graph(self, entries, slots, pos0, device_tokens=None):
        B = len(entries)
        lens_after = [p + 1 for p in pos0]
        g = self._graph_for(_bucket(B))
        g.fill(slots, [int(e.tokens[0]) for e in entries], lens_after, self)
        g.upload()
        if device_tokens is not None:
            g.tokens[:B].copy_(device_tokens)            # behind the upload, before the replay
        logits = g.run()
        rows = [i for i, e in enumerate(entries) for _ in e.want]
        if rows == list(range(B)):
            return logits[:B].clone()
        idx = torch.tensor(rows, dtype=torch.long, device=self.device)
        return logits.index_select(0, idx)
