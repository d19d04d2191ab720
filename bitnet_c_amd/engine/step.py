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
        the first), for kernels that store a page's positions together."""
        if self._page_tiles is None:
            self._page_tiles = torch.tensor(_page_tiles(self.n_new, self.pos0),
                                            dtype=torch.int32).reshape(-1, 4).to(self.device)
        return self._page_tiles

    def tiles(self, qt: int) -> torch.Tensor:
        """[n, 4] int32: (sequence, first row, rows <= qt, position of the first) covering all new
        tokens, for the prompt form of the attention kernel, in the order that gives its workgroups
        equal work (ops.pair_tiles)."""
        t = self._tiles.get(qt)
        if t is None:
            rows, r = [], 0
            for s, (n, p0) in enumerate(zip(self.n_new, self.pos0)):
                for i in range(0, n, qt):
                    rows.append((s, r + i, min(qt, n - i), p0 + i))
                r += n
            t = torch.tensor(ops.pair_tiles(rows), dtype=torch.int32).reshape(-1, 4).to(self.device)
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


def _by_length(lens) -> List[int]:
    """The rows ordered by length, longest first (ties by row)."""
    return sorted(range(len(lens)), key=lambda i: (-lens[i], i))


MAX_GRAPH_ROWS = 64       # decode steps of more sequences than this run eagerly


def _bucket(n: int) -> int:
    b = 1
    while b < n:
        b *= 2
    return b


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


class Engine:
    """A model, its cache and the step function over both."""

    def __init__(self, model: DecoderModel, max_tokens: int, max_seq_len: int = 0, max_slots: int = 0,
                 use_graphs: bool = True):
        ops.require_gpu()
        self.model, self.device = model, model.device
        needs, kv_from = model.cache_needs()
        self.cache = PagedCache(needs, kv_from, max_tokens, dtype=model.dtype, device=self.device,
                                max_slots=max_slots or None)
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
        # One captured step per number of rows (1, 2, 4 .. MAX_GRAPH_ROWS): at most seven, made at a batch's
        # start (prepare_decode) or at first use.  They share one memory pool: what a capture frees, the next
        # reuses, and each keeps only its own inputs and logits ([rows, vocab] float32).
        self._graphs: Dict[int, _DecodeGraph] = {}
        self.graph_pool = torch.cuda.graph_pool_handle() if self.use_graphs else None
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
                    max_seq_len: int = 0, max_slots: int = 0, use_graphs: bool = True, n_seqs: int = 1) -> "Engine":
        """max_tokens: positions that the cache holds; 0: n_seqs sequences of the longest length there can be
        (the model's max_positions, or max_seq_len when that is less: the reference sizes its cache by
        min(context length, --maxseq), src/model.c:256-257), or as many as fit into the free device memory."""
        ops.require_gpu()
        arch, config = load_config(folder)
        plan = arch.build_plan(config)
        model = DecoderModel(plan, dtype, device)
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

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Runs the entries' tokens as one batch; returns float32 logits [wanted, vocab] in the
        order of the entries and of each entry's `want`.  On an error nothing has changed."""
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        self._validate(entries)
        slots = [e.slot for e in entries]
        n_new = [len(e.tokens) for e in entries]
        pos0 = [self.cache.length(s) for s in slots]
        try:
            self.cache.reserve(slots, n_new)
        except CacheFull as err:
            raise StepError(str(err)) from None
        is_decode = all(n == 1 for n in n_new)
        try:
            if is_decode and self.use_graphs and self.tap is None and len(entries) <= MAX_GRAPH_ROWS:
                logits = self._step_graph(entries, slots, pos0)
            else:
                logits = self._step_eager(entries, slots, n_new, pos0, is_decode)
        except BaseException:
            self.cache.unreserve(slots)          # the step did not happen: its pages go back
            raise
        self.cache.commit(slots, n_new)
        self.steps_run += 1
        return logits

    def _step_eager(self, entries, slots, n_new, pos0, is_decode):
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
        d_order = take(len(order)) if is_decode else None
        d_tables = {g: take(tables[g].numel()).view(tables[g].shape) for g in sorted(tables)}
        ctx = StepContext(dev, self.model.dtype, d_tokens, d_pos, d_seq, d_lens, d_want, d_slots, is_decode,
                          slots, n_new, pos0, by_length=d_order)
        ctx.tap = self.tap
        max_len = max(lens_after)
        views = [self.cache.view(i, d_tables, max_len) for i in range(len(self.model.plan.schedule))]
        return self.model.forward(ctx, views)

    def prepare_decode(self, n_seqs: int) -> None:
        """Captures, now, every graph that decode steps of up to n_seqs sequences will replay (the batch
        shrinks as sequences end), so that no later step waits for a capture.  Does nothing for what is there."""
        if not self.use_graphs or self.tap is not None:
            return
        rows = _bucket(min(max(n_seqs, 1), MAX_GRAPH_ROWS))
        while rows >= 1:
            self._graph_for(rows)
            rows //= 2

    def _graph_for(self, rows: int) -> _DecodeGraph:
        g = self._graphs.get(rows)
        if g is None:
            g = _DecodeGraph(self, rows)
            self._graphs[rows] = g
            self.graphs_built += 1
        return g

    def _step_graph(self, entries, slots, pos0):
        B = len(entries)
        lens_after = [p + 1 for p in pos0]
        g = self._graph_for(_bucket(B))
        g.fill(slots, [int(e.tokens[0]) for e in entries], lens_after, self)
        g.upload()
        logits = g.run()
        rows = [i for i, e in enumerate(entries) for _ in e.want]
        if rows == list(range(B)):
            return logits[:B].clone()
        idx = torch.tensor(rows, dtype=torch.long, device=self.device)
        return logits.index_select(0, idx)
