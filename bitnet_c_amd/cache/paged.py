"""The cache: what every live sequence keeps between steps.

A *slot* stands for one sequence: its length, its pages in every group, its row of the
state area.  Keys and values live in pages of PAGE positions; a page id addresses the
same page in every entry of its group.  Entries of the schedule whose mixers need the
same kind of storage (same kv heads, key and value widths, value layout and window: equal
KVNeed) form a *group* with storage,
a page pool and block tables of its own, so a group that keeps a window of keys gives
pages back while a sequence grows and a group that keeps all keys does not.  Beside the
pages there is a state area: for every entry that asks for it, a tensor of fixed shape
per slot, zero when a slot is handed out, with one more row at index `padding_slot` that no
sequence owns: the padding rows of a captured step address it, so that a mixer which reads
and writes its state by the step's device-side slot ids needs no special case for them.

The reference gives each request a session with contiguous [layer][position][kv_dim]
arrays and a zeroed recurrent state (src/model_session.c:332-368, src/session.c:113-172)
and wraps positions past the end (src/transformer.c:139); here a sequence that would
outgrow the cache is an error and changes nothing.

All bookkeeping is host-side Python and runs without a GPU; storage is allocated on
`device` (None: bookkeeping only).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import torch

from ..csrc.build import header_constant
from ..ops import kernel_v_layout
from ..parts.base import CacheNeed, KVNeed, KVView

PAGE = header_constant("BN_PAGE")        # positions per page: defined once, in csrc/common.h


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    pass


class PagePool:
    """Page ids 0..n-1; a page is either free or held by exactly one owner."""

    def __init__(self, n_pages: int):
        self.n_pages = int(n_pages)
        self._free = list(range(self.n_pages - 1, -1, -1))     # pop() hands out the lowest id first
        self._held = [False] * self.n_pages

    @property
    def n_free(self) -> int:
        return len(self._free)

    def take(self, n: int) -> List[int]:
        if n > len(self._free):
            raise CacheFull(f"{n} pages wanted, {len(self._free)} of {self.n_pages} free")
        got = [self._free.pop() for _ in range(n)]
        for p in got:
            self._held[p] = True
        return got

    def give_back(self, pages: Sequence[int]) -> None:
        for p in pages:
            if not (0 <= p < self.n_pages) or not self._held[p]:
                raise CacheError(f"page {p} is given back but is not held")
            self._held[p] = False
            self._free.append(p)

    def check(self) -> None:
        if sorted(self._free) != [p for p in range(self.n_pages) if not self._held[p]]:
            raise CacheError("page pool is inconsistent: a page is lost or free twice")


@dataclass
class _Group:
    need: KVNeed
    entries: List[int]                       # schedule entries that own storage here, in order
    pool: PagePool
    pages: Dict[int, List[int]]              # slot -> page of each PAGE positions (-1: given back)
    v_transposed: bool = False               # the layout of v that the group's need asks for
    blocked: bool = False                    # keys and values in the matrix-core kernels' own order (sizes as v_transposed)
    k: Optional[torch.Tensor] = None         # [entries, pages, Hkv, PAGE, head_dim]
    v: Optional[torch.Tensor] = None         # [entries, pages, Hkv, PAGE, v_dim], or [.., v_dim, PAGE] when v_transposed


class PagedCache:
    @staticmethod
    def _layout(need: KVNeed, dtype) -> str:
        """The layout of a need's pages: what it names, else what this library's attention kernels read at the cache's
        type (and, where the values are as wide as the keys, at the head size)."""
        if need.v_layout:
            if need.v_layout == "blocked" and dtype != torch.bfloat16:
                raise CacheError("blocked pages are bf16 pages")
            return need.v_layout
        return kernel_v_layout(dtype, need.head_dim if need.v_dim == need.head_dim else 0)

    def __init__(self, needs: Sequence[CacheNeed], kv_from: Sequence[Optional[int]], max_tokens: int,
                 dtype=torch.bfloat16, device=None, max_slots: Optional[int] = None):
        """needs[i], kv_from[i]: what schedule entry i's mixer keeps, and the entry whose keys
        and values it reads instead of its own.  max_tokens: positions that all live sequences
        may hold together, each sequence's count rounded up to a multiple of PAGE."""
        if max_tokens < PAGE:
            raise CacheError(f"max_tokens {max_tokens} is below one page ({PAGE})")
        self.tables_version = 0          # grows whenever any sequence's list of pages changes
        self._slot_version: Dict[int, int] = {}   # slot -> tables_version at the last change of its pages
        self.n_pages = max_tokens // PAGE
        self.max_slots = int(max_slots) if max_slots else self.n_pages
        self.dtype, self.device = dtype, device
        self.groups: List[_Group] = []
        self._entry_group: List[Optional[tuple]] = []          # entry -> (group index, index in group)
        self.kv_from = list(kv_from)
        by_need: Dict[KVNeed, int] = {}
        for i, need in enumerate(needs):
            if need.kv is None or kv_from[i] is not None:
                self._entry_group.append(None)
                continue
            gi = by_need.get(need.kv)
            if gi is None:
                gi = len(self.groups)
                by_need[need.kv] = gi
                layout = self._layout(need.kv, dtype)                    # the need says how its values lie
                self.groups.append(_Group(need.kv, [], PagePool(self.n_pages), {}, v_transposed=layout != "rows",
                                          blocked=layout == "blocked"))
            self._entry_group.append((gi, len(self.groups[gi].entries)))
            self.groups[gi].entries.append(i)
        for i, src in enumerate(kv_from):
            if src is not None:
                if self._entry_group[src] is None:
                    raise CacheError(f"entry {i} reads the cache of entry {src}, which keeps none")
                a, b = needs[i].kv, needs[src].kv
                if a is not None and b is not None and (
                        (a.n_kv_heads, a.head_dim, a.v_dim) != (b.n_kv_heads, b.head_dim, b.v_dim)
                        or self._layout(a, dtype) != self._layout(b, dtype)):
                    raise CacheError(f"entry {i} reads the cache of entry {src} but their kv shapes or layouts differ")
                self._entry_group[i] = self._entry_group[src]
        self._free_slots = list(range(self.max_slots - 1, -1, -1))
        self._len: Dict[int, int] = {}
        self.states: Dict[int, torch.Tensor] = {}
        self._state_needs = {i: n.state for i, n in enumerate(needs) if n.state is not None}
        if device is not None:
            for g in self.groups:
                lead = (len(g.entries), self.n_pages, g.need.n_kv_heads)
                g.k = torch.zeros(lead + (PAGE, g.need.head_dim), dtype=dtype, device=device)
                g.v = torch.zeros(lead + ((g.need.v_dim, PAGE) if g.v_transposed else (PAGE, g.need.v_dim)),
                                  dtype=dtype, device=device)
            for i, sn in self._state_needs.items():
                self.states[i] = torch.zeros((self.max_slots + 1,) + tuple(sn.shape), dtype=sn.dtype, device=device)

    @property
    def padding_slot(self) -> int:
        """The row of the state area that belongs to no sequence."""
        return self.max_slots

    def _touch(self, slot: int) -> None:
        self.tables_version += 1
        self._slot_version[slot] = self.tables_version

    def slot_version(self, slot: int) -> int:
        """A number that changes whenever the slot's pages change or the slot is handed out again."""
        return self._slot_version[slot]

    def pages_of(self, group: int, slot: int) -> List[int]:
        return self.groups[group].pages[slot]

    # ---- slots ------------------------------------------------------------------
    def alloc_slot(self) -> int:
        if not self._free_slots:
            raise CacheFull(f"all {self.max_slots} sequence slots are in use")
        s = self._free_slots.pop()
        self._len[s] = 0
        self._touch(s)
        for g in self.groups:
            g.pages[s] = []
        for t in self.states.values():
            t[s].zero_()
        return s

    def free_slot(self, slot: int) -> None:
        if slot not in self._len:
            raise CacheError(f"slot {slot} is freed but is not in use")
        self._touch(slot)
        for g in self.groups:
            g.pool.give_back([p for p in g.pages.pop(slot) if p >= 0])
        del self._len[slot]
        self._free_slots.append(slot)

    def length(self, slot: int) -> int:
        if slot not in self._len:
            raise CacheError(f"slot {slot} is not in use")
        return self._len[slot]

    def live_slots(self) -> List[int]:
        return sorted(self._len)

    @property
    def n_free_slots(self) -> int:
        return len(self._free_slots)

    # ---- growth -----------------------------------------------------------------
    def reserve(self, slots: Sequence[int], n_new: Sequence[int]) -> None:
        """Pages for positions [len, len + n_new) of every slot, in every group; either all of
        it happens or none (CacheFull)."""
        if len(set(slots)) != len(slots):
            raise CacheError("a slot appears twice in one step")
        plan = []
        for g in self.groups:
            want = 0
            for s, n in zip(slots, n_new):
                have = len(g.pages[s]) if s in g.pages else None
                if have is None:
                    raise CacheError(f"slot {s} is not in use")
                need = (self._len[s] + n + PAGE - 1) // PAGE - have
                plan.append((g, s, max(0, need)))
                want += max(0, need)
            if want > g.pool.n_free:
                raise CacheFull(f"the step needs {want} more pages of {PAGE} positions, "
                                f"{g.pool.n_free} of {g.pool.n_pages} are free")
        for g, s, need in plan:
            if need:
                g.pages[s].extend(g.pool.take(need))
                self._touch(s)

    def unreserve(self, slots: Sequence[int]) -> None:
        """Gives back what reserve() took for a step that did not run: every page beyond the slot's length."""
        for s in slots:
            if s not in self._len:
                continue
            keep = (self._len[s] + PAGE - 1) // PAGE
            for g in self.groups:
                pl = g.pages[s]
                if len(pl) > keep:
                    g.pool.give_back([p for p in pl[keep:] if p >= 0])
                    del pl[keep:]
                    self._touch(s)

    def commit(self, slots: Sequence[int], n_new: Sequence[int]) -> None:
        """The step has run: lengths grow; groups that keep a window give back the pages that
        no later position can see."""
        for s, n in zip(slots, n_new):
            self._len[s] += n
            for g in self.groups:
                if g.need.window > 0:
                    first_visible = self._len[s] - g.need.window + 1     # for the next position
                    pl = g.pages[s]
                    for i in range(len(pl)):
                        if pl[i] >= 0 and PAGE * i + PAGE - 1 < first_visible:
                            g.pool.give_back([pl[i]])
                            pl[i] = -1
                            self._touch(s)

    # ---- views ------------------------------------------------------------------
    def group_of(self, entry: int) -> Optional[int]:
        eg = self._entry_group[entry]
        return None if eg is None else eg[0]

    def block_table(self, group: int, slots: Sequence[int], width: int = 0) -> torch.Tensor:
        """Host int32 [len(slots), width]; a slot of -1 gives a row of zeros (padding).  A page that a windowed
        group has given back (-1 in the slot's list) appears as page 0: no kernel reads below a window, and if one
        ever did it would read a page that exists."""
        g = self.groups[group]
        w = max([width, 1] + [len(g.pages[s]) for s in slots if s >= 0])
        bt = torch.zeros((len(slots), w), dtype=torch.int32)
        for r, s in enumerate(slots):
            if s >= 0:
                pl = g.pages[s]
                if pl:
                    bt[r, :len(pl)] = torch.tensor(pl, dtype=torch.int32).clamp_(min=0)
        return bt

    def view(self, entry: int, block_tables: Dict[int, torch.Tensor], max_len: int) -> KVView:
        eg = self._entry_group[entry]
        st = self.states.get(entry)
        if eg is None:
            return KVView(state=st, writes=False, max_len=max_len)
        gi, idx = eg
        g = self.groups[gi]
        return KVView(k_pages=g.k[idx] if g.k is not None else None,
                      v_pages=g.v[idx] if g.v is not None else None,
                      v_transposed=g.v_transposed, blocked=g.blocked, block_table=block_tables.get(gi),
                      writes=self.kv_from[entry] is None, state=st, max_len=max_len)

    def check(self) -> None:
        """No page lost, held twice or free twice; no slot both free and in use."""
        for g in self.groups:
            g.pool.check()
            held = [p for pl in g.pages.values() for p in pl if p >= 0]
            if len(held) != len(set(held)):
                raise CacheError("a page is held by two sequences")
            if len(held) + g.pool.n_free != g.pool.n_pages:
                raise CacheError("a page is lost")
            if set(g.pages) != set(self._len):
                raise CacheError("a group's slots differ from the live slots")
        if set(self._free_slots) & set(self._len) or len(self._free_slots) + len(self._len) != self.max_slots:
            raise CacheError("a slot is lost or both free and in use")
