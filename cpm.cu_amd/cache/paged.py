"""The sequence cache: a slot per live sequence, pages of tokens per slot.

What the model's mixers need is declared as ``CacheNeeds`` (per-token streams
such as keys and values, fixed-size per-slot state, all tokens or a trailing
window).  Cache entries with equal needs form a *group*; each group has page
pool storage of its own and a page table of its own, so a group that keeps a
window gives old pages back while a group that keeps everything does not.

A slot is acquired when a sequence starts and released when it ends; its pages
return to the pools and its fixed-size state is zeroed at the next acquire.
Tokens are addressed as (slot, position); a stream's row for a token lies at
``page_table[slot, position // page_size] * rows_per_page + (position % page_size) // every``.

The reference engine holds one sequence in one contiguous buffer per layer
(src/model/kvcache.cuh:7-65) plus compressed-key buffers beside it
(src/model/minicpm4/minicpm4_kvcache.cuh:204-255); slots, pages and groups are
this engine's own.  All bookkeeping is host-side Python over plain lists; the
device sees the page tables and the pools.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch


class CacheError(RuntimeError):
    pass


@dataclass(frozen=True)
class StreamSpec:
    """One row of ``width`` elements for every ``every`` tokens."""
    width: int
    every: int = 1
    dtype: Optional[torch.dtype] = None       # None: the engine's element type


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size state per slot, zeroed when a slot is acquired."""
    shape: Tuple[int, ...]
    dtype: Optional[torch.dtype] = None


@dataclass(frozen=True)
class CacheNeeds:
    """What one cache entry (a mixer's storage) asks for."""
    streams: Tuple[Tuple[str, StreamSpec], ...] = ()
    state: Tuple[Tuple[str, StateSpec], ...] = ()
    window: Optional[int] = None              # None: keep every token; w: only the last w tokens are read

    def group_key(self):
        return (self.streams, self.state, self.window)


@dataclass
class CacheView:
    """What a mixer sees of its cache entry."""
    streams: Dict[str, torch.Tensor]          # name -> [n_pages, page_size // every, width]
    state: Dict[str, torch.Tensor]            # name -> [max_slots, *shape]
    page_table: Optional[torch.Tensor]        # int32 [max_slots, table_width] of the entry's group
    page_size: int
    window: Optional[int]


class _Group:
    def __init__(self, needs: CacheNeeds, entries: List[int], n_pages: int, max_slots: int, table_width: int,
                 page_size: int, device, dtype):
        self.needs = needs
        self.entries = entries
        self.n_pages = n_pages
        self.page_size = page_size
        self.free_pages: List[int] = list(range(n_pages - 1, -1, -1))   # pop() gives the lowest page first
        # host page table: slot -> list of physical pages by page number (-1: given back / never held)
        self.pages: List[List[int]] = [[] for _ in range(max_slots)]
        self.table = torch.zeros((max_slots, table_width), dtype=torch.int32, device=device)
        self.table_host = torch.zeros((max_slots, table_width), dtype=torch.int32)
        self.dirty: set = set()
        self.storage: Dict[int, Dict[str, torch.Tensor]] = {}
        self.state: Dict[int, Dict[str, torch.Tensor]] = {}
        for e in entries:
            self.storage[e] = {}
            for name, s in needs.streams:
                if page_size % s.every:
                    raise CacheError(f"cache stream '{name}' keeps a row every {s.every} tokens, which does not "
                                     f"divide the page of {page_size} tokens")
                self.storage[e][name] = torch.zeros((n_pages, page_size // s.every, s.width),
                                                    dtype=s.dtype or dtype, device=device)
            self.state[e] = {name: torch.zeros((max_slots,) + tuple(s.shape), dtype=s.dtype or dtype, device=device)
                             for name, s in needs.state}

    def held(self, slot: int) -> int:
        return sum(1 for p in self.pages[slot] if p >= 0)


def _element_size(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


def _window_pages(window: int, step: int, page_size: int) -> int:
    """The most pages a sequence holds in a group that keeps a trailing window, when it grows by at most
    ``step`` tokens at once: the step's first query still reads window - 1 tokens back."""
    return (step + window - 2) // page_size + 2


def _pool_pages(needs: CacheNeeds, n_pages: int, max_slots: int, max_seq_len: int, step: int, page_size: int) -> int:
    """Pages of a group's pool: a group that keeps every token gets one for every page of tokens the cache
    holds; a group that keeps a window never holds more than its window's pages for every slot."""
    if needs.window is None:
        return n_pages
    per_slot = min(-(-max_seq_len // page_size), _window_pages(needs.window, step, page_size))
    return min(n_pages, max_slots * per_slot)


class SequenceCache:
    """Slots, pages and per-slot state for all cache entries of a model."""

    @staticmethod
    def plan_bytes(needs: Sequence[CacheNeeds], max_tokens: int, max_slots: int, max_seq_len: int,
                   page_size: int, dtype: torch.dtype, max_step_tokens: Optional[int] = None) -> int:
        """Device bytes of a cache built with these arguments (pools, per-slot state, page tables), without
        building it: what an engine checks against its memory limit beforehand."""
        n_pages = -(-max_tokens // page_size)
        seq_pages = -(-max_seq_len // page_size)
        step = max_step_tokens or max_seq_len
        total = 0
        seen = set()
        for n in needs:
            pool = _pool_pages(n, n_pages, max_slots, max_seq_len, step, page_size)
            for _, st in n.streams:
                total += pool * (page_size // st.every) * st.width * _element_size(st.dtype or dtype)
            for _, st in n.state:
                count = 1
                for d in st.shape:
                    count *= int(d)
                total += max_slots * count * _element_size(st.dtype or dtype)
            if n.group_key() not in seen:
                seen.add(n.group_key())
                total += max_slots * (seq_pages if n.window is not None else min(seq_pages, n_pages)) * 4
        return total

    @staticmethod
    def tokens_for(needs: Sequence[CacheNeeds], budget_bytes: int, max_slots: int, max_seq_len: int,
                   page_size: int, dtype: torch.dtype, max_step_tokens: Optional[int] = None) -> int:
        """The most tokens (a whole number of pages, at most max_slots sequences of max_seq_len) whose cache fits
        ``budget_bytes``; 0 if not even a page for every slot does."""
        hi = max_slots * (-(-max_seq_len // page_size))

        def fits(pages: int) -> bool:
            return SequenceCache.plan_bytes(needs, pages * page_size, max_slots, max_seq_len, page_size, dtype,
                                            max_step_tokens) <= budget_bytes
        if not fits(max_slots):
            return 0
        lo = max_slots
        while lo < hi:
            mid = (lo + hi + 1) // 2
            if fits(mid):
                lo = mid
            else:
                hi = mid - 1
        return lo * page_size

    def __init__(self, needs: List[CacheNeeds], max_tokens: int, max_slots: int, max_seq_len: int,
                 page_size: int = 64, device="cpu", dtype=torch.float32, max_step_tokens: Optional[int] = None):
        if page_size <= 0 or max_tokens <= 0 or max_slots <= 0 or max_seq_len <= 0:
            raise CacheError("cache sizes must be positive")
        self.max_step_tokens = int(max_step_tokens or max_seq_len)
        self.page_size = page_size
        self.max_slots = max_slots
        self.max_seq_len = max_seq_len
        self.device = torch.device(device)
        self.dtype = dtype
        self.n_pages = -(-max_tokens // page_size)
        seq_pages = -(-max_seq_len // page_size)
        # a page table has an entry for every page number a sequence can reach: a group that keeps every token
        # cannot hold more pages than its pool has, a group that keeps a window can (it gives old pages back)
        self.table_width = min(seq_pages, self.n_pages)
        self.groups: List[_Group] = []
        self.entry_group: List[int] = []
        by_key: Dict[object, List[int]] = {}
        for e, n in enumerate(needs):
            by_key.setdefault(n.group_key(), []).append(e)
        self.entry_group = [0] * len(needs)
        for key, entries in by_key.items():
            width = seq_pages if needs[entries[0]].window is not None else self.table_width
            pool = _pool_pages(needs[entries[0]], self.n_pages, max_slots, max_seq_len, self.max_step_tokens, page_size)
            g = _Group(needs[entries[0]], entries, pool, max_slots, width, page_size, self.device, dtype)
            for e in entries:
                self.entry_group[e] = len(self.groups)
            self.groups.append(g)
        self._has_window = any(g.needs.window is not None for g in self.groups)
        self.has_state = any(g.needs.state for g in self.groups)
        self.free_slots: List[int] = list(range(max_slots - 1, -1, -1))
        self.live: Dict[int, int] = {}        # slot -> tokens held
        self._views: Dict[int, CacheView] = {}

    # ---- slots ----
    def acquire(self) -> int:
        if not self.free_slots:
            raise CacheError(f"no free slot: all {self.max_slots} are held by live sequences")
        slot = self.free_slots.pop()
        self.live[slot] = 0
        for g in self.groups:
            for e in g.entries:
                for t in g.state[e].values():
                    t[slot].zero_()
        return slot

    def release(self, slot: int):
        if slot not in self.live:
            raise CacheError(f"slot {slot} is not held (released twice, or never acquired)")
        for g in self.groups:
            for p in g.pages[slot]:
                if p >= 0:
                    g.free_pages.append(p)
            g.pages[slot] = []
        del self.live[slot]
        self.free_slots.append(slot)

    def length(self, slot: int) -> int:
        try:
            return self.live[slot]
        except KeyError:
            raise CacheError(f"slot {slot} is not held by a live sequence") from None

    # ---- tokens ----
    def _first_kept(self, g: _Group, old: int) -> int:
        """The first page number a group still needs when the next query sits at position ``old``."""
        if g.needs.window is None:
            return 0
        return max(old - g.needs.window + 1, 0) // self.page_size

    def _group_need(self, g: _Group, slot: int, old: int, new: int) -> Tuple[int, int]:
        """(pages the group must take, pages it gives back first) to grow the slot from old to new tokens."""
        pages = g.pages[slot]
        n_pg = -(-new // self.page_size)
        if g.needs.window is None:
            return max(n_pg - len(pages), 0), 0
        first_kept = self._first_kept(g, old)
        need = max(n_pg - max(len(pages), first_kept), 0)
        need += sum(1 for pn in range(first_kept, min(len(pages), n_pg)) if pages[pn] < 0)
        freed = 0
        for pn in range(min(first_kept, len(pages)) - 1, -1, -1):
            if pages[pn] < 0:
                break
            freed += 1
        return need, freed

    def room_for(self, passes: Sequence[Sequence[Tuple[int, int]]]) -> Optional[str]:
        """None if the groups can take the tokens of a step that runs as these forward passes, each a list of
        (slot, n_new) extended one after the other, else the reason.  Nothing is changed: the passes are played
        through on counts alone.  Each group is asked for what it really needs: one that keeps a window gives
        pages back from pass to pass, so a long prompt may bring more tokens than its pool holds."""
        for gi, g in enumerate(self.groups):
            free = len(g.free_pages)
            state: Dict[int, Tuple[int, int, int]] = {}        # slot -> (tokens, first held page number, page numbers)
            for one in passes:
                for slot, n_new in one:
                    if slot not in state:
                        pages = g.pages[slot]
                        lo = next((pn for pn, p in enumerate(pages) if p >= 0), len(pages))
                        state[slot] = (self.length(slot), lo, len(pages))
                    old, lo, hi = state[slot]
                    new = old + n_new
                    first_kept = self._first_kept(g, old)
                    lo2 = max(lo, first_kept)
                    free += max(min(lo2, hi) - lo, 0)                  # given back before anything is taken
                    hi2 = -(-new // self.page_size)
                    need = max(hi2 - max(hi, first_kept), 0)
                    if need > free:
                        return (f"the cache is full: this step needs {need} more pages of {self.page_size} tokens"
                                f"{'' if len(self.groups) == 1 else f' in cache group {gi}'} for slot {slot}, "
                                f"{free} are free of {g.n_pages}")
                    free -= need
                    state[slot] = (new, lo2, max(hi, hi2))
        return None

    def pages_to_hold(self, length: int, step: int) -> List[int]:
        """Per group, the most pages a sequence of ``length`` tokens holds at any time when it grows by at most
        ``step`` tokens at once (what a planner reserves for it)."""
        out = []
        for g in self.groups:
            full = -(-length // self.page_size)
            if g.needs.window is None:
                out.append(full)
            else:
                out.append(min(full, _window_pages(g.needs.window, step, self.page_size)))
        return out

    def capacity(self) -> List[int]:
        """Pages of each group's pool."""
        return [g.n_pages for g in self.groups]

    def free_page_count(self) -> int:
        return min(len(g.free_pages) for g in self.groups) if self.groups else self.n_pages

    def extend(self, slot: int, n_new: int) -> int:
        """Make room for n_new more tokens of the slot; returns the position of the first of them."""
        old = self.length(slot)
        new = old + n_new
        if n_new <= 0:
            raise CacheError(f"slot {slot}: a step must bring at least one token")
        if new > self.max_seq_len:
            raise CacheError(f"slot {slot}: {new} tokens exceed the longest sequence this engine holds "
                             f"({self.max_seq_len})")
        n_pg = -(-new // self.page_size)
        # check every group before touching any, so a refused step changes nothing
        for g in self.groups:
            need, freed = self._group_need(g, slot, old, new)
            if need > len(g.free_pages) + freed:
                raise CacheError(f"the cache is full: slot {slot} needs {need} more pages of {self.page_size} tokens, "
                                 f"{len(g.free_pages) + freed} are free of {g.n_pages}")
        for g in self.groups:
            pages = g.pages[slot]
            # the step's first query (position `old`) still reads back to old - window + 1
            first_kept = self._first_kept(g, old)
            changed = []
            for pn in range(min(first_kept, len(pages)) - 1, -1, -1):
                if pages[pn] < 0:
                    break                       # everything before an entry given back was given back earlier
                g.free_pages.append(pages[pn])
                pages[pn] = -1
                changed.append(pn)
            while len(pages) < n_pg:
                pn = len(pages)
                pages.append(g.free_pages.pop() if pn >= first_kept else -1)
                changed.append(pn)
            if changed:
                row = g.table_host[slot]
                for pn in changed:
                    row[pn] = max(pages[pn], 0)
                g.dirty.add(slot)
        self.live[slot] = new
        return old

    def truncate(self, slot: int, length: int):
        """Forget the slot's tokens from ``length`` on (a step that failed after extend): their pages return
        to the pools.  Pages that a windowed group gave back while the slot grew stay given back, so a group
        that keeps a window can only go back to a length whose next query reads none of them (the start of the
        slot's last extend always is one); a shorter length is refused and nothing changes."""
        have = self.length(slot)
        if not 0 <= length <= have:
            raise CacheError(f"slot {slot}: cannot truncate {have} tokens to {length}")
        n_pg = -(-length // self.page_size)
        for gi, g in enumerate(self.groups):
            if g.needs.window is None:
                continue
            pages = g.pages[slot]
            gone = [pn for pn in range(self._first_kept(g, length), min(n_pg, len(pages))) if pages[pn] < 0]
            if gone:
                raise CacheError(f"slot {slot}: cannot truncate to {length} tokens: cache group {gi} keeps a window of "
                                 f"{g.needs.window} tokens and has already given back page {gone[0]}, which the query "
                                 f"at position {length} would read")
        for g in self.groups:
            pages = g.pages[slot]
            while len(pages) > n_pg:
                p = pages.pop()
                if p >= 0:
                    g.free_pages.append(p)
        self.live[slot] = length

    # ---- fixed-size state ----
    def snapshot_state(self, slots: Sequence[int]):
        """Copies of the slots' fixed-size state (None when no entry has any): what restore_state puts back
        after a forward pass that advanced the state and then failed."""
        if not self.has_state:
            return None
        idx = torch.tensor(list(slots), dtype=torch.long).to(self.device)
        return idx, [[(t, t.index_select(0, idx)) for t in g.state[e].values()] for g in self.groups for e in g.entries]

    def restore_state(self, snapshot):
        if snapshot is None:
            return
        idx, saved = snapshot
        for entry in saved:
            for t, rows in entry:
                t.index_copy_(0, idx, rows)

    def extend_one(self, slot: int) -> int:
        """extend(slot, 1) for the decode loop: nothing but the length changes while the token fits the
        slot's last page and no group drops pages."""
        old = self.live[slot]
        if old % self.page_size and not self._has_window:
            self.live[slot] = old + 1
            return old
        return self.extend(slot, 1)

    def sync(self):
        """Copy the page-table rows that changed to the device (before kernels read them)."""
        for g in self.groups:
            if not g.dirty:
                continue
            if self.device.type == "cpu":
                g.table.copy_(g.table_host)
            else:
                rows = sorted(g.dirty)
                idx = torch.tensor(rows, dtype=torch.long)
                g.table.index_copy_(0, idx.to(self.device), g.table_host[idx].to(self.device))
            g.dirty.clear()

    # ---- views ----
    def view(self, entry: int) -> CacheView:
        v = self._views.get(entry)
        if v is None:
            g = self.groups[self.entry_group[entry]]
            v = CacheView(g.storage[entry], g.state[entry], g.table, self.page_size, g.needs.window)
            self._views[entry] = v
        return v

    # ---- accounting (tests and reports) ----
    def check(self):
        """Every page is free or held exactly once; every slot is free or live exactly once."""
        for gi, g in enumerate(self.groups):
            held = [p for pages in g.pages for p in pages if p >= 0]
            allp = held + g.free_pages
            if len(allp) != g.n_pages or len(set(allp)) != g.n_pages:
                raise CacheError(f"group {gi}: pages lost or held twice ({len(held)} held, {len(g.free_pages)} free, "
                                 f"{g.n_pages} in all)")
        slots = list(self.live) + self.free_slots
        if len(slots) != self.max_slots or len(set(slots)) != self.max_slots:
            raise CacheError("slots lost or held twice")
        for s in range(self.max_slots):
            if s not in self.live and any(g.pages[s] for g in self.groups):
                raise CacheError(f"free slot {s} still holds pages")

    def bytes(self) -> int:
        n = 0
        for g in self.groups:
            for d in list(g.storage.values()) + list(g.state.values()):
                n += sum(t.numel() * t.element_size() for t in d.values())
        return n
