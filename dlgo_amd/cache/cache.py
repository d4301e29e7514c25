"""The cache: a slot for each live sequence, paged keys and values for each run
of a layer, and fixed-size per-sequence state beside them.

computerex/dlgo keeps one sequence: per layer `Keys, Vals [maxPos][kvDim]` and a
length (memory/kvcache.go:5-36), reset by setting the length to zero without
clearing (kvcache.go:25-27,74-78), and for recurrent layers a fixed-size state
that is zero-filled on reset (memory/ssmstate.go:4-69).  Here:

* a *slot* is one live sequence: its length and, per group, the pages it holds;
* cache units (one per run of a layer that keeps keys/values) with equal needs
  (kv heads, head size, window) form a *group* with storage of its own: a pool of
  pages of 64 tokens, one page id covering all units of the group, and a page
  table [slot, page index] the kernels read.  A windowed group gives pages back
  as soon as no later token can see them and has a smaller pool;
* giving a slot back returns its pages at once; data is never cleared, because
  attention reads positions below the length only;
* fixed-size state lives in [slot, ...] tensors per unit and is zeroed when a
  slot is handed out.

The bookkeeping is plain host code and runs without a GPU.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..parts.base import CacheNeed

PAGE = 64


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    pass


class PagePool:
    """Free list of page ids with double-free and foreign-id checks."""

    def __init__(self, n_pages: int):
        self.n_pages = n_pages
        self._free = list(range(n_pages - 1, -1, -1))   # pop() hands out low ids first
        self._held = np.zeros(n_pages, dtype=bool)

    @property
    def n_free(self) -> int:
        return len(self._free)

    def take(self, n: int) -> List[int]:
        if n > len(self._free):
            raise OutOfPages(f"cache full: {n} pages wanted, {len(self._free)} of {self.n_pages} free")
        out = [self._free.pop() for _ in range(n)]
        self._held[out] = True
        return out

    def give(self, pages: Sequence[int]) -> None:
        for p in pages:
            if not (0 <= p < self.n_pages) or not self._held[p]:
                raise CacheError(f"page {p} given back but not held")
            self._held[p] = False
            self._free.append(p)


@dataclass
class GroupSpec:
    kv_heads: int
    head_dim: int
    window: Optional[int]
    units: List[int] = field(default_factory=list)     # cache unit ids, in storage order


class KVGroup:
    def __init__(self, spec: GroupSpec, n_pages: int, max_slots: int, max_pages_per_seq: int,
                 dtype: torch.dtype, device: torch.device):
        self.spec = spec
        self.pool = PagePool(n_pages)
        self.unit_elems = 2 * spec.kv_heads * PAGE * spec.head_dim     # keys then values of one unit in a page
        self.page_stride = self.unit_elems * len(spec.units)
        self.v_off = spec.kv_heads * PAGE * spec.head_dim
        # never cleared and never read beyond a sequence's length
        self.storage = torch.empty(n_pages * self.page_stride, dtype=dtype, device=device)
        self.table_host = np.full((max_slots, max_pages_per_seq), -1, dtype=np.int32)
        self.table = torch.full((max_slots, max_pages_per_seq), -1, dtype=torch.int32, device=device)
        self.dirty: set = set()
        self.version = 0             # counts the changes of table_host: who keeps a copy of some rows knows when it is stale

    def touch(self, slot: int) -> None:
        """Row `slot` of the page table changed on the host."""
        self.dirty.add(slot)
        self.version += 1

    def unit_view(self, index_in_group: int) -> torch.Tensor:
        """Storage from the first element of this unit's part of page 0."""
        return self.storage[index_in_group * self.unit_elems:]

    def first_needed_page(self, length: int) -> int:
        """Lowest page index that a token at position >= length can still see."""
        if self.spec.window is None:
            return 0
        lo = length - self.spec.window + 1
        return max(0, lo) // PAGE


class Cache:
    def __init__(self, unit_needs: Sequence[Sequence[CacheNeed]], max_tokens: int, max_ctx: int, dtype: torch.dtype,
                 device, max_slots: Optional[int] = None, max_step_tokens: Optional[int] = None):
        """unit_needs[u]: what cache unit u asks for.  max_tokens: the most tokens live sequences hold together,
        each sequence rounded up to whole pages.  max_ctx: the longest sequence."""
        self.device = torch.device(device)
        self.dtype = dtype
        if max_tokens < 1 or max_ctx < 1:
            raise CacheError("cache: max_tokens and max_ctx must be positive")
        self.n_pages = (max_tokens + PAGE - 1) // PAGE
        self.max_ctx = min(max_ctx, self.n_pages * PAGE)
        self.max_pages_per_seq = (self.max_ctx + PAGE - 1) // PAGE
        self.max_slots = max_slots if max_slots is not None else min(self.n_pages, 4096)
        self.max_step_tokens = max_step_tokens or self.max_ctx

        self.groups: List[KVGroup] = []
        self.unit_group: Dict[int, Tuple[int, int]] = {}     # unit -> (group index, index in group)
        self.state: Dict[int, torch.Tensor] = {}            # unit -> [max_slots, *shape]
        specs: Dict[Tuple[int, int, Optional[int]], GroupSpec] = {}
        for u, needs in enumerate(unit_needs):
            for need in needs:
                if need.kind == "kv":
                    key = (need.kv_heads, need.head_dim, need.window)
                    if need.kv_heads < 1 or need.head_dim < 1 or (need.window is not None and need.window < 1):
                        raise CacheError(f"cache unit {u}: bad key/value need {need}")
                    spec = specs.setdefault(key, GroupSpec(*key))
                    if u in self.unit_group:
                        raise CacheError(f"cache unit {u} asks for keys/values twice")
                    self.unit_group[u] = (list(specs).index(key), len(spec.units))
                    spec.units.append(u)
                elif need.kind == "state":
                    if u in self.state:
                        raise CacheError(f"cache unit {u} asks for state twice")
                    self.state[u] = torch.zeros((self.max_slots, *need.state_shape), dtype=need.state_dtype, device=self.device)
                elif need.kind != "none":
                    raise CacheError(f"cache unit {u}: unknown need kind {need.kind!r}")
        for spec in specs.values():
            n_pages = self.n_pages
            per_seq = self.max_pages_per_seq
            if spec.window is not None:
                per_seq = min(per_seq, (spec.window + min(self.max_step_tokens, self.max_ctx) + PAGE - 1) // PAGE + 1)
                n_pages = min(n_pages, self.max_slots * per_seq)
            group = KVGroup(spec, n_pages, self.max_slots, self.max_pages_per_seq, dtype, self.device)
            group.pages_per_seq = per_seq       # the most pages one sequence holds of this group at any time
            self.groups.append(group)

        self._stages: list = []          # staging for sync_tables
        self._stage_next = 0
        self._free_slots = list(range(self.max_slots - 1, -1, -1))
        self._live = np.zeros(self.max_slots, dtype=bool)
        self.lengths = np.zeros(self.max_slots, dtype=np.int64)
        # pages held per slot and group: page index -> page id
        self._held: List[List[Dict[int, int]]] = [[{} for _ in self.groups] for _ in range(self.max_slots)]

    # -- slots ---------------------------------------------------------------
    @property
    def n_free_slots(self) -> int:
        return len(self._free_slots)

    def live_slots(self) -> List[int]:
        return [int(s) for s in np.nonzero(self._live)[0]]

    def alloc_slot(self) -> int:
        if not self._free_slots:
            raise CacheError(f"no free slot: all {self.max_slots} are in use")
        slot = self._free_slots.pop()
        self._live[slot] = True
        self.lengths[slot] = 0
        for t in self.state.values():
            t[slot].zero_()
        return slot

    def free_slot(self, slot: int) -> None:
        self._check_live(slot)
        for gi, g in enumerate(self.groups):
            held = self._held[slot][gi]
            g.pool.give(list(held.values()))
            if held:
                g.table_host[slot, list(held.keys())] = -1
                g.touch(slot)
            held.clear()
        self._live[slot] = False
        self.lengths[slot] = 0
        self._free_slots.append(slot)

    def copy_slot(self, src: int, length: Optional[int] = None) -> int:
        """A new slot that holds what `src` holds below `length` (all of it by default): keys and values are copied page
        by page into pages of its own, per-sequence state is copied as it is now.  computerex/dlgo: KVCache.Clone
        (memory/kvcache.go:38-55).  State is not a function of a length, so with state units only the whole sequence
        can be copied; a windowed group must still hold every page that a token at `length` sees."""
        self._check_live(src)
        have = int(self.lengths[src])
        n = have if length is None else int(length)
        if n < 0 or n > have:
            raise CacheError(f"copy_slot: slot {src} holds {have} tokens, {n} asked")
        if n != have and self.state:
            raise CacheError("copy_slot: per-sequence state cannot be copied at an earlier length")
        if not self._free_slots:
            raise CacheError(f"no free slot: all {self.max_slots} are in use")
        plans = []
        for gi, g in enumerate(self.groups):
            held = self._held[src][gi]
            last = (n - 1) // PAGE if n > 0 else -1
            idx = list(range(g.first_needed_page(n), last + 1))
            missing = [i for i in idx if i not in held]
            if missing:
                raise CacheError(f"copy_slot: slot {src} no longer holds pages {missing} that a token at {n} sees")
            if len(idx) > g.pool.n_free:
                raise OutOfPages(f"cache full: the copy needs {len(idx)} pages of {PAGE} tokens, {g.pool.n_free} of {g.pool.n_pages} are free")
            plans.append(idx)
        dst = self.alloc_slot()
        for gi, (g, idx) in enumerate(zip(self.groups, plans)):
            if not idx:
                continue
            pages = g.pool.take(len(idx))
            src_pages = [self._held[src][gi][i] for i in idx]
            for i, p in zip(idx, pages):
                self._held[dst][gi][i] = p
                g.table_host[dst, i] = p
            g.touch(dst)
            by_page = g.storage.view(g.pool.n_pages, g.page_stride)
            if self.device.type != "cuda":
                by_page[torch.as_tensor(pages, dtype=torch.int64)] = by_page[torch.as_tensor(src_pages, dtype=torch.int64)]
                continue
            # the page numbers travel as the changed table rows do (pinned, in a copy that nothing waits for); the pages
            # are copied by the library's own kernel
            from ..kernels import ops
            k = len(pages)
            st = self._table_stage(2 * k)
            st[0].numpy()[:k] = src_pages
            st[0].numpy()[k:2 * k] = pages
            st[2][:2 * k].copy_(st[0][:2 * k], non_blocking=True)
            ops.copy_rows(by_page, by_page, src_rows=st[2][:k], dst_rows=st[2][k:2 * k], n=k)
            ev = torch.cuda.Event()
            ev.record()
            st[4] = ev
        self.lengths[dst] = n
        for t in self.state.values():
            t[dst].copy_(t[src])
        return dst

    def _check_live(self, slot: int) -> None:
        if not (0 <= slot < self.max_slots) or not self._live[slot]:
            raise CacheError(f"slot {slot} is not in use")

    def length(self, slot: int) -> int:
        self._check_live(slot)
        return int(self.lengths[slot])

    # -- pages ---------------------------------------------------------------
    def pages_wanted(self, slot: int, new_len: int, group: int) -> List[int]:
        """Page indices the slot lacks in `group` to hold positions below new_len."""
        g = self.groups[group]
        held = self._held[slot][group]
        first = g.first_needed_page(int(self.lengths[slot]))
        last = (new_len - 1) // PAGE
        return [i for i in range(first, last + 1) if i not in held]

    def can_reserve(self, wants: Sequence[Tuple[int, int]]) -> Optional[str]:
        """None if every (slot, new_len) fits, else the reason."""
        for slot, new_len in wants:
            self._check_live(slot)
            if new_len > self.max_ctx:
                return f"slot {slot}: {new_len} tokens exceed the context of {self.max_ctx}"
        for gi, g in enumerate(self.groups):
            # a windowed group: a sequence never holds more than its window and the longest piece of a step, because
            # each piece gives back what no later token sees before the next piece asks for more
            if g.spec.window is None:
                need = sum(len(self.pages_wanted(s, n, gi)) for s, n in wants)
            else:
                need = sum(min(len(self.pages_wanted(s, n, gi)), max(0, g.pages_per_seq - len(self._held[s][gi]))) for s, n in wants)
            if need > g.pool.n_free:
                return f"cache full: the step needs {need} more pages of {PAGE} tokens, {g.pool.n_free} of {g.pool.n_pages} are free"
        return None

    def page_demand(self, n_tokens: int) -> Tuple[int, ...]:
        """Per group: the most pages a sequence that grows to n_tokens holds at any time (a windowed group: its window
        and the longest step, whatever the length)."""
        whole = (min(n_tokens, self.max_ctx) + PAGE - 1) // PAGE
        return tuple(whole if g.spec.window is None else min(whole, g.pages_per_seq) for g in self.groups)

    def free_pages(self) -> Tuple[int, ...]:
        """Per group: pages that new sequences can still take."""
        return tuple(g.pool.n_free for g in self.groups)

    def reserve(self, wants: Sequence[Tuple[int, int]]) -> None:
        """Make room so that each slot can hold positions below its new length."""
        why = self.can_reserve(wants)
        if why:
            raise OutOfPages(why)
        for gi, g in enumerate(self.groups):
            for slot, new_len in wants:
                idx = self.pages_wanted(slot, new_len, gi)
                if not idx:
                    continue
                pages = g.pool.take(len(idx))
                for i, p in zip(idx, pages):
                    self._held[slot][gi][i] = p
                    g.table_host[slot, i] = p
                g.touch(slot)

    def advance(self, slot: int, n_tokens: int) -> None:
        """The slot now holds n_tokens more; pages no later token can see go back to their pool."""
        self._check_live(slot)
        self.lengths[slot] += n_tokens
        for gi, g in enumerate(self.groups):
            if g.spec.window is None:
                continue
            first = g.first_needed_page(int(self.lengths[slot]))
            held = self._held[slot][gi]
            gone = [i for i in held if i < first]
            if gone:
                g.pool.give([held.pop(i) for i in gone])
                g.table_host[slot, gone] = -1
                g.touch(slot)

    @property
    def has_windows(self) -> bool:
        return any(g.spec.window is not None for g in self.groups)

    def advance_many(self, slots: np.ndarray, n_tokens: int) -> None:
        """advance() for several live slots at once."""
        if self.has_windows:
            for s in slots:
                self.advance(int(s), n_tokens)
        else:
            self.lengths[slots] += n_tokens

    def _table_stage(self, n_rows: int):
        """Pinned host buffers (row numbers, rows) that no copy in flight still reads, and their device twins."""
        if not self._stages:
            self._stages = [None] * 4
        i = self._stage_next
        self._stage_next = (i + 1) % len(self._stages)
        st = self._stages[i]
        if st is not None and st[4] is not None:
            st[4].synchronize()
        if st is None or st[0].shape[0] < n_rows:
            cap = max(2 * n_rows, 64)
            st = [torch.empty(cap, dtype=torch.int32, pin_memory=True),
                  torch.empty((cap, self.max_pages_per_seq), dtype=torch.int32, pin_memory=True),
                  torch.empty(cap, dtype=torch.int32, device=self.device),
                  torch.empty((cap, self.max_pages_per_seq), dtype=torch.int32, device=self.device), None]
            self._stages[i] = st
        return st

    def sync_tables(self) -> None:
        """Bring the device page tables up to date (rows of slots that changed).  The rows travel through pinned memory in
        copies that the host does not wait for: a copy from ordinary memory would hold it until the device has caught up,
        and a loop that queues a step ahead would lose its lead at every page a sequence begins."""
        for g in self.groups:
            if not g.dirty:
                continue
            rows = sorted(g.dirty)
            g.dirty.clear()
            if self.device.type != "cuda":
                g.table.index_copy_(0, torch.as_tensor(rows, dtype=torch.int64), torch.from_numpy(g.table_host[rows]))
                continue
            n = len(rows)
            st = self._table_stage(n)
            st[0].numpy()[:n] = rows
            st[1].numpy()[:n] = g.table_host[rows]
            st[2][:n].copy_(st[0][:n], non_blocking=True)
            st[3][:n].copy_(st[1][:n], non_blocking=True)
            from ..kernels import ops
            ops.copy_rows(st[3], g.table, dst_rows=st[2], n=n)        # table[rows[i]] = the staged row i
            ev = torch.cuda.Event()
            ev.record()
            st[4] = ev

    # -- views for the parts --------------------------------------------------
    def kv_view(self, unit: int) -> "KVView":
        gi, ui = self.unit_group[unit]
        g = self.groups[gi]
        return KVView(g.unit_view(ui), g.page_stride, g.v_off, g.table, g.spec.kv_heads, g.spec.head_dim, g.spec.window, gi)

    def state_of(self, unit: int) -> torch.Tensor:
        return self.state[unit]

    def held_pages(self, slot: int, group: int = 0) -> Dict[int, int]:
        return dict(self._held[slot][group])

    def check_consistent(self) -> None:
        """No page lost, none held twice (used by tests and cheap enough to call anywhere)."""
        for gi, g in enumerate(self.groups):
            seen: Dict[int, int] = {}
            for slot in range(self.max_slots):
                for i, p in self._held[slot][gi].items():
                    if not self._live[slot]:
                        raise CacheError(f"free slot {slot} holds page {p}")
                    if p in seen:
                        raise CacheError(f"page {p} held by slots {seen[p]} and {slot}")
                    seen[p] = slot
                    if g.table_host[slot, i] != p:
                        raise CacheError(f"page table of slot {slot} disagrees at index {i}")
            if len(seen) + g.pool.n_free != g.pool.n_pages:
                raise CacheError(f"group {gi}: {len(seen)} held + {g.pool.n_free} free != {g.pool.n_pages} pages")
        if len(self._free_slots) + int(self._live.sum()) != self.max_slots or len(set(self._free_slots)) != len(self._free_slots):
            raise CacheError("slot accounting broken")


def kv_bytes_per_token(unit_needs: Sequence[Sequence[CacheNeed]], dtype: torch.dtype) -> int:
    """Bytes of keys and values that one token adds over all cache units (a windowed unit counts like a full one)."""
    item = torch.empty(0, dtype=dtype).element_size()
    return sum(2 * need.kv_heads * need.head_dim * item for needs in unit_needs for need in needs if need.kind == "kv")


def tokens_that_fit(unit_needs: Sequence[Sequence[CacheNeed]], dtype: torch.dtype, free_bytes: int, recordings_bytes: int = 0,
                    keep_free: float = 0.2, reserve_bytes: int = 2 << 30) -> int:
    """How many tokens (a whole number of pages) a cache may be sized for when `free_bytes` of device memory are left:
    a fifth of it and 2 GiB stay free for the step's buffers, and `recordings_bytes` for what the recordings of steps
    will keep (they do not exist yet when the cache is sized)."""
    per_token = kv_bytes_per_token(unit_needs, dtype)
    budget = int(free_bytes * (1.0 - keep_free)) - reserve_bytes - int(recordings_bytes)
    if per_token == 0:
        return 1 << 20
    return max(0, budget // (per_token * PAGE)) * PAGE


@dataclass
class KVView:
    """What an attention kernel needs of one cache unit."""
    cache: torch.Tensor        # flat storage starting at this unit's part of page 0
    page_stride: int           # elements from a page to the next
    v_off: int                 # elements from a page's keys to its values
    page_table: torch.Tensor   # [max_slots, max_pages] int32 on the device
    kv_heads: int
    head_dim: int
    window: Optional[int]
    group: int = 0             # index of the storage group (its page table is shared by the group's units)
