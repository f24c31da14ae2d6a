"""Cache manager: pages of keys and values, block tables per request, state slots.

Layers whose mixers have the same needs (kv heads, head size, window) form a group;
each group has a page pool of its own and every live request a block table per group
(logical page -> physical page). A request gets a slot at admission; the slot indexes
the block tables and the per-request state tensors of fixed size. Pages are taken when
positions need them, given back when a window has passed them or the request ends,
and used again, last freed first.

All bookkeeping is host-side Python and needs no GPU; device memory is allocated only
if a device is given.

Reference: ``kestrel/kv_cache.py:271-452`` (block table, free page and free row lists,
LIFO reuse, ``reserve``/``erase``), ``:88-132`` (per-layer ``[pages, Hkv, page_size, hd]``
tensors), ``:236-268`` (per-layer specs, ``None`` for layers without keys and values);
per-request state keyed by the row id: ``kestrel/runtime/uncached_paged.py:178-186``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..parts.base import LayerCache
from ..parts.specs import CacheSpec, StateSpec


class OutOfPages(RuntimeError):
    """A group's pool cannot back the positions asked for."""


class PagePool:
    """Free list of one group's physical pages with promises for admitted requests."""

    def __init__(self, n_pages: int) -> None:
        if n_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.n_pages = n_pages
        self._free: List[int] = list(reversed(range(n_pages)))  # page 0 is handed out first
        self._is_free = [True] * n_pages
        self.promised_unheld = 0

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def available(self) -> int:
        """Pages that are neither held nor promised to an admitted request."""
        return len(self._free) - self.promised_unheld

    def take(self, count: int) -> List[int]:
        if count > len(self._free):
            raise OutOfPages(f"{count} pages wanted, {len(self._free)} free of {self.n_pages}")
        pages = [self._free.pop() for _ in range(count)]
        for p in pages:
            self._is_free[p] = False
        return pages

    def give_back(self, pages: Sequence[int]) -> None:
        for p in pages:
            if not 0 <= p < self.n_pages:
                raise AssertionError(f"page {p} does not exist")
            if self._is_free[p]:
                raise AssertionError(f"page {p} freed twice")
            self._is_free[p] = True
            self._free.append(p)


@dataclass
class _Group:
    spec: CacheSpec
    entries: List[int]                 # schedule entries that own a cache in this group
    pool: PagePool
    # per tensor the specification names: [len(entries), pages, *shape of a page]; for attention
    # "k" [.., Hkv, page_size, hd] and "v" [.., Hkv, hd, page_size]
    tensors: Dict[str, torch.Tensor] = field(default_factory=dict)

    @property
    def k(self) -> Optional[torch.Tensor]:
        return self.tensors.get("k")

    @property
    def v(self) -> Optional[torch.Tensor]:
        return self.tensors.get("v")


class _SlotState:
    __slots__ = ("tables", "length", "quota", "first_page")

    def __init__(self, n_groups: int) -> None:
        self.tables: List[List[int]] = [[] for _ in range(n_groups)]   # -1 = given back
        self.length = 0                                                 # positions backed so far
        self.quota: List[int] = [0] * n_groups                          # pages promised at admission
        self.first_page: List[int] = [0] * n_groups                     # logical pages below it are given back


class CacheManager:
    """``needs``: per schedule entry ``(CacheSpec or None, StateSpec or None, reads_cache_of)``."""

    def __init__(self, needs, page_size: int, n_pages: int, max_requests: int, dtype: torch.dtype = torch.float32,
                 device: Optional[torch.device] = None) -> None:
        if page_size <= 0 or n_pages <= 0 or max_requests <= 0:
            raise ValueError("page_size, n_pages and max_requests must be positive")
        self.page_size, self.n_pages, self.max_requests = page_size, n_pages, max_requests
        self.dtype, self.device = dtype, device
        self.needs = list(needs)
        self.groups: List[_Group] = []
        by_key: Dict[Tuple, int] = {}
        self._entry_group: List[Optional[int]] = [None] * len(self.needs)
        self._entry_index: List[Optional[int]] = [None] * len(self.needs)
        for entry, (cache_spec, _state, reads) in enumerate(self.needs):
            if reads is not None or cache_spec is None:
                continue
            key = cache_spec.group_key
            if key not in by_key:
                by_key[key] = len(self.groups)
                self.groups.append(_Group(cache_spec, [], PagePool(n_pages)))
            g = by_key[key]
            self._entry_group[entry] = g
            self._entry_index[entry] = len(self.groups[g].entries)
            self.groups[g].entries.append(entry)
        for entry, (cache_spec, _state, reads) in enumerate(self.needs):
            if reads is None:
                continue
            owner_spec = self.needs[reads][0]
            if cache_spec is None or owner_spec is None or cache_spec.group_key != owner_spec.group_key:
                raise ValueError(f"schedule entry {entry} cannot read the cache of entry {reads}: their needs differ")
            self._entry_group[entry] = self._entry_group[reads]
            self._entry_index[entry] = self._entry_index[reads]
        self._free_slots: List[int] = list(reversed(range(max_requests)))
        self._slots: Dict[int, _SlotState] = {}
        self.states: List[Optional[torch.Tensor]] = [None] * len(self.needs)
        if device is not None:
            self._allocate_device()

    # ------------------------------------------------------------------ device memory
    def _allocate_device(self) -> None:
        for group in self.groups:
            # the layout of a page is the specification's business, not the manager's
            for name, shape in group.spec.page_tensors(self.page_size).items():
                group.tensors[name] = torch.zeros((len(group.entries), self.n_pages, *shape), dtype=self.dtype,
                                                  device=self.device)
        for entry, (_c, state_spec, _r) in enumerate(self.needs):
            if state_spec is not None:
                # one row more than there are slots: the last one is a spare that rows without a
                # request (slot -1, the rows that pad a captured batch) may read and write
                self.states[entry] = torch.zeros((self.max_requests + 1, *state_spec.shape),
                                                 dtype=getattr(torch, state_spec.dtype), device=self.device)

    def bytes_per_page(self) -> int:
        size = torch.empty((), dtype=self.dtype).element_size()
        total = 0
        for g in self.groups:
            for shape in g.spec.page_tensors(self.page_size).values():
                count = 1
                for extent in shape:
                    count *= int(extent)
                total += len(g.entries) * count * size
        return total

    def layer_caches(self) -> List[LayerCache]:
        """One ``LayerCache`` per schedule entry."""
        out = []
        for entry, (cache_spec, _state, reads) in enumerate(self.needs):
            g = self._entry_group[entry]
            tensors = {}
            if g is not None:
                tensors = {name: t[self._entry_index[entry]] for name, t in self.groups[g].tensors.items()}
            out.append(LayerCache(group=g, tensors=tensors, writes=reads is None, state=self.states[entry]))
        return out

    # ------------------------------------------------------------------ sizes
    def pages_for(self, group: int, length: int, portion: int = 1) -> int:
        """Pages a request of ``length`` tokens holds at most in ``group`` when it is fed in
        portions of at most ``portion`` tokens."""
        full = -(-length // self.page_size)
        window = self.groups[group].spec.window
        if window is None:
            return full
        # live keys span at most window - 1 + portion positions, which touch one page more
        return min(full, -(-(window - 1 + portion) // self.page_size) + 1)

    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    @property
    def live_slots(self) -> List[int]:
        return sorted(self._slots)

    def pages_available(self, group: int = 0) -> int:
        return self.groups[group].pool.available

    def can_admit(self, length: int, portion: int = 1) -> bool:
        """A free slot, and in every group enough pages that nobody was promised."""
        if not self._free_slots:
            return False
        return all(self.pages_for(g, length, portion) <= grp.pool.available for g, grp in enumerate(self.groups))

    # ------------------------------------------------------------------ life of a request
    def admit(self, reserve_length: int = 0, portion: int = 1) -> int:
        """A slot for a new request. ``reserve_length`` > 0 promises it the pages for that
        many tokens, so that later ``ensure`` calls up to there cannot fail."""
        if not self._free_slots:
            raise OutOfPages("no free request slot")
        quotas = [self.pages_for(g, reserve_length, portion) if reserve_length else 0
                  for g in range(len(self.groups))]
        for g, grp in enumerate(self.groups):
            if quotas[g] > grp.pool.available:
                raise OutOfPages(f"Cannot reserve {quotas[g]} pages for a sequence of length {reserve_length}. "
                                 f"Only {grp.pool.available} pages available.")
        slot = self._free_slots.pop()
        state = _SlotState(len(self.groups))
        state.quota = quotas
        for g, grp in enumerate(self.groups):
            grp.pool.promised_unheld += quotas[g]
        self._slots[slot] = state
        for tensor in self.states:
            if tensor is not None:
                tensor[slot].zero_()
        return slot

    def _held(self, state: _SlotState, g: int) -> int:
        return sum(1 for p in state.tables[g] if p >= 0)

    def _owed(self, state: _SlotState, g: int) -> int:
        """Pages promised to the request that it does not hold yet."""
        return max(0, state.quota[g] - self._held(state, g))

    def ensure(self, slot: int, length: int) -> None:
        """Back positions ``[0, length)`` of the request (beyond what a window gave back)
        in every group; nothing changes if any group cannot."""
        state = self._slots[slot]
        if length <= state.length:
            return
        needs = []
        for g, grp in enumerate(self.groups):
            need = max(0, -(-length // self.page_size) - len(state.tables[g]))
            beyond_promise = need - min(need, self._owed(state, g))
            if beyond_promise > grp.pool.available:
                raise OutOfPages(f"Cannot reserve {need} pages for a sequence of length {length} in slot {slot}. "
                                 f"Only {grp.pool.available + need - beyond_promise} pages available.")
            needs.append(need)
        for g, grp in enumerate(self.groups):
            if needs[g]:
                before = self._owed(state, g)
                state.tables[g].extend(grp.pool.take(needs[g]))
                grp.pool.promised_unheld += self._owed(state, g) - before
        state.length = length

    def trim(self, slot: int, length: int) -> int:
        """Give back the pages of windowed groups that no position >= ``length`` reads any
        more. Returns the number of pages freed."""
        state = self._slots[slot]
        freed = 0
        for g, grp in enumerate(self.groups):
            window = grp.spec.window
            if window is None:
                continue
            first_needed = max(0, length + 1 - window)        # lowest key the next query reads
            dead_below = min(first_needed // self.page_size, len(state.tables[g]))
            before = self._owed(state, g)
            dead = []
            for logical in range(state.first_page[g], dead_below):
                if state.tables[g][logical] >= 0:
                    dead.append(state.tables[g][logical])
                    state.tables[g][logical] = -1
            state.first_page[g] = max(state.first_page[g], dead_below)
            if dead:
                grp.pool.give_back(dead)
                # a promise covers the pages held at one time: a page given back is owed again
                grp.pool.promised_unheld += self._owed(state, g) - before
                freed += len(dead)
        return freed

    def release(self, slot: int) -> None:
        """The request has ended: all its pages and its slot are given back."""
        state = self._slots.pop(slot, None)
        if state is None:
            raise AssertionError(f"slot {slot} released twice or never admitted")
        for g, grp in enumerate(self.groups):
            held = [p for p in state.tables[g] if p >= 0]
            grp.pool.promised_unheld -= self._owed(state, g)
            grp.pool.give_back(list(reversed(held)))
        self._free_slots.append(slot)

    # ------------------------------------------------------------------ views
    def length(self, slot: int) -> int:
        return self._slots[slot].length

    def block_table(self, group: int, slot: int) -> List[int]:
        return self._slots[slot].tables[group]

    def slot_of_position(self, group: int, slot: int, position: int) -> int:
        """``page * page_size + offset`` of a position (``kestrel/kv_cache.py:524-551``)."""
        page = self._slots[slot].tables[group][position // self.page_size]
        if page < 0:
            raise AssertionError(f"position {position} of slot {slot} was given back")
        return page * self.page_size + position % self.page_size

    def window_start(self, group: int, position: int) -> int:
        window = self.groups[group].spec.window
        return 0 if window is None else max(0, position + 1 - window)

    # ------------------------------------------------------------------ invariants
    def check(self) -> None:
        """No page lost, held twice or both held and free; promises add up."""
        for g, grp in enumerate(self.groups):
            seen: Dict[int, int] = {}
            for slot, state in self._slots.items():
                for p in state.tables[g]:
                    if p < 0:
                        continue
                    if p in seen:
                        raise AssertionError(f"group {g}: page {p} held by slots {seen[p]} and {slot}")
                    seen[p] = slot
            free = list(grp.pool._free)
            if len(set(free)) != len(free):
                raise AssertionError(f"group {g}: a page is in the free list twice")
            if set(free) & set(seen):
                raise AssertionError(f"group {g}: pages both held and free: {sorted(set(free) & set(seen))}")
            if len(free) + len(seen) != grp.pool.n_pages:
                raise AssertionError(f"group {g}: {grp.pool.n_pages - len(free) - len(seen)} pages lost")
            owed = sum(self._owed(s, g) for s in self._slots.values())
            if owed != grp.pool.promised_unheld:
                raise AssertionError(f"group {g}: promises {grp.pool.promised_unheld} != owed {owed}")
        if len(set(self._free_slots)) != len(self._free_slots) or set(self._free_slots) & set(self._slots):
            raise AssertionError("slot bookkeeping broken")
        if len(self._free_slots) + len(self._slots) != self.max_requests:
            raise AssertionError("a slot was lost")
