"""The cache manager: pages of keys and values with a block table per request, and slots
for per-request state of fixed size.  Host-side bookkeeping only; the device tensors that
the pages index belong to the engine.

The reference gives every request private pages that it allocates lazily and returns when
the request's buffer is closed (core/src/main/java/io/teknek/deliverance/tensor/
KvBufferCache.java:826-841,851-865); there is no pool with a limit and nothing is shared
between requests.  Here a pool of fixed size serves all requests:

* A *group* is a set of cache slots (one per caching layer call) with the same needs: all
  keys, or a window of the last w.  Each group has pages of its own; one page id names the
  same page in every slot of the group.
* A request's *block table* for a group lists the page of each run of ``page_size``
  positions; the entry is -1 once a window has passed that run and the page went back.
* ``extend`` reserves pages for a request's next tokens (all groups or nothing);
  ``commit`` makes them part of the request and returns pages that a window has passed;
  ``close`` returns everything.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np


class CacheError(RuntimeError):
    """Misuse of the cache manager (unknown request, double free, ...)."""


class OutOfPages(CacheError):
    """Not enough free pages (or state slots) for what was asked."""


@dataclass(frozen=True)
class KVGroupSpec:
    """Cache slots that share pages.  ``window`` None keeps every key."""
    slots: Tuple[int, ...]
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size for one cache slot: ``elems`` 32-bit floats."""
    slot: int
    elems: int


class PagePool:
    """Page ids 0..n-1 with an owner each; free ids are handed out lowest first after reuse
    in last-freed-first order."""

    def __init__(self, n_pages: int):
        if n_pages < 0:
            raise CacheError("a pool cannot have a negative number of pages")
        self.n_pages = n_pages
        self._free: List[int] = list(range(n_pages - 1, -1, -1))
        self._owner: List[Optional[Hashable]] = [None] * n_pages

    @property
    def n_free(self) -> int:
        return len(self._free)

    def take(self, n: int, owner: Hashable) -> List[int]:
        if owner is None:
            raise CacheError("pages need an owner")
        if n > len(self._free):
            raise OutOfPages(f"asked for {n} pages, {len(self._free)} free of {self.n_pages}")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._owner[p] = owner
        return out

    def give(self, pages: Sequence[int], owner: Hashable) -> None:
        for p in pages:
            if p < 0 or p >= self.n_pages:
                raise CacheError(f"page {p} is not in the pool")
            if self._owner[p] is None:
                raise CacheError(f"page {p} freed twice")
            if self._owner[p] != owner:
                raise CacheError(f"page {p} belongs to {self._owner[p]!r}, not to {owner!r}")
            self._owner[p] = None
            self._free.append(p)

    def owner_of(self, page: int):
        return self._owner[page]


@dataclass
class _Request:
    length: int = 0                     # positions committed
    pending: int = 0                    # positions reserved by extend, not yet committed
    tables: List[List[int]] = field(default_factory=list)   # per group
    state_slot: int = -1


class CacheManager:
    def __init__(self, groups: Sequence[KVGroupSpec], page_size: int, pages_per_group: Sequence[int],
                 state_specs: Sequence[StateSpec] = (), n_state_slots: int = 0):
        if page_size <= 0:
            raise CacheError("page_size must be positive")
        if len(groups) != len(pages_per_group):
            raise CacheError("one page count per group is needed")
        self.groups = list(groups)
        self.page_size = page_size
        self.pools = [PagePool(n) for n in pages_per_group]
        self.state_specs = list(state_specs)
        self.n_state_slots = n_state_slots
        self._free_slots: List[int] = list(range(n_state_slots - 1, -1, -1))
        self._slot_owner: List[Optional[Hashable]] = [None] * n_state_slots
        self._reqs: Dict[Hashable, _Request] = {}
        # called with (group, pages) whenever pages go back to a pool (a debug run poisons them)
        self.on_release: Optional[Callable[[int, Sequence[int]], None]] = None

    # ---- requests ----------------------------------------------------------------
    def __contains__(self, rid) -> bool:
        return rid in self._reqs

    def live(self):
        return list(self._reqs.keys())

    def open(self, rid: Hashable) -> int:
        """Start a request; returns its state slot (-1 when the model keeps no state)."""
        if rid in self._reqs:
            raise CacheError(f"request {rid!r} is already open")
        slot = -1
        if self.n_state_slots:
            if not self._free_slots:
                raise OutOfPages(f"no state slot free of {self.n_state_slots}")
            slot = self._free_slots.pop()
            self._slot_owner[slot] = rid
        self._reqs[rid] = _Request(tables=[[] for _ in self.groups], state_slot=slot)
        return slot

    def can_open(self) -> bool:
        return self.n_state_slots == 0 or bool(self._free_slots)

    def _req(self, rid) -> _Request:
        try:
            return self._reqs[rid]
        except KeyError:
            raise CacheError(f"request {rid!r} is not open") from None

    def length(self, rid) -> int:
        return self._req(rid).length

    def pending(self, rid) -> int:
        """Positions reserved beyond ``length`` and not yet committed."""
        return self._req(rid).pending

    def state_slot(self, rid) -> int:
        return self._req(rid).state_slot

    def table(self, rid, group: int) -> List[int]:
        return self._req(rid).tables[group]

    # ---- pages -------------------------------------------------------------------
    def _first_live_page(self, group: int, first_query_pos: int) -> int:
        """Index of the first page a query at ``first_query_pos`` or later can still see."""
        w = self.groups[group].window
        if w is None:
            return 0
        lo = max(0, first_query_pos - w + 1)
        return lo // self.page_size

    def pages_needed(self, rid, n_new: int) -> List[int]:
        """New pages per group to hold positions [length, length + pending + n_new)."""
        r = self._req(rid)
        end = r.length + r.pending + n_new
        want = -(-end // self.page_size)
        return [max(0, want - len(t)) for t in r.tables]

    def can_extend(self, rid, n_new: int) -> bool:
        return all(n <= pool.n_free for n, pool in zip(self.pages_needed(rid, n_new), self.pools))

    def extend(self, rid, n_new: int) -> int:
        """Reserve room for ``n_new`` more positions; returns the first new position.
        Either every group gets its pages or nothing changes."""
        if n_new <= 0:
            raise CacheError("extend needs a positive number of positions")
        r = self._req(rid)
        need = self.pages_needed(rid, n_new)
        for n, pool in zip(need, self.pools):
            if n > pool.n_free:
                raise OutOfPages(
                    f"request {rid!r} needs {need} new pages per group, free: {[p.n_free for p in self.pools]}")
        for g, (n, pool) in enumerate(zip(need, self.pools)):
            r.tables[g].extend(pool.take(n, rid))
        start = r.length + r.pending
        r.pending += n_new
        return start

    def _give(self, group: int, pages: Sequence[int], rid) -> None:
        self.pools[group].give(pages, rid)
        if pages and self.on_release is not None:
            self.on_release(group, pages)

    def commit(self, rid, n: Optional[int] = None) -> List[Tuple[int, int]]:
        """The reserved positions (the first ``n`` of them, when given: a later step may have
        reserved more already) now belong to the request.  Pages that every later query
        has left behind (window groups) go back; returns them as (group, page)."""
        r = self._req(rid)
        k = r.pending if n is None else n
        if not (0 <= k <= r.pending):
            raise CacheError(f"request {rid!r}: cannot commit {k} of {r.pending} reserved positions")
        r.length += k
        r.pending -= k
        released = []
        for g, pool in enumerate(self.pools):
            first = self._first_live_page(g, r.length)     # the next query sits at r.length
            t = r.tables[g]
            for j in range(min(first, len(t))):
                if t[j] >= 0:
                    self._give(g, [t[j]], rid)
                    released.append((g, t[j]))
                    t[j] = -1
        return released

    def rollback(self, rid) -> None:
        """Drop a reservation that was never run (pages beyond the committed length go back)."""
        r = self._req(rid)
        keep = -(-r.length // self.page_size)
        for g, pool in enumerate(self.pools):
            t = r.tables[g]
            extra = [p for p in t[keep:] if p >= 0]
            self._give(g, extra, rid)
            del t[keep:]
        r.pending = 0

    def close(self, rid) -> None:
        """End of a request: every page and the state slot go back."""
        r = self._req(rid)
        for g in range(len(self.pools)):
            self._give(g, [p for p in r.tables[g] if p >= 0], rid)
        if r.state_slot >= 0:
            if self._slot_owner[r.state_slot] != rid:
                raise CacheError(f"state slot {r.state_slot} is not held by {rid!r}")
            self._slot_owner[r.state_slot] = None
            self._free_slots.append(r.state_slot)
        del self._reqs[rid]

    # ---- addressing --------------------------------------------------------------
    def slots_for(self, rid, group: int, start: int, n: int) -> List[int]:
        """Cache row (page * page_size + offset) of positions start .. start+n-1."""
        t = self._req(rid).tables[group]
        ps = self.page_size
        if n > 16:                                   # long portions: the same by arrays
            pos = np.arange(start, start + n, dtype=np.int64)
            pages = np.asarray(t, dtype=np.int64)[pos // ps]
            if (pages < 0).any():
                p = int(pos[pages < 0][0])
                raise CacheError(f"position {p} of {rid!r} lies in a page that was given back")
            return (pages * ps + pos % ps).tolist()
        out = []
        for p in range(start, start + n):
            page = t[p // ps]
            if page < 0:
                raise CacheError(f"position {p} of {rid!r} lies in a page that was given back")
            out.append(page * ps + p % ps)
        return out

    # ---- invariants (used by tests and by debug runs) ------------------------------
    def check(self) -> None:
        for g, pool in enumerate(self.pools):
            held = {}
            for rid, r in self._reqs.items():
                for p in r.tables[g]:
                    if p < 0:
                        continue
                    if p in held:
                        raise CacheError(f"group {g}: page {p} held by {held[p]!r} and {rid!r}")
                    held[p] = rid
                    if pool.owner_of(p) != rid:
                        raise CacheError(f"group {g}: page {p} in the table of {rid!r} but owned by {pool.owner_of(p)!r}")
                want = -(-(r.length + r.pending) // self.page_size)
                if len(r.tables[g]) != want:
                    raise CacheError(f"group {g}: table of {rid!r} has {len(r.tables[g])} entries for "
                                     f"{r.length + r.pending} positions")
            free = pool._free
            if len(set(free)) != len(free):
                raise CacheError(f"group {g}: a page is on the free list twice")
            if set(free) & set(held):
                raise CacheError(f"group {g}: a page is both free and held")
            if len(free) + len(held) != pool.n_pages:
                raise CacheError(f"group {g}: {len(free)} free + {len(held)} held != {pool.n_pages} pages")
        slots = [r.state_slot for r in self._reqs.values() if r.state_slot >= 0]
        if len(set(slots)) != len(slots):
            raise CacheError("a state slot is held twice")
        if self.n_state_slots and len(slots) + len(self._free_slots) != self.n_state_slots:
            raise CacheError("state slots lost")

    def stats(self) -> dict:
        return {"pages_free": [p.n_free for p in self.pools], "pages_total": [p.n_pages for p in self.pools],
                "requests": len(self._reqs), "state_slots_free": len(self._free_slots)}
