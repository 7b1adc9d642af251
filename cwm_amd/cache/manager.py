"""The cache manager: pages of keys and values per layer group, a block table per
request and group, and slots for per-request state of fixed size.

Bookkeeping only (no device memory; see `storage.py` for the tensors).  The life
of a request:

    slot = manager.admit(rid)            # a state slot; tables start empty
    ok = manager.extend(rid, n_new)      # pages for positions [length, length+n_new)
    ... the step writes and reads the cache ...
    freed = manager.advance(rid, n_new)  # length += n_new; window groups give back
                                         # pages no later query can reach
    manager.release(rid)                 # everything back

`extend` is all-or-nothing over the groups: if any group lacks pages nothing is
taken and it returns False; the scheduler then decides what to do (it preempts).
Pages are given back after a step, never inside it: the first query of a portion
still reads window-1 keys before it.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Hashable, List, Mapping, Optional, Sequence, Union

from ..parts.base import CacheSpec, PagedKVSpec, StateSpec
from .pages import GroupTable, OutOfPages, PageAccountingError, PagePool, pages_for


@dataclass
class LayerGroup:
    """Cache slots whose layers keep the same span of keys: they share a pool and
    block tables, and each has pages of its own in device memory.  Which keys are
    kept is the answer of `spec`, the need of the group's first slot."""

    index: int
    spec: PagedKVSpec
    cache_ids: List[int]
    pool: PagePool

    @property
    def window(self) -> Optional[int]:
        return self.spec.window

    def first_page_needed(self, length: int, page_size: int) -> int:
        """Lowest logical page, pinned ones apart, that a query at position >= `length`
        can still read."""
        return self.spec.first_key_needed(length) // page_size

    def pinned_pages(self, page_size: int) -> int:
        """Logical pages at the start of a sequence that are never given back."""
        return pages_for(self.spec.pinned_keys(), page_size)

    def most_pages(self, length: int, step_tokens: int, page_size: int) -> int:
        """Most pages that a request of `length` tokens holds of this group at any time
        when a step brings at most `step_tokens` (a page of slack for where the span
        starts inside a page)."""
        need = pages_for(length, page_size)
        span = self.spec.keys_kept(step_tokens)
        if span is not None:
            need = min(need, self.pinned_pages(page_size) + pages_for(span, page_size) + 1)
        return need


class _Request:
    __slots__ = ("rid", "slot", "length", "tables")

    def __init__(self, rid: Hashable, slot: int, n_groups: int) -> None:
        self.rid = rid
        self.slot = slot
        self.length = 0
        self.tables = [GroupTable() for _ in range(n_groups)]


class CacheManager:
    def __init__(
        self,
        specs: Sequence[CacheSpec],
        page_size: int,
        num_pages: Union[int, Mapping[Optional[int], int]],
        max_requests: int,
    ) -> None:
        """`specs[i]` is what cache slot i needs (a `PagedKVSpec`, a `StateSpec` or
        None).  `num_pages` is the pool size of every group, or a mapping from a
        group's `retention()` (for the built-in need its window, None for the keep-all
        group) to its pool size."""
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        if max_requests <= 0:
            raise ValueError("max_requests must be positive")
        self.page_size = page_size
        self.max_requests = max_requests
        self.specs = list(specs)
        self.groups: List[LayerGroup] = []
        self.group_of_cache: Dict[int, int] = {}
        self.state_caches: List[int] = []
        by_retention: Dict[Hashable, LayerGroup] = {}
        for cid, spec in enumerate(self.specs):
            if isinstance(spec, PagedKVSpec):
                if spec.window is not None and spec.window < 1:
                    raise ValueError("a window holds at least one key")
                key = spec.retention()
                grp = by_retention.get(key)
                if grp is None:
                    if isinstance(num_pages, Mapping):
                        if key not in num_pages:
                            raise ValueError(f"no pool size given for the group that keeps {key!r}")
                        n = num_pages[key]
                    else:
                        n = num_pages
                    grp = LayerGroup(index=len(self.groups), spec=spec, cache_ids=[], pool=PagePool(n))
                    by_retention[key] = grp
                    self.groups.append(grp)
                grp.cache_ids.append(cid)
                self.group_of_cache[cid] = grp.index
            elif isinstance(spec, StateSpec):
                self.state_caches.append(cid)
            elif spec is not None:
                raise TypeError(f"cache slot {cid}: unknown cache need {spec!r}")
        self._free_slots = list(range(max_requests - 1, -1, -1))
        self._requests: Dict[Hashable, _Request] = {}

    # ---- requests ------------------------------------------------------------ #
    def has_free_slot(self) -> bool:
        return bool(self._free_slots)

    def __contains__(self, rid: Hashable) -> bool:
        return rid in self._requests

    def live_requests(self) -> List[Hashable]:
        return list(self._requests)

    def admit(self, rid: Hashable) -> int:
        """Give `rid` a state slot and empty tables; returns the slot."""
        if rid in self._requests:
            raise KeyError(f"request {rid!r} is already live")
        if not self._free_slots:
            raise OutOfPages("no free request slot")
        slot = self._free_slots.pop()
        self._requests[rid] = _Request(rid, slot, len(self.groups))
        return slot

    def slot(self, rid: Hashable) -> int:
        return self._requests[rid].slot

    def length(self, rid: Hashable) -> int:
        return self._requests[rid].length

    # ---- pages ---------------------------------------------------------------- #
    def pages_missing(self, rid: Hashable, n_new: int) -> List[int]:
        """Pages each group still has to take before `n_new` more tokens fit."""
        req = self._requests[rid]
        need = pages_for(req.length + n_new, self.page_size)
        return [max(0, need - len(req.tables[g.index].pages)) for g in self.groups]

    def can_extend(self, rid: Hashable, n_new: int) -> bool:
        missing = self.pages_missing(rid, n_new)
        return all(m <= g.pool.free_count for m, g in zip(missing, self.groups))

    def extend(self, rid: Hashable, n_new: int) -> bool:
        """Take the pages that positions [length, length + n_new) need in every
        group.  All or nothing."""
        if n_new <= 0:
            raise ValueError("extend needs at least one token")
        if not self.can_extend(rid, n_new):
            return False
        req = self._requests[rid]
        need = pages_for(req.length + n_new, self.page_size)
        for g in self.groups:
            table = req.tables[g.index]
            while len(table.pages) < need:
                table.pages.append(g.pool.take())
        return True

    def advance(self, rid: Hashable, n_new: int) -> List[List[int]]:
        """The step has written `n_new` tokens.  Returns, per group, the pages
        given back because no later query reads them (the window has passed them, and
        they are not pinned)."""
        req = self._requests[rid]
        new_len = req.length + n_new
        if any(len(req.tables[g.index].pages) < pages_for(new_len, self.page_size) for g in self.groups):
            raise PageAccountingError(f"request {rid!r} advanced past the pages it holds")
        req.length = new_len
        freed: List[List[int]] = []
        for g in self.groups:
            table = req.tables[g.index]
            gone: List[int] = []
            first = g.first_page_needed(new_len, self.page_size)
            for lp in range(max(table.first_held, g.pinned_pages(self.page_size)), min(first, len(table.pages))):
                page = table.pages[lp]
                if page >= 0:
                    g.pool.give(page)
                    gone.append(page)
                    table.pages[lp] = -1
            table.first_held = max(table.first_held, min(first, len(table.pages)))
            freed.append(gone)
        return freed

    def release(self, rid: Hashable) -> List[List[int]]:
        """The request is finished (or preempted): all pages and the slot go back."""
        req = self._requests.pop(rid)
        freed: List[List[int]] = []
        for g in self.groups:
            gone = req.tables[g.index].held()
            for page in gone:
                g.pool.give(page)
            freed.append(gone)
        self._free_slots.append(req.slot)
        return freed

    def table(self, group: int, rid: Hashable) -> List[int]:
        return self._requests[rid].tables[group].pages

    def table_width(self, rids: Sequence[Hashable]) -> int:
        return max((len(self._requests[r].tables[0].pages) if self.groups else 0) for r in rids) if rids else 0

    def free_pages(self) -> List[int]:
        return [g.pool.free_count for g in self.groups]

    def pages_held(self, rid: Hashable) -> List[int]:
        return [len(self._requests[rid].tables[g.index].held()) for g in self.groups]

    # ---- checks --------------------------------------------------------------- #
    def check(self) -> None:
        """No page lost, held twice or both held and free; no slot shared."""
        for g in self.groups:
            owner: Dict[int, Hashable] = {}
            for req in self._requests.values():
                for page in req.tables[g.index].held():
                    if page in owner:
                        raise PageAccountingError(
                            f"group {g.index}: page {page} is held by {owner[page]!r} and {req.rid!r}"
                        )
                    if g.pool.is_free(page):
                        raise PageAccountingError(f"group {g.index}: page {page} is held and free")
                    owner[page] = req.rid
            if len(owner) + g.pool.free_count != g.pool.num_pages:
                raise PageAccountingError(
                    f"group {g.index}: {len(owner)} held + {g.pool.free_count} free != {g.pool.num_pages} pages"
                )
        slots = [r.slot for r in self._requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise PageAccountingError("a state slot is used twice")
        if len(slots) + len(self._free_slots) != self.max_requests:
            raise PageAccountingError("a state slot is lost")
