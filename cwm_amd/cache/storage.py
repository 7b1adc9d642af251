"""Device memory of the cache: one paged tensor per cache slot that keeps keys and
values, one slot array per cache slot that keeps fixed-size state.

A paged slot is [num_pages, *spec.page_shape(page_size)]: the cache need of the slot's mixer says how its
page is laid out, and only that mixer's kernels look inside.  The layout of `PagedKVSpec` itself, which the
attention kernels of this package read: [num_pages, 2, n_kv_heads, page_size * head_dim]; plane 0
holds a page's keys as [slot, dim], plane 1 its values in blocks of VB keys as
[slot // VB, dim, slot % VB] with VB = 8 for page sizes that are multiples of 8 and
the whole page otherwise (8 consecutive keys of one dimension are 16 contiguous
bytes: an operand of the matrix-core attention kernel).  The reference keeps keys and values as column halves
of one row-major tensor per layer (cwm/fastgen/utils/cache.py:85-97,131-132).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Sequence

import torch

from ..parts.base import PagedKVSpec, StateSpec
from .manager import CacheManager


@dataclass
class PagedKVView:
    """What an attention mixer gets for one call: its pages and the step's block
    table of its group (int32 [B, W] on the device, -1 where no page is held)."""

    cache: torch.Tensor
    block_table: torch.Tensor
    page_size: int
    window: Optional[int]
    group: int


@dataclass
class StateView:
    """What a mixer with fixed-size state gets: the slot array [max_requests, ...]
    and the slot of each sequence of the step (int32 [B] on the device)."""

    state: torch.Tensor
    slots: torch.Tensor


class CacheStorage:
    def __init__(self, manager: CacheManager, device: torch.device, dtype: torch.dtype) -> None:
        self.manager = manager
        self.device = device
        self.dtype = dtype
        self.paged: Dict[int, torch.Tensor] = {}
        self.state: Dict[int, torch.Tensor] = {}
        for cid, spec in enumerate(manager.specs):
            if isinstance(spec, PagedKVSpec):
                pool = manager.groups[manager.group_of_cache[cid]].pool
                self.paged[cid] = torch.zeros((pool.num_pages, *spec.page_shape(manager.page_size)), dtype=dtype, device=device)
            elif isinstance(spec, StateSpec):
                self.state[cid] = torch.zeros((manager.max_requests, *spec.shape), dtype=spec.dtype, device=device)

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in list(self.paged.values()) + list(self.state.values()))

    def zero_state(self, slot: int) -> None:
        """A request has been admitted to `slot`: its state starts at zero."""
        for t in self.state.values():
            t[slot].zero_()

    def fill_pages(self, group: int, pages: Sequence[int], value: float) -> None:
        """Overwrite given-back pages (tests poison them to show stale reads)."""
        if not pages:
            return
        idx = torch.as_tensor(list(pages), dtype=torch.long, device=self.device)
        for cid in self.manager.groups[group].cache_ids:
            self.paged[cid][idx] = value

    def view(self, cache_id: int, batch) -> object:
        spec = self.manager.specs[cache_id]
        if isinstance(spec, PagedKVSpec):
            g = self.manager.group_of_cache[cache_id]
            return PagedKVView(
                cache=self.paged[cache_id],
                block_table=batch.block_tables[g],
                page_size=self.manager.page_size,
                window=spec.window,
                group=g,
            )
        if isinstance(spec, StateSpec):
            return StateView(state=self.state[cache_id], slots=batch.state_slots)
        return None
