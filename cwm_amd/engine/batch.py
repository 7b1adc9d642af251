"""The descriptor of one step's batch: which tokens run, where they sit in their
sequences, where their keys and values go, and which rows' logits are wanted.

The reference's prefill call takes per sequence (tokens already cached, new tokens)
and derives the same vectors on the host (cwm/fastgen/forward.py:504-519,875-894);
a decoded token is the case of one new token.  Here one descriptor serves portions
of prompts and decoded tokens alike, and it goes to the device in a single copy.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..cache.pages import pages_for


@dataclass
class Portion:
    """The next tokens of one request in this step, and the places among them
    (indices into `tokens`) whose logits are wanted."""

    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class StepBatch:
    n_tokens: int
    n_seqs: int
    n_logit_rows: int
    tokens: torch.Tensor  # int32 [T]
    positions: torch.Tensor  # int32 [T] absolute position of each token in its sequence
    seq_of_token: torch.Tensor  # int32 [T] index of the token's sequence in this batch
    cu_q: torch.Tensor  # int32 [B + 1] first token of each sequence in the batch
    kv_len: torch.Tensor  # int32 [B] tokens of each sequence after this step
    state_slots: torch.Tensor  # int32 [B] state slot of each sequence
    logit_rows: torch.Tensor  # int32 [R] tokens whose logits are wanted
    block_tables: List[torch.Tensor]  # per layer group int32 [B, W]
    # host copies
    q_lens: List[int] = field(default_factory=list)
    kv_lens: List[int] = field(default_factory=list)
    rids: List[Hashable] = field(default_factory=list)
    page_size: int = 0
    scratch: Dict[Any, Any] = field(default_factory=dict)  # per-step plans that kernels' wrappers keep
    static: Any = None  # for a step that is captured and replayed: the fixed homes of such plans (`ops.StaticPlans`)

    @property
    def max_kv_len(self) -> int:
        return max(self.kv_lens) if self.kv_lens else 0


class BatchError(ValueError):
    pass


def build_batch(
    portions: Sequence[Portion],
    manager: CacheManager,
    device: torch.device,
    vocab_size: int,
    tokens_device: Optional[torch.Tensor] = None,
    table_width: Optional[int] = None,
    into: Optional[torch.Tensor] = None,
) -> StepBatch:
    """Descriptor for `portions`; the pages of their tokens must already be held
    (`CacheManager.extend`).  `tokens_device` (int32 [T] on the device) takes the place of the
    portions' token ids, which then only count: a decode step whose tokens the step before has
    sampled and which have not been to the host.  `table_width`: columns of the block tables (at
    least what the longest sequence needs; the rest holds -1).  `into`: an int32 vector on the
    device that receives the descriptor instead of a new one, so that steps of one shape (the same
    numbers of tokens, sequences, wanted rows and table columns) have their vectors at the same
    addresses."""
    if not portions:
        raise BatchError("a step needs at least one portion")
    n_seqs = len(portions)
    rids: List[Hashable] = [portion.rid for portion in portions]
    if len(set(rids)) != n_seqs:
        twice = next(r for r in rids if rids.count(r) > 1)
        raise BatchError(f"request {twice!r} appears twice in one step")
    for rid in rids:
        if rid not in manager:
            raise BatchError(f"request {rid!r} has not been admitted")
    q_lens = [len(portion.tokens) for portion in portions]
    for rid, n_new in zip(rids, q_lens):
        if n_new == 0:
            raise BatchError(f"request {rid!r} brings no token to this step")
    old_lens = [manager.length(rid) for rid in rids]
    for rid, n_new in zip(rids, q_lens):
        if any(m > 0 for m in manager.pages_missing(rid, n_new)):
            raise BatchError(f"request {rid!r}: pages for {n_new} more tokens have not been reserved")
    kv_lens = [o + n for o, n in zip(old_lens, q_lens)]
    slots = [manager.slot(rid) for rid in rids]
    n_tokens = sum(q_lens)
    # all vectors at once: a decode step of many requests is many portions of one token
    q_arr = np.asarray(q_lens, dtype=np.int64)
    cu = np.zeros(n_seqs + 1, dtype=np.int64)
    np.cumsum(q_arr, out=cu[1:])
    tokens = np.fromiter((t for portion in portions for t in portion.tokens), dtype=np.int64, count=n_tokens)
    bad = (tokens < 0) | (tokens >= vocab_size)
    if bad.any():
        where = int(np.argmax(bad))
        b = int(np.searchsorted(cu, where, side="right")) - 1
        raise BatchError(f"request {rids[b]!r}: token id {int(tokens[where])} is outside the vocabulary of {vocab_size}")
    seq_of_token = np.repeat(np.arange(n_seqs, dtype=np.int32), q_arr)
    # position of a token: its place in the portion plus what the sequence held before
    positions = (np.arange(n_tokens, dtype=np.int64) - np.repeat(cu[:-1] - np.asarray(old_lens, dtype=np.int64), q_arr)).astype(np.int32)
    tokens = tokens.astype(np.int32)
    rows: List[int] = []
    for b, portion in enumerate(portions):
        base = int(cu[b])
        for w in portion.want:
            if not 0 <= int(w) < q_lens[b]:
                raise BatchError(f"request {portion.rid!r}: wanted place {w} is outside its {q_lens[b]} tokens")
            rows.append(base + int(w))
    cu_q = cu

    page_size = manager.page_size
    width = max(1, max((kv + page_size - 1) // page_size for kv in kv_lens))
    if table_width is not None:
        if table_width < width:
            raise BatchError(f"block tables of {table_width} columns do not hold the {width} pages of the longest sequence")
        width = table_width
    tables = []
    columns = np.arange(width, dtype=np.int64)[None, :]
    last_page = np.asarray([pages_for(kv, page_size) for kv in kv_lens], dtype=np.int64)[:, None]
    for g in manager.groups:
        tbl = np.full((n_seqs, width), -1, dtype=np.int32)
        for b, rid in enumerate(rids):
            pages = manager.table(g.index, rid)
            n = min(len(pages), width)
            tbl[b, :n] = pages[:n]
        # every page that this step's queries can read, or that its tokens are written to, is held
        first_page = np.asarray(
            [g.first_page_needed(kv - q, page_size) for kv, q in zip(kv_lens, q_lens)], dtype=np.int64
        )[:, None]
        needed = ((columns >= first_page) | (columns < g.pinned_pages(page_size))) & (columns < last_page)
        bad = needed & ((tbl < 0) | (tbl >= g.pool.num_pages))
        if bad.any():
            b = int(np.argmax(bad.any(axis=1)))
            first, last = int(first_page[b, 0]), int(last_page[b, 0])
            raise BatchError(
                f"request {rids[b]!r}: group {g.index} holds no page for some of the logical pages {first}..{last - 1} "
                f"that this step reads or writes (table {tbl[b, first:last].tolist()}, pool of {g.pool.num_pages})"
            )
        tables.append(tbl)

    # one buffer, one copy
    segments = [
        tokens,
        positions,
        seq_of_token,
        np.asarray(cu_q, dtype=np.int32),
        np.asarray(kv_lens, dtype=np.int32),
        np.asarray(slots, dtype=np.int32),
        np.asarray(rows, dtype=np.int32),
    ] + [t.reshape(-1) for t in tables]
    offsets = []
    total = 0
    for seg in segments:
        offsets.append(total)
        total += (seg.size + 3) // 4 * 4  # keep every segment 16-byte aligned
    use_pinned = device.type == "cuda"
    host = torch.empty(max(total, 4), dtype=torch.int32, pin_memory=use_pinned)
    host_np = host.numpy()
    for off, seg in zip(offsets, segments):
        host_np[off : off + seg.size] = seg
    if into is None:
        dev = host.to(device, non_blocking=use_pinned)
    else:
        if into.dtype != torch.int32 or into.dim() != 1 or into.numel() < host.numel() or into.device.type != device.type:
            raise BatchError(f"the descriptor's {host.numel()} numbers do not fit the vector given for them")
        dev = into
        dev[: host.numel()].copy_(host, non_blocking=use_pinned)

    def seg(i: int) -> torch.Tensor:
        return dev[offsets[i] : offsets[i] + segments[i].size]

    if tokens_device is not None:
        if tokens_device.dtype != torch.int32 or tokens_device.numel() != tokens.size or not tokens_device.is_contiguous():
            raise BatchError(f"tokens on the device must be a contiguous int32 [{tokens.size}] tensor")
    return StepBatch(
        n_tokens=int(tokens.size),
        n_seqs=n_seqs,
        n_logit_rows=len(rows),
        tokens=seg(0) if tokens_device is None else tokens_device.reshape(-1),
        positions=seg(1),
        seq_of_token=seg(2),
        cu_q=seg(3),
        kv_len=seg(4),
        state_slots=seg(5),
        logit_rows=seg(6),
        block_tables=[seg(7 + i).view(n_seqs, width) for i in range(len(tables))],
        q_lens=q_lens,
        kv_lens=kv_lens,
        rids=rids,
        page_size=page_size,
    )
