"""Work lists of the matrix-core attention kernel, built on the host per step.

For every sequence and 16-row tile (rows are (token, head of the group) pairs) the
list names the keys the tile reads.  A sequence that brings few rows (a decoded
token, a short portion) has a long key range cut into chunks at fixed absolute
positions so that many blocks share the reading; the chunks' partial results
are merged by a second kernel.  Whether and where a sequence is cut depends on its
own lengths only.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np

ROWS_PER_TILE = 16
SPLIT_MAX_TILES = 8  # sequences with more row tiles than this are not split
WIDE_TILES = 8  # row tiles (128 rows) of one block of the kernel that shares keys and values through LDS
WIDE_CHUNK = 8192  # keys after which such a block's range is cut (at fixed absolute positions, like the others)
WIDE_CHUNK_FINE = 2048  # the same for a sequence with very few such blocks


def chunk_keys(n_keys):
    """Keys per chunk (a multiple of 128: four wavefronts take a chunk's tiles of 32 keys in turn) for a row tile
    that reads `n_keys` keys (a number or an array of them).  Up to 2,048 keys are not cut: a block of four
    wavefronts reads them and leaves no partial result (64 sequences of 1,024 keys: 45 us a layer of the 32B
    shape against 59 us in two chunks with their merge; a lone sequence of 1,024 keys pays 15 us against 10 us
    in chunks of 256).  Longer ranges are cut so that a few sequences still spread over the chip: 512 keys up
    to 8,192 (eight sequences in a window of 8,192 keys: 54 us against 58 us in chunks of 1,024), 1,024 up to
    65,536, then 2,048 (eight sequences of 131,072 keys: 647 us against 665 us in chunks of 4,096)."""
    n = np.asarray(n_keys)
    return np.where(n <= 2048, 2048, np.where(n <= 8192, 512, np.where(n <= 65536, 1024, 2048)))


MERGE_MID_MAX = 32  # partials up to which an item is merged by 4 wavefronts instead of 16
WORK_INTS = 6
PARTIAL_PAD = 4


@dataclass
class AttentionPlan:
    work: np.ndarray  # int32 [n_work, 6]: sequence, first row, first key, end key, partial slot or -1, 0
    work_wide: np.ndarray  # the same for items of WIDE_TILES row tiles; last int: the number of chunks of the item
    merge: np.ndarray  # int32 [n_merge, 4]: sequence, first row, first partial slot, number of partials
    n_partials: int
    n_merge_wide: int = 0  # how many of the last merge items belong to cut wide items (few partials each)
    n_merge_mid: int = 0  # how many before those have at most MERGE_MID_MAX partials; the items before them have more


def build_plan(
    q_lens: Sequence[int], kv_lens: Sequence[int], group: int, window: Optional[int], wide_cut_below: int = 0
) -> AttentionPlan:
    """`wide_cut_below`: a sequence with fewer wide items than this has their keys cut at multiples of
    WIDE_CHUNK (its blocks alone would leave compute units idle), with fewer than an eighth of it at
    multiples of WIDE_CHUNK_FINE; the caller derives the number from the model's heads and the chip,
    so that it is the same whatever else the batch holds."""
    q = np.asarray(q_lens, dtype=np.int64)
    kv = np.asarray(kv_lens, dtype=np.int64)
    n_rows = q * group
    n_tiles = (n_rows + ROWS_PER_TILE - 1) // ROWS_PER_TILE
    is_wide = n_tiles > SPLIT_MAX_TILES

    # ---- sequences with many rows: WIDE_TILES tiles form a block that shares keys and values in LDS
    wide_seq, wide_row0, wide_lo, wide_hi, wide_n_tiles, wide_cut = [], [], [], [], [], []
    for b in np.nonzero(is_wide)[0]:
        lo, hi, row0 = _tile_ranges(int(q[b]), int(kv[b]), int(n_tiles[b]), group, window)
        n_wide = (int(n_tiles[b]) + WIDE_TILES - 1) // WIDE_TILES
        first = np.arange(n_wide) * WIDE_TILES
        last = np.minimum(first + WIDE_TILES - 1, int(n_tiles[b]) - 1)
        wide_seq.append(np.full(n_wide, b, dtype=np.int64))
        wide_row0.append(row0[first])
        wide_lo.append(lo[first])
        wide_hi.append(hi[last])
        wide_n_tiles.append(last - first + 1)
        wide_cut.append(np.full(n_wide, 0 if n_wide >= wide_cut_below else (WIDE_CHUNK if 8 * n_wide >= wide_cut_below else WIDE_CHUNK_FINE)))

    # ---- all tiles of the other sequences at once, in the order (sequence, tile, chunk)
    small = np.nonzero(~is_wide)[0]
    tiles_of = n_tiles[small]
    seq = np.repeat(small, tiles_of)  # sequence of each tile
    first = np.cumsum(tiles_of) - tiles_of
    tile = np.arange(int(tiles_of.sum()), dtype=np.int64) - np.repeat(first, tiles_of)  # tile index within its sequence
    row0 = tile * ROWS_PER_TILE
    n_old = (kv - q)[seq]
    first_tok = row0 // group
    last_tok = np.minimum(row0 + ROWS_PER_TILE - 1, n_rows[seq] - 1) // group
    hi = n_old + last_tok + 1  # exclusive
    lo = np.zeros_like(hi) if window is None else np.maximum(0, n_old + first_tok - (window - 1))
    chunk = chunk_keys(hi - lo)
    c0 = lo // chunk
    n_chunks = (hi - 1) // chunk - c0 + 1
    split = n_chunks > 1
    slot0 = np.cumsum(np.where(split, n_chunks, 0)) - np.where(split, n_chunks, 0)  # first partial slot of a split tile
    item_tile = np.repeat(np.arange(tile.size), n_chunks)
    item_first = np.cumsum(n_chunks) - n_chunks
    c = np.arange(int(n_chunks.sum()), dtype=np.int64) - item_first[item_tile]  # chunk index within its tile
    ck = chunk[item_tile]
    work = np.zeros((c.size, WORK_INTS), dtype=np.int32)
    work[:, 0] = seq[item_tile]
    work[:, 1] = row0[item_tile]
    work[:, 2] = np.maximum(lo[item_tile], (c0[item_tile] + c) * ck)
    work[:, 3] = np.minimum(hi[item_tile], (c0[item_tile] + c + 1) * ck)
    work[:, 4] = np.where(split[item_tile], slot0[item_tile] + c, -1)
    merge = np.zeros((int(split.sum()), 4), dtype=np.int32)
    merge[:, 0] = seq[split]
    merge[:, 1] = row0[split]
    merge[:, 2] = slot0[split]
    merge[:, 3] = n_chunks[split]
    # items with many partials first: they are merged by more wavefronts than the others
    many = merge[:, 3] > MERGE_MID_MAX
    merge = np.concatenate([merge[many], merge[~many]], axis=0)
    n_merge_mid = int((~many).sum())
    n_partials = int(n_chunks[split].sum())

    # ---- wide items whose keys cross multiples of their chunk length are cut there into blocks of their own; a
    # block then leaves a partial result for each of its row tiles (tile t of an item with n chunks has
    # the slots first + t * n .. first + t * n + n - 1), which the merge kernel adds like the others
    wide_arr = np.zeros((0, WORK_INTS), dtype=np.int32)
    n_merge_wide = 0
    if wide_seq:
        w_seq, w_row0 = np.concatenate(wide_seq), np.concatenate(wide_row0)
        w_lo, w_hi, w_tiles = np.concatenate(wide_lo), np.concatenate(wide_hi), np.concatenate(wide_n_tiles)
        w_chunk = np.concatenate(wide_cut)  # 0: not cut
        w_size = np.maximum(w_chunk, 1)
        w_c0 = w_lo // w_size
        w_nc = np.where(w_chunk > 0, (w_hi - 1) // w_size - w_c0 + 1, 1)
        w_split = w_nc > 1
        w_slots = np.where(w_split, w_nc * w_tiles, 0)
        w_first = n_partials + np.cumsum(w_slots) - w_slots  # first slot of a split item
        n_partials += int(w_slots.sum())
        of = np.repeat(np.arange(w_seq.size), w_nc)  # the item of each block
        c = np.arange(int(w_nc.sum()), dtype=np.int64) - (np.cumsum(w_nc) - w_nc)[of]
        wide_arr = np.zeros((of.size, WORK_INTS), dtype=np.int32)
        wide_arr[:, 0] = w_seq[of]
        wide_arr[:, 1] = w_row0[of]
        wide_arr[:, 2] = np.where(w_split[of], np.maximum(w_lo[of], (w_c0[of] + c) * w_size[of]), w_lo[of])
        wide_arr[:, 3] = np.where(w_split[of], np.minimum(w_hi[of], (w_c0[of] + c + 1) * w_size[of]), w_hi[of])
        wide_arr[:, 4] = np.where(w_split[of], w_first[of] + c, -1)
        wide_arr[:, 5] = w_nc[of]
        if wide_arr.shape[0] > 1:
            # longest first: blocks start in list order, and the last ones to start should be short
            wide_arr = wide_arr[np.argsort(wide_arr[:, 2] - wide_arr[:, 3], kind="stable")]
        if w_split.any():
            items = np.nonzero(w_split)[0]
            of_t = np.repeat(items, w_tiles[items])  # the item of each row tile of a split item
            t = np.arange(of_t.size, dtype=np.int64) - (np.cumsum(w_tiles[items]) - w_tiles[items])[np.repeat(np.arange(items.size), w_tiles[items])]
            wide_merge = np.zeros((of_t.size, 4), dtype=np.int32)
            wide_merge[:, 0] = w_seq[of_t]
            wide_merge[:, 1] = w_row0[of_t] + ROWS_PER_TILE * t
            wide_merge[:, 2] = w_first[of_t] + t * w_nc[of_t]
            wide_merge[:, 3] = w_nc[of_t]
            merge = np.concatenate([merge, wide_merge], axis=0)
            n_merge_wide = wide_merge.shape[0]
    return AttentionPlan(
        work=np.ascontiguousarray(work),
        work_wide=np.ascontiguousarray(wide_arr),
        merge=np.ascontiguousarray(merge),
        n_partials=n_partials,
        n_merge_wide=n_merge_wide,
        n_merge_mid=n_merge_mid,
    )


def _tile_ranges(n_new: int, kv: int, n_tiles: int, group: int, window: Optional[int]):
    """First and end key and first row of each 16-row tile of one sequence."""
    n_old = kv - n_new
    n_rows = n_new * group
    row0 = np.arange(n_tiles, dtype=np.int64) * ROWS_PER_TILE
    first_tok = row0 // group
    last_tok = np.minimum(row0 + ROWS_PER_TILE - 1, n_rows - 1) // group
    key_hi = n_old + last_tok + 1  # exclusive
    key_lo = np.zeros_like(row0) if window is None else np.maximum(0, n_old + first_tok - (window - 1))
    return key_lo, key_hi, row0


# an item that no kernel acts on: its first row lies beyond every sequence's rows and it names no key
NULL_ROW = 1 << 24
NULL_WORK = (0, NULL_ROW, 0, 0, -1, 0)
NULL_MERGE = (0, NULL_ROW, 0, 0)


@dataclass(frozen=True)
class PlanCapacity:
    """Sizes of a plan's lists that do not change from step to step: a captured step launches these many
    items whatever the step holds, and the unused ones are null items."""

    work: int
    merge_many: int
    merge_mid: int

    @property
    def merge(self) -> int:
        return self.merge_many + self.merge_mid

    @property
    def ints(self) -> int:
        return self.work * WORK_INTS + self.merge * 4

    @staticmethod
    def covering(plans: Sequence[AttentionPlan]) -> "PlanCapacity":
        """Room for the largest of `plans` in every list: the caller hands in the step's plan and the plans of the
        same step with its sequences grown as far as the capture allows (and grown just to every length at which
        the rule of `chunk_keys` changes, since a longer range may be cut into fewer chunks than a shorter one).  A
        list that stays empty in all of them gets no launch at all."""
        work = merge_many = merge_mid = 0
        for plan in plans:
            n_many = plan.merge.shape[0] - plan.n_merge_mid - plan.n_merge_wide
            work = max(work, plan.work.shape[0])
            merge_many = max(merge_many, n_many)
            merge_mid = max(merge_mid, plan.n_merge_mid)
        return PlanCapacity(work=work, merge_many=merge_many, merge_mid=merge_mid)


# lengths of a key range at which `chunk_keys` changes (the last length of each rule)
CHUNK_RULE_ENDS = (2048, 8192, 65536)


def capacity_until(
    q_lens: Sequence[int], kv_lens: Sequence[int], group: int, window: Optional[int], wide_cut_below: int, max_keys: int
) -> "tuple[AttentionPlan, PlanCapacity]":
    """The step's plan, and the sizes of its lists for as long as no sequence holds more than `max_keys` keys
    (every sequence growing by a token a step): the sequences as they are, all of them grown to `max_keys`, and
    grown to each length in between at which the rule for cutting the keys changes."""
    plan = build_plan(q_lens, kv_lens, group, window, wide_cut_below)
    plans = [plan]
    for length in sorted({max_keys, *(n + d for n in CHUNK_RULE_ENDS for d in (0, 1) if n + d < max_keys)}):
        grown = [min(max(kv, length), max(kv, max_keys)) for kv in kv_lens]
        if grown != list(kv_lens):
            plans.append(build_plan(q_lens, grown, group, window, wide_cut_below))
    capacity = PlanCapacity.covering(plans)
    if window is not None and max(max(kv_lens), max_keys) > window:
        # a window's range moves over the fixed positions of the cuts: at some steps it straddles one cut more than at
        # others, whatever its length (a window shorter than a chunk is cut in two now and then).  While no sequence
        # is longer than the window every range starts at key 0, as without a window.
        tiles = int((plan.work[:, 4] < 0).sum()) + plan.merge.shape[0]
        capacity = PlanCapacity(work=capacity.work + tiles, merge_many=capacity.merge_many, merge_mid=max(capacity.merge_mid, tiles))
    return plan, capacity


def pad_plan(plan: AttentionPlan, capacity: PlanCapacity) -> Optional[np.ndarray]:
    """`plan` as one int32 vector of `capacity.ints` numbers: the work items, then the merge items of many
    partials, then those of few, each list filled up with null items.  None if the plan does not fit, or has
    items that a captured step does not take (blocks of many rows)."""
    n_merge = plan.merge.shape[0]
    n_many = n_merge - plan.n_merge_mid - plan.n_merge_wide
    if plan.work_wide.shape[0] or plan.n_merge_wide:
        return None
    if plan.work.shape[0] > capacity.work or n_many > capacity.merge_many or plan.n_merge_mid > capacity.merge_mid:
        return None
    work = np.tile(np.asarray(NULL_WORK, dtype=np.int32), (capacity.work, 1))
    work[: plan.work.shape[0]] = plan.work
    merge = np.tile(np.asarray(NULL_MERGE, dtype=np.int32), (capacity.merge, 1))
    merge[:n_many] = plan.merge[:n_many]
    merge[capacity.merge_many : capacity.merge_many + plan.n_merge_mid] = plan.merge[n_many:]
    return np.concatenate([work.reshape(-1), merge.reshape(-1)])
