"""The work lists of the matrix-core attention kernel (host arithmetic only): every row tile's keys are
covered once by its items, partial results have places of their own that exactly one merge item reads, and
the lists of a fixed length that a captured step uses hold the same items, filled up with null items."""

import numpy as np
import pytest

from cwm_amd.ops.attention_plan import (
    capacity_until,
    MERGE_MID_MAX, NULL_ROW, ROWS_PER_TILE, WIDE_TILES, PlanCapacity, build_plan, pad_plan,
)


def random_batch(rng, decode_only):
    n = int(rng.integers(1, 9))
    kv, q = [], []
    for _ in range(n):
        new = 1 if decode_only or rng.random() < 0.5 else int(rng.integers(2, 300))
        old = int(rng.integers(0, 20000)) if rng.random() < 0.7 else int(rng.integers(0, 200))
        q.append(new)
        kv.append(old + new)
    return q, kv


def tile_spans(q, kv, group, window):
    """(sequence, first row) -> (first key, end key) that the tile's rows read together."""
    spans = {}
    for b, (n_new, n_kv) in enumerate(zip(q, kv)):
        n_old, rows = n_kv - n_new, n_new * group
        for row0 in range(0, rows, ROWS_PER_TILE):
            first_tok, last_tok = row0 // group, min(row0 + ROWS_PER_TILE - 1, rows - 1) // group
            lo = 0 if window is None else max(0, n_old + first_tok - (window - 1))
            spans[b, row0] = (lo, n_old + last_tok + 1)
    return spans


@pytest.mark.parametrize("seed", range(40))
def test_every_tile_is_covered_once(seed):
    rng = np.random.default_rng(seed)
    q, kv = random_batch(rng, decode_only=seed % 2 == 0)
    group = int(rng.choice([1, 2, 3, 6, 8, 16, 24]))
    window = None if rng.random() < 0.5 else int(rng.choice([1, 8, 100, 8192]))
    plan = build_plan(q, kv, group, window, wide_cut_below=int(rng.choice([0, 64])))
    spans = tile_spans(q, kv, group, window)
    covered = {}
    slots = set()
    for b, row0, first, end, slot, _ in plan.work.tolist():
        assert first < end
        covered.setdefault((b, row0), []).append((first, end, slot))
        if slot >= 0:
            assert slot not in slots
            slots.add(slot)
    wide_rows = set()
    for b, row0, first, end, slot, chunks in plan.work_wide.tolist():
        n_tiles = min(WIDE_TILES, (q[b] * group - row0 + ROWS_PER_TILE - 1) // ROWS_PER_TILE)
        for t in range(n_tiles):
            wide_rows.add((b, row0 + ROWS_PER_TILE * t))
        assert first < end and (slot >= 0) == (chunks > 1)
    for key, (lo, hi) in spans.items():
        if key in wide_rows:
            assert key not in covered
            continue
        items = sorted(covered[key])
        assert items[0][0] == lo and items[-1][1] == hi, (key, items, lo, hi)
        assert all(a[1] == b[0] for a, b in zip(items, items[1:])), (key, items)
        assert all(s >= 0 for _, _, s in items) == (len(items) > 1) and (len(items) > 1 or items[0][2] == -1)
    n_narrow = plan.merge.shape[0] - plan.n_merge_wide
    read = set()
    for i, (b, row0, first, count) in enumerate(plan.merge.tolist()):
        if i < n_narrow:
            items = sorted(covered[b, row0])
            assert [s for _, _, s in items] == list(range(first, first + count))
            assert (count > MERGE_MID_MAX) == (i < n_narrow - plan.n_merge_mid)
        assert not read & set(range(first, first + count))
        read |= set(range(first, first + count))
    assert slots <= read and len(read) == plan.n_partials


@pytest.mark.parametrize("seed", range(30))
def test_lists_of_a_fixed_length(seed):
    rng = np.random.default_rng(100 + seed)
    q, kv = random_batch(rng, decode_only=True)
    group = int(rng.choice([1, 4, 6, 16, 24]))
    window = None if rng.random() < 0.5 else int(rng.choice([8, 100, 8192]))
    max_keys = int(max(kv) * rng.choice([1.0, 1.25, 1.6])) + int(rng.integers(1, 300))
    plan, capacity = capacity_until(q, kv, group, window, 0, max_keys)
    flat = pad_plan(plan, capacity)
    assert flat is not None and flat.dtype == np.int32 and flat.size == capacity.ints
    work = flat[: capacity.work * 6].reshape(-1, 6)
    merge = flat[capacity.work * 6 :].reshape(-1, 4)
    n_work, n_merge = plan.work.shape[0], plan.merge.shape[0]
    n_many = n_merge - plan.n_merge_mid
    assert np.array_equal(work[:n_work], plan.work)
    assert (work[n_work:, 1] == NULL_ROW).all() and (work[n_work:, 2] >= work[n_work:, 3]).all() and (work[n_work:, 4] == -1).all()
    assert np.array_equal(merge[:n_many], plan.merge[:n_many])
    assert (merge[n_many : capacity.merge_many, 1] == NULL_ROW).all()
    mid = merge[capacity.merge_many :]
    assert np.array_equal(mid[: plan.n_merge_mid], plan.merge[n_many:])
    assert (mid[plan.n_merge_mid :, 1] == NULL_ROW).all() and (mid[plan.n_merge_mid :, 3] == 0).all()
    # every later step of the same requests fits until the longest has `max_keys` keys: a token a step, checked at steps
    # spread over the way and around every length at which the rule of the cut changes
    room = max_keys - max(kv)
    steps = set(np.linspace(0, room, 40).astype(int).tolist())
    for n in kv:
        for end in (2048, 8192, 65536):
            steps |= {end - n + d for d in (-1, 0, 1, 2) if 0 <= end - n + d <= room}
    for t in sorted(steps):
        later = build_plan(q, [n + t for n in kv], group, window)
        assert pad_plan(later, capacity) is not None, (t, kv, max_keys, window)
    # much later they do not fit, and that is said
    much_later = build_plan(q, [4 * n + 5000 + max_keys for n in kv], group, window)
    if window is None:
        assert pad_plan(much_later, capacity) is None


def test_a_step_that_cannot_be_cut_has_no_merge_list():
    """Sequences that stay within 2,048 keys while the capture is in use are never cut: the capture holds no
    launch of the merge kernel at all.  One that may cross 2,048 keys has room for its partial results."""
    _, capacity = capacity_until([1] * 5, [900, 1024, 1300, 40, 1700], 6, None, 0, 2040)
    assert capacity.merge == 0 and capacity.work == 5
    # the same in a layer whose window no sequence outgrows meanwhile; a window that one has outgrown moves over the cuts
    _, capacity = capacity_until([1] * 5, [900, 1024, 1300, 40, 1700], 6, 8192, 0, 2040)
    assert capacity.merge == 0 and capacity.work == 5
    _, capacity = capacity_until([1] * 5, [900, 1024, 1300, 40, 1700], 6, 1000, 0, 2040)
    assert capacity.merge_mid == 5 and capacity.work == 10
    _, capacity = capacity_until([1] * 5, [900, 1024, 1300, 40, 1700], 6, None, 0, 2300)
    assert capacity.merge_mid == 5 and capacity.work == 5 * 5  # 2,300 keys are five chunks of 512
    _, capacity = capacity_until([1] * 2, [8000, 100], 6, None, 0, 10000)
    assert capacity.work == 2 * 16  # 8,192 keys in 16 chunks of 512 are more items than 10,000 keys in 10 chunks of 1,024


def test_a_step_with_blocks_of_many_rows_has_no_list_of_a_fixed_length():
    plan = build_plan([400, 1], [400, 900], 6, None)
    assert plan.work_wide.shape[0] > 0
    assert pad_plan(plan, PlanCapacity(work=10000, merge_many=100, merge_mid=100)) is None
