"""Builders of replay traces (the JSON steps that `bin/trace_run` reads) in the four
regimes the tests compare, and helpers to run them and to gather logits by request
and position."""

from __future__ import annotations

import random
from typing import Dict, List, Sequence, Tuple

import numpy as np

PORTION_SIZES = [16, 7, 2, 5, 3, 11, 2, 9, 4, 2, 13]


def random_tokens(seed: int, length: int, vocab: int) -> List[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(length)]


def round_up(n: int, m: int = 64) -> int:
    return (n + m - 1) // m * m


def whole(requests: Dict[str, List[int]]) -> List[dict]:
    """Each request alone, its whole sequence in one step."""
    steps = []
    for i, (rid, toks) in enumerate(requests.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def tail_one_by_one(requests: Dict[str, List[int]], tail: int = 32) -> List[dict]:
    """Most of a request in one step, the last `tail` tokens one per step."""
    steps = []
    n = 0
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        n += 1
        for p in range(head, len(toks)):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": [toks[p]], "want": [0]}], "end": [rid] if p == len(toks) - 1 else []})
            n += 1
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests: Dict[str, List[int]], sizes: Sequence[int] = PORTION_SIZES) -> List[dict]:
    """Each request alone, in portions of changing size, down to two tokens."""
    steps = []
    n = 0
    for r, (rid, toks) in enumerate(requests.items()):
        cur = 0
        k = r  # start the size cycle at another place for each request
        while cur < len(toks):
            size = min(sizes[k % len(sizes)], len(toks) - cur)
            k += 1
            last = cur + size == len(toks)
            steps.append(
                {"step": n, "entries": [{"id": rid, "tokens": toks[cur : cur + size], "want": list(range(size))}], "end": [rid] if last else []}
            )
            n += 1
            cur += size
    return steps


def mixed(requests: Dict[str, List[int]], max_live: int = 4, decode_tail: int = 12, sizes: Sequence[int] = PORTION_SIZES) -> List[dict]:
    """Up to `max_live` requests at a time: portions of some beside single decoded
    tokens of others; now and then a request sits a step out; a new request is let
    in only every other step, so that they are at different stages."""
    pending = list(requests.items())
    live: List[Tuple[str, List[int]]] = []
    cursor: Dict[str, int] = {}
    steps = []
    n = 0
    while pending or live:
        if pending and len(live) < max_live and (n % 2 == 0 or not live):
            rid, toks = pending.pop(0)
            live.append((rid, toks))
            cursor[rid] = 0
        entries = []
        ended = []
        for idx, (rid, toks) in enumerate(live):
            cur = cursor[rid]
            remaining = len(toks) - cur
            if len(live) > 1 and (n + 2 * idx) % 5 == 4 and remaining > 1:
                continue  # sits this step out
            if remaining <= decode_tail:
                size = 1
            else:
                size = min(sizes[(n + 3 * idx) % len(sizes)], remaining - decode_tail)
            entries.append({"id": rid, "tokens": toks[cur : cur + size], "want": list(range(size))})
            cursor[rid] = cur + size
            if cursor[rid] == len(toks):
                ended.append(rid)
        if not entries:  # everyone sat out: let the first one run
            rid, toks = live[0]
            cur = cursor[rid]
            entries.append({"id": rid, "tokens": toks[cur : cur + 1], "want": [0]})
            cursor[rid] = cur + 1
            if cursor[rid] == len(toks):
                ended.append(rid)
        steps.append({"step": n, "entries": entries, "end": ended})
        live = [(rid, toks) for rid, toks in live if rid not in ended]
        n += 1
    return steps


def max_live_tokens(steps: List[dict], multiple: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to `multiple`."""
    held: Dict[str, int] = {}
    peak = 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(round_up(v, multiple) for v in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return peak


def gather(steps: List[dict], outputs: Dict[int, np.ndarray], lengths: Dict[str, int], vocab: int) -> Dict[str, np.ndarray]:
    """Logits by request and position from per-step outputs [wanted, vocab]."""
    result = {rid: np.full((n, vocab), np.nan, dtype=np.float32) for rid, n in lengths.items()}
    cursor: Dict[str, int] = {}
    for st in steps:
        out = outputs.get(st["step"])
        row = 0
        for e in st["entries"]:
            base = cursor.get(e["id"], 0)
            for w in e.get("want", []):
                result[e["id"]][base + w] = out[row]
                row += 1
            cursor[e["id"]] = base + len(e["tokens"])
        for rid in st["end"]:
            cursor.pop(rid, None)
        if out is not None:
            assert row == out.shape[0], f"step {st['step']}: {out.shape[0]} rows written, {row} wanted"
    return result


class PageUse:
    """Which (request, logical page) every physical page of every layer group has served, read off the
    manager's block tables.  `note` is called whenever tables may have changed (after pages were taken:
    right after `extend`, or after a step if nothing can both take and give back in between)."""

    def __init__(self, manager) -> None:
        self.manager = manager
        self.served: Dict[int, Dict[int, set]] = {g.index: {} for g in manager.groups}

    def note(self) -> None:
        for g in self.manager.groups:
            for rid in self.manager.live_requests():
                for logical, page in enumerate(self.manager.table(g.index, rid)):
                    if page >= 0:
                        self.served[g.index].setdefault(page, set()).add((rid, logical))

    def pages_used_again(self, group: int) -> int:
        """Physical pages of the group that have held more than one (request, logical page)."""
        return sum(1 for users in self.served[group].values() if len(users) > 1)

    def pages_shared_between_requests(self, group: int) -> int:
        return sum(1 for users in self.served[group].values() if len({rid for rid, _ in users}) > 1)


def run_in_process(replayer, steps: List[dict], page_use: "PageUse | None" = None) -> Dict[int, np.ndarray]:
    outputs = {}
    if page_use is not None:
        # the replayer takes a step's pages before it runs the step and gives pages back after it
        inner = replayer.runner.step

        def step_and_note(portions):
            page_use.note()
            return inner(portions)

        replayer.runner.step = step_and_note
    try:
        for st in steps:
            out = replayer.step(st["entries"], st["end"])
            if out is not None:
                outputs[st["step"]] = out
            replayer.manager.check()
    finally:
        if page_use is not None:
            del replayer.runner.step
    return outputs
