"""Trace replay: feeds given token ids through a model step by step and writes the
logits at the wanted places.  Nothing is sampled.  It drives the same model, step
function, cache manager and kernels that generation uses.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input holds one JSON object per line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

`entries` gives for each request its next tokens and the places among them whose
logits are wanted; all entries of a step run as one batch.  `end` names requests
that are finished after the step; their pages go back.  For a step in which
something is wanted, `<out>/<step>.f32` receives the logits [wanted, vocab] as
little-endian float32 in the order of the entries and of `want`.  After every step
`done <step>` is printed and flushed.  `--max-tokens` is the most tokens that live
requests hold at any time, each request's count rounded up to a multiple of 64;
every layer group's pool is made for that many, so pages are used again.

Further options: `--page-size P` (tokens in a page, default 16; pools of pages that do
not divide 64 get one more page per live request, since a request's last page may be
partly filled beyond its multiple of 64); `--pages all=N,8192=M` sets the pools' sizes in
pages outright, by the group's window (`all`: the group that keeps every key);
`--random-config FILE --seed S [--std X]` runs the configuration in FILE with random
weights instead of a model folder; `--page-log FILE` writes, per step, the pages every
request took and the pages that went back to each group's pool, as JSON lines;
`--graphs N` runs steps of single tokens whose logits are all wanted as generation does by
default: captured as HIP graphs, one per number of requests and at most N of them, and
replayed (default 0: every step is launched kernel by kernel).

The reference has no such tool; its nearest hooks are prompt log-probabilities
(cwm/fastgen/forward.py:908-924) and the eager decode path
(cwm/fastgen/generate.py:313-315).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict, List, Optional

import numpy as np
import torch

REPLAY_PAGE_SIZE = 16  # divides 64, so a pool of max_tokens / 16 pages always suffices
REPLAY_MAX_REQUESTS = 16


REPLAY_MAX_LIVE = 4  # requests live at a time in a trace


class Replayer:
    """Model + cache + step function driven by explicit steps."""

    def __init__(
        self,
        model_dir: Optional[str],
        dtype: str,
        max_tokens: int,
        device: str = "cuda:0",
        page_size: int = REPLAY_PAGE_SIZE,
        max_requests: int = REPLAY_MAX_REQUESTS,
        poison_freed_pages: bool = False,
        pages: Optional[Dict[Optional[int], int]] = None,
        random_config: Optional[dict] = None,
        seed: int = 0,
        std: float = 0.02,
        page_log: Optional[str] = None,
        num_graphs: int = 0,
    ) -> None:
        from .cache import CacheManager, CacheStorage
        from .engine import ModelRunner, load_model, random_model
        from .engine.runner import weak_callback
        from .parts.base import PagedKVSpec

        if max_tokens <= 0:
            raise ValueError("--max-tokens must be positive")
        if page_size <= 0:
            raise ValueError("--page-size must be positive")
        self.device = torch.device(device)
        if (model_dir is None) == (random_config is None):
            raise ValueError("give a model folder or a configuration for random weights, not both")
        if random_config is not None:
            self.model, self.config = random_model(random_config, seed, dtype, self.device, std=std)
        else:
            self.model, self.config = load_model(model_dir, dtype, self.device)
        num_pages = max(1, (max_tokens + page_size - 1) // page_size)
        if 64 % page_size != 0:
            num_pages += REPLAY_MAX_LIVE
        sizes: object = num_pages
        if pages is not None:
            sizes = {}
            for spec in self.model.cache_specs:
                if isinstance(spec, PagedKVSpec):  # pools are keyed by what the cache need keeps (its window; None: all)
                    sizes[spec.retention()] = pages.get(spec.retention(), num_pages)
            unknown = set(pages) - set(sizes)
            if unknown:
                raise ValueError(f"--pages names groups that the model does not have: {sorted(map(str, unknown))}; its groups: {sorted(map(str, sizes))}")
        self.manager = CacheManager(self.model.cache_specs, page_size, sizes, max_requests)
        self.storage = CacheStorage(self.manager, self.device, self.model.runtime.act_dtype)
        self.runner = ModelRunner(self.model, self.manager, self.storage, num_graphs=num_graphs)
        self.poison_freed_pages = poison_freed_pages
        self._given: Dict[int, List[int]] = {}
        self._log = open(page_log, "w", encoding="utf-8") if page_log else None
        self._steps = 0
        self.runner.on_pages_freed = weak_callback(self._pages_freed)

    def _pages_freed(self, group: int, pages: List[int]) -> None:
        self._given.setdefault(group, []).extend(pages)
        if self.poison_freed_pages:
            self.storage.fill_pages(group, pages, float("nan"))

    def close(self) -> None:
        if self._log is not None:
            self._log.close()
            self._log = None

    def step(self, entries: List[dict], end: List[object]) -> Optional[np.ndarray]:
        """One step; returns logits [wanted, vocab] or None."""
        from .engine import Portion

        portions = []
        taken: Dict[str, Dict[int, List[int]]] = {}
        self._given = {}
        for entry in entries:
            rid = entry["id"]
            tokens = [int(t) for t in entry["tokens"]]
            want = [int(w) for w in entry.get("want", [])]
            if not tokens:
                if want:
                    raise ValueError(f"request {rid!r}: logits are wanted at places {want} of no tokens")
                continue  # an entry that brings nothing this step
            if rid not in self.manager:
                self.runner.admit(rid)
            before = [len(self.manager.table(g.index, rid)) for g in self.manager.groups]
            if not self.manager.extend(rid, len(tokens)):
                raise RuntimeError(
                    f"request {rid!r}: no pages left for {len(tokens)} more tokens "
                    f"(free pages per group: {self.manager.free_pages()}); --max-tokens is too small for this trace"
                )
            if self._log is not None:
                new = {g.index: self.manager.table(g.index, rid)[before[g.index] :] for g in self.manager.groups}
                taken[str(rid)] = {g: p for g, p in new.items() if p}
            portions.append(Portion(rid=rid, tokens=tokens, want=want))
        logits = self.runner.step(portions) if portions else None
        for rid in end:
            if rid in self.manager:
                self.runner.release(rid)
        if self._log is not None:
            record = {"step": self._steps, "take": {r: t for r, t in taken.items() if t}, "give": self._given,
                      "free": self.manager.free_pages()}
            self._log.write(json.dumps(record) + "\n")
            self._log.flush()
        self._steps += 1
        if logits is None:
            return None
        return logits.detach().to("cpu", torch.float32).numpy()


def main(argv: Optional[List[str]] = None) -> int:
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--model", help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    parser.add_argument("--out", required=True, help="folder that receives <step>.f32")
    parser.add_argument("--max-tokens", type=int, required=True)
    parser.add_argument("--device", default="cuda:0")
    parser.add_argument("--page-size", type=int, default=REPLAY_PAGE_SIZE, help="tokens in a page")
    parser.add_argument("--pages", default="", help="pool sizes in pages by group, e.g. all=40,8192=12 (default: from --max-tokens)")
    parser.add_argument("--random-config", help="a config.json to run with random weights instead of --model")
    parser.add_argument("--seed", type=int, default=0, help="seed of those random weights")
    parser.add_argument("--std", type=float, default=0.02, help="standard deviation of those random weights")
    parser.add_argument("--page-log", help="file that receives the pages taken and given back, one JSON line a step")
    parser.add_argument("--graphs", type=int, default=0, help="decode steps kept as HIP graphs (0: none)")
    args = parser.parse_args(argv)
    if (args.model is None) == (args.random_config is None):
        parser.error("give exactly one of --model and --random-config")
    pages = None
    if args.pages:
        pages = {}
        for item in args.pages.split(","):
            key, _, value = item.partition("=")
            pages[None if key.strip() == "all" else int(key)] = int(value)
    random_config = None
    if args.random_config:
        with open(args.random_config, "r", encoding="utf-8") as fh:
            random_config = json.load(fh)

    os.makedirs(args.out, exist_ok=True)
    replayer = Replayer(
        args.model, args.dtype, args.max_tokens, device=args.device, page_size=args.page_size, pages=pages,
        random_config=random_config, seed=args.seed, std=args.std, page_log=args.page_log, num_graphs=args.graphs,
    )
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        logits = replayer.step(record.get("entries", []), record.get("end", []))
        if logits is not None and logits.shape[0] > 0:
            logits.astype("<f4").tofile(os.path.join(args.out, f"{step}.f32"))
        print(f"done {step}", flush=True)
    replayer.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
