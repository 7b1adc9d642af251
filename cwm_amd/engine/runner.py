"""The step function: one batch of (request, its next tokens) through the model.

It runs only the tokens it is given, as one batch, reading earlier tokens from the
cache, and returns float32 logits at the wanted places.  Portions of prompts and
single decoded tokens may share a step and a portion may be cut anywhere.  The
reference has two entry points for this, `prefill` for ragged new tokens and
`decode` for one token per lane (cwm/fastgen/forward.py:824-961), and never mixes
them in one call (cwm/fastgen/generate.py:480-498).
"""

from __future__ import annotations

import gc
import sys
import threading
import weakref
from collections import OrderedDict
from dataclasses import dataclass
from typing import Any, Callable, Hashable, List, Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..cache.pages import pages_for
from ..cache.storage import CacheStorage
from ..models.model import Model
from .batch import Portion, StepBatch, build_batch


@dataclass
class CapturedStep:
    """A decode step of `n_seqs` requests as a HIP graph, with what it reads and writes at fixed addresses
    (the reference's DecodeGraph, cwm/fastgen/generate.py:71-75,339-373)."""

    graph: Any  # torch.cuda.CUDAGraph
    descriptor: torch.Tensor  # the step's descriptor (int32), filled anew before every replay
    table_width: int  # columns of its block tables: the sequences may grow to that many pages
    plans: Any  # ops.StaticPlans: the kernels' work lists, likewise
    tokens: torch.Tensor  # the descriptor's token ids
    logits: torch.Tensor  # where a replay leaves its logits


# HIP refuses the destruction of a graph while any stream of the process captures, and torch ends the process when
# that happens in a destructor.  Every capture and every drop of a captured step in this module holds this lock, so
# that runners on several threads do not destroy one runner's graphs during another's capture.
_GRAPH_LOCK = threading.RLock()


def weak_callback(method: Callable) -> Callable:
    """`method` (bound) as a callback that does not keep its object alive: an engine that registers its own
    method with a part of itself would otherwise sit in a cycle of references, and its cache and graphs would
    stay on the device until the collector finds it."""
    ref = weakref.WeakMethod(method)

    def call(*args: Any) -> Any:
        target = ref()
        return target(*args) if target is not None else None

    return call


class ModelRunner:
    # a step is worth a capture when the host took at least this share of the step's time to launch it
    HOST_BOUND_SHARE = 0.85

    def __init__(
        self, model: Model, manager: CacheManager, storage: CacheStorage, num_graphs: int = 0, graphs_where_host_bound: bool = False
    ) -> None:
        """`num_graphs`: decode steps (one token of every request, the logits of all wanted) are captured as
        HIP graphs, one per number of requests, and replayed, which spares the host the launch of every
        kernel; at most so many are kept, the least recently used goes.  0, a model some part of which is
        not `replayable`, or a device that is no GPU: every step is launched kernel by kernel.
        `graphs_where_host_bound`: a number of requests gets its capture only if launching its step keeps
        the host busy for most of the step's time (measured on its second and third step; where the GPU's
        time is the longer one a replay gains nothing, and its lists of a fixed length cost a little)."""
        if model.runtime is None:
            raise RuntimeError("the model has no weights yet (Model.bind)")
        self.model = model
        self.manager = manager
        self.storage = storage
        self.device = model.runtime.device
        # called as on_pages_freed(group, pages) whenever pages go back to a pool
        self.on_pages_freed: Optional[Callable[[int, List[int]], None]] = None
        self.num_graphs = num_graphs if self.device.type == "cuda" and model.replayable else 0
        self.graphs_where_host_bound = graphs_where_host_bound
        self._host_share: dict = {}  # number of requests -> shares of the step's time that the host spent launching it
        self._captured: "OrderedDict[int, CapturedStep]" = OrderedDict()
        self._graph_pool: Any = None
        self.n_captures = 0
        self.n_replays = 0

    def __del__(self) -> None:
        # the captured steps' graphs go here, under the lock, not whenever the last reference happens to fall
        captured = getattr(self, "_captured", None)
        if captured:
            with _GRAPH_LOCK:
                captured.clear()

    def _drop_capture(self, n: Optional[int] = None, oldest: bool = False) -> None:
        """Destroy the capture of `n` requests, the least recently used one, or (neither given) all of them."""
        with _GRAPH_LOCK:
            if oldest:
                self._captured.popitem(last=False)
            elif n is None:
                self._captured.clear()
            else:
                self._captured.pop(n, None)

    # ---- requests ------------------------------------------------------------- #
    def admit(self, rid: Hashable) -> int:
        slot = self.manager.admit(rid)
        self.storage.zero_state(slot)
        return slot

    def release(self, rid: Hashable) -> None:
        freed = self.manager.release(rid)
        self._report(freed)

    def _report(self, freed: Sequence[Sequence[int]]) -> None:
        if self.on_pages_freed is not None:
            for group, pages in enumerate(freed):
                if pages:
                    self.on_pages_freed(group, list(pages))

    # ---- the step ---------------------------------------------------------------- #
    @torch.inference_mode()
    def step(self, portions: Sequence[Portion], tokens_device: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run `portions` (pages already reserved with `CacheManager.extend`) and
        return logits [R, V], rows ordered by portion and then by `want`; None if no
        place is wanted.  Afterwards every request's length has grown by its portion
        and window groups have given back the pages that fell out of reach.  With
        `tokens_device` the token ids come from that device tensor (see `build_batch`)."""
        if (
            self.num_graphs > 0 and portions
            and all(len(p.tokens) == 1 and len(p.want) == 1 and p.want[0] == 0 and p.rid in self.manager for p in portions)
        ):
            logits = self._decode_step(portions, tokens_device)
        else:
            batch = build_batch(portions, self.manager, self.device, self.model.vocab_size, tokens_device)
            logits = self.model.forward(batch, self.storage)
        for portion in portions:
            self._report(self.manager.advance(portion.rid, len(portion.tokens)))
        return logits

    # ---- decode steps as graphs ---------------------------------------------------- #
    def _decode_step(self, portions: Sequence[Portion], tokens_device: Optional[torch.Tensor]) -> torch.Tensor:
        """A step of one token per request: the replay of its capture if there is one that still holds it,
        else the step itself, launched kernel by kernel, and then its capture for the steps to come."""
        n = len(portions)
        page = self.manager.page_size
        width = max(pages_for(self.manager.length(p.rid) + 1, page) for p in portions)
        held = self._captured.get(n)
        if held is not None and width <= held.table_width:
            batch = self._static_batch(portions, held.descriptor, held.table_width, held.plans, tokens_device)
            if held.plans.refresh(batch):
                held.graph.replay()
                self._captured.move_to_end(n)
                self.n_replays += 1
                return held.logits.clone()  # the next replay writes there again
        if held is not None:
            # outgrown: its tables or work lists have no room for this step.  Whether a step of so many requests is
            # still worth a capture at the lengths it has now is measured anew.
            self._drop_capture(n)
            self._host_share.pop(n, None)
        if self.graphs_where_host_bound and not self._worth_a_capture(n):
            return self._launched_and_timed(portions, tokens_device, n)
        table_width = width + max(width // 4, 2)
        n_groups = len(self.manager.groups)
        descriptor = torch.empty(8 * (n + 4) + n_groups * (n * table_width + 4), dtype=torch.int32, device=self.device)
        from .. import ops

        plans = ops.StaticPlans(self.device, max_keys=table_width * page)
        batch = self._static_batch(portions, descriptor, table_width, plans, tokens_device)
        try:
            logits = self.model.forward(batch, self.storage)  # this step; the work lists find their homes in it
        except ops.KernelError as exc:
            # a kernel has no form of a fixed length for this model's steps: they are launched as they come (what
            # the refused run has written to the cache, this run writes again)
            print(f"[cwm_amd] decode steps are not captured as graphs: {exc}", file=sys.stderr, flush=True)
            self.num_graphs = 0
            return self.model.forward(build_batch(portions, self.manager, self.device, self.model.vocab_size, tokens_device), self.storage)
        # No graph may be destroyed while a stream captures (HIP refuses it, and an error in a destructor ends the
        # process): whatever garbage holds one, a dropped engine for instance, is collected now, and the collector
        # stays off until the capture has ended.
        # (The collector's switch is the process's: it covers this thread's garbage and, with the lock, other
        # runners' captured steps; a graph that other code of the process destroys on another thread is not covered.)
        with _GRAPH_LOCK:
            gc.collect()
            collector_was_on = gc.isenabled()
            gc.disable()
            try:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, pool=self._graph_pool):
                    static_logits = self.model.forward(batch, self.storage)
            except Exception as exc:  # the step above has run and stands; later ones are launched kernel by kernel
                print(f"[cwm_amd] decode steps are not captured as graphs: {type(exc).__name__}: {exc}", file=sys.stderr, flush=True)
                self.num_graphs = 0
                self._captured.clear()
                self._graph_pool = None
                # the stream must have left capture mode and the device must answer, or later launches would fail
                # with an error that names none of this
                if torch.cuda.is_current_stream_capturing():
                    raise RuntimeError("a failed capture of a decode step left the stream capturing") from exc
                torch.cuda.synchronize(self.device)
                return logits
            finally:
                if collector_was_on:
                    gc.enable()
            if self._graph_pool is None:
                self._graph_pool = graph.pool()
            self._captured[n] = CapturedStep(graph, descriptor, table_width, plans, batch.tokens, static_logits)
            self.n_captures += 1
            while len(self._captured) > self.num_graphs:
                self._drop_capture(oldest=True)
        return logits

    def _worth_a_capture(self, n: int) -> bool:
        shares = self._host_share.get(n, ())
        return len(shares) >= 3 and min(shares[1:3]) >= self.HOST_BOUND_SHARE

    def _launched_and_timed(self, portions: Sequence[Portion], tokens_device: Optional[torch.Tensor], n: int) -> torch.Tensor:
        """The step, launched kernel by kernel; the first three such steps of `n` requests are timed, on the
        host and on the device (the first one of them may load libraries and does not count)."""
        import time

        shares = self._host_share.setdefault(n, [])
        batch = build_batch(portions, self.manager, self.device, self.model.vocab_size, tokens_device)
        if len(shares) >= 3:
            return self.model.forward(batch, self.storage)
        torch.cuda.synchronize(self.device)
        start = time.perf_counter()
        logits = self.model.forward(batch, self.storage)
        launched = time.perf_counter() - start
        torch.cuda.synchronize(self.device)
        shares.append(launched / max(time.perf_counter() - start, 1e-9))
        return logits

    def _static_batch(
        self, portions: Sequence[Portion], descriptor: torch.Tensor, table_width: int, plans: Any, tokens_device: Optional[torch.Tensor]
    ) -> StepBatch:
        batch = build_batch(portions, self.manager, self.device, self.model.vocab_size, None, table_width, descriptor)
        batch.static = plans
        if tokens_device is not None:
            if tokens_device.dtype != torch.int32 or tokens_device.numel() != batch.n_tokens:
                raise ValueError(f"tokens on the device must be int32 [{batch.n_tokens}]")
            batch.tokens.copy_(tokens_device.reshape(-1))
        return batch
