"""The generation engine: a model, its cache, the step function, the scheduler and
the sampler behind the reference's interface, token ids in and token ids out.

    engine = Engine.from_folder("model_dir", GenArgs(max_batch=8, max_seq=4096))
    q = queue.Queue(); q.put(Packet("a", tokens=[1, 2, 3], max_gen=16)); q.put(None)
    for packet in engine.generate(q): ...

`generate(q)` follows the contract of the reference's generator
(cwm/fastgen/api.py:68-86; loop cwm/fastgen/generate.py:446-519): requests are read
from a queue, results come back in completion order linked by `thread_id`, None in
the queue ends it once running requests are done, and None may be yielded to hand
control back.
"""

from __future__ import annotations

import logging
import os
import queue
import signal
import time
import weakref
from typing import Any, Dict, Generator, Hashable, Iterable, List, Optional, Sequence, Union

import torch

from ..cache.manager import CacheManager
from ..cache.storage import CacheStorage
from ..models.model import Model
from ..parts.base import PagedKVSpec
from ..sampling.sampler import RequestStream, Sampler, effective_temperature
from .api import GenArgs, Packet
from .loading import load_model, random_model
from .metrics import MetricsLog
from .runner import ModelRunner, weak_callback
from .scheduler import Request, Scheduler


def pool_sizes(
    model: Model,
    args: GenArgs,
    device: torch.device,
    free_bytes: Optional[int] = None,
) -> Dict[Hashable, int]:
    """Pages of every layer group, keyed by what the group's cache need answers to `retention()`
    (its window; None for the group that keeps all keys).

    With `max_seq` given, the keep-all group holds that many tokens
    (cwm/fastgen/generate.py:245-251) and a group with window W the same, or less if
    `max_batch` requests cannot fill it: a request never holds more than W - 1 + max_prefill
    tokens there (plus a page of slack at either end).

    With a negative `max_seq` the pools share what is free on the device after a reserve for
    activations (the reference's rule, cwm/fastgen/utils/tune.py:90-107, which knows one pool
    only).  The split follows what one expected request needs of each group: `expected_seq`
    tokens of the keep-all group against min(expected_seq, W - 1 + max_prefill) of a window
    group; `expected_seq` defaults to the context length that the model's configuration
    names.  Without either, every group gets room for the same number of tokens.  A window
    group is never made larger than `max_batch` requests can fill; what that saves goes to the
    keep-all group.  No pool is sized for the worst case of `max_batch` requests up front:
    when any group runs out of pages the scheduler preempts, whichever group it is.
    `free_bytes` stands in for the measured free memory (tests).
    """
    page = args.cache_block
    esize = 4 if model.runtime.act_dtype == torch.float32 else 2
    per_page: Dict[Hashable, int] = {}
    kept: Dict[Hashable, Optional[int]] = {}  # most tokens one request holds of a group; None: all
    for spec in model.cache_specs:
        if isinstance(spec, PagedKVSpec):
            key = spec.retention()
            per_page[key] = per_page.get(key, 0) + spec.bytes_per_token(esize) * page
            span = spec.keys_kept(args.max_prefill)
            kept[key] = None if span is None else spec.pinned_keys() + span
    if not per_page:
        return {}
    keep_all = [key for key in per_page if kept[key] is None]

    def request_cap(tokens: int) -> int:
        """Most pages that `max_batch` requests can hold of a group that keeps `tokens` of each."""
        return args.max_batch * ((tokens + page - 1) // page + 2)

    sizes: Dict[Hashable, int] = {}
    if args.max_seq > 0:
        cap_pages = (args.max_seq + page - 1) // page
        for key in per_page:
            sizes[key] = max(1, cap_pages if kept[key] is None else min(request_cap(kept[key]), cap_pages))
        return sizes

    if free_bytes is None:
        if device.type != "cuda":
            raise ValueError("max_seq must be given when no HIP device is used")
        free_bytes, _total = torch.cuda.mem_get_info(device)
    # nine tenths of what is free after the reserve: the rest is slack for the allocator
    budget = int(0.9 * (free_bytes - int(args.prefill_gb * 1e9)))
    expected = args.expected_seq if args.expected_seq > 0 else (model.plan.max_positions or 0)
    # pages that one expected request holds of each group
    share: Dict[Hashable, int] = {}
    for key in per_page:
        if expected <= 0:
            share[key] = 1
        else:
            tokens = expected if kept[key] is None else min(expected, kept[key])
            share[key] = (tokens + page - 1) // page + 1
    per_request = sum(share[key] * per_page[key] for key in per_page)
    requests = budget / per_request if budget > 0 else 0.0
    for key in per_page:
        sizes[key] = int(requests * share[key])
        if kept[key] is not None and sizes[key] > request_cap(kept[key]):
            sizes[key] = request_cap(kept[key])
    if keep_all:  # what the caps saved
        rest = budget - sum(sizes[key] * per_page[key] for key in per_page if kept[key] is not None)
        per_token = sum(per_page[key] for key in keep_all)
        for key in keep_all:
            sizes[key] = max(sizes[key], rest // per_token)
    smallest = min(sizes.values())
    if smallest < 1:
        raise MemoryError(
            f"{free_bytes / 1e9:.1f} GB of free memory less {args.prefill_gb} GB for activations leave no room for "
            f"one page of {page} tokens in every layer group (bytes per page: {per_page})"
        )
    return sizes


class Engine:
    def __init__(
        self,
        args: GenArgs,
        model: Model,
        stop_tokens: Iterable[int] = (),
        seed: int = 17,
    ) -> None:
        if model.runtime is None:
            raise RuntimeError("the model has no weights yet")
        self.args = args
        self.model = model
        self.device = model.runtime.device
        self.stop_tokens = set(int(t) for t in stop_tokens)
        self.seed = seed
        self.max_batch = args.max_batch
        sizes = pool_sizes(model, args, self.device)
        self.manager = CacheManager(model.cache_specs, args.cache_block, sizes, args.max_batch)
        self.storage = CacheStorage(self.manager, self.device, model.runtime.act_dtype)
        # decode steps as graphs, one per number of requests (the reference captures one per bucket of batch sizes and
        # pads, cwm/fastgen/generate.py:313-373, and has the same switch to go without)
        use_graphs = not os.environ.get("FG_NO_CUDA_GRAPHS")
        self.runner = ModelRunner(
            model, self.manager, self.storage, num_graphs=max(0, args.num_cuda_graphs) if use_graphs else 0, graphs_where_host_bound=True
        )
        # a request joins others only when its known tokens and some room to decode fit
        # (the reference asks for 128 tokens of room, cwm/fastgen/generate.py:596-597)
        self.scheduler = Scheduler(self.manager, args.max_batch, args.max_prefill, headroom=min(128, args.cache_block))
        self.sampler = Sampler(self.device)
        self.metrics = MetricsLog()
        self.scheduler.on_event = weak_callback(self._scheduler_event)
        self._last_active = 0
        # a window of traced steps (cwm/fastgen/generate.py:148-156,397-434)
        self._profile_state = "inactive"
        self._profile_iter = 0
        self._profile_ctx: Any = None
        self.profile_iters = int(os.environ.get("FG_PROFILE_ITERS", "8"))
        self.profile_dir = os.environ.get("FG_PROFILE_DIR", "/tmp")
        self.last_profile_path: Optional[str] = None
        if None in sizes:
            self.max_seq = sizes[None] * args.cache_block
        else:
            self.max_seq = args.max_seq if args.max_seq > 0 else max(sizes.values()) * args.cache_block
        # counters in the manner of the reference's throughput log (serve/fgserve.py:330-349)
        self.n_steps = 0  # model steps
        self.n_iterations = 0  # calls of step(): a burst of decode steps is one
        self.n_sequences = 0
        self.n_generated = 0
        self._reported = 0
        self.last_step_tokens = 0  # tokens and sequences that the latest step ran
        self.last_step_sequences = 0
        self.last_step_burst = 1  # decode steps that the latest call of step() ran without a host sync between them

    # ---- construction ------------------------------------------------------------ #
    @classmethod
    def from_folder(
        cls,
        checkpoint_dir: str,
        args: Optional[GenArgs] = None,
        dtype: Union[str, torch.dtype] = "bfloat16",
        device: Union[str, torch.device] = "cuda:0",
        stop_tokens: Iterable[int] = (),
        seed: int = 17,
    ) -> "Engine":
        model, _config = load_model(checkpoint_dir, dtype, device)
        return cls(args or GenArgs(), model, stop_tokens, seed)

    @classmethod
    def from_random(
        cls,
        config: Dict[str, Any],
        weight_seed: int,
        args: Optional[GenArgs] = None,
        dtype: Union[str, torch.dtype] = "bfloat16",
        device: Union[str, torch.device] = "cuda:0",
        stop_tokens: Iterable[int] = (),
        seed: int = 17,
        std: float = 0.02,
    ) -> "Engine":
        model, _config = random_model(config, weight_seed, dtype, device, std=std)
        return cls(args or GenArgs(), model, stop_tokens, seed)

    # ---- requests ----------------------------------------------------------------- #
    def submit(self, packet: Packet) -> None:
        """Queue a request (cwm/fastgen/generate.py:86-106: its longest length is
        prompt + max_gen, capped by the cache)."""
        if packet.stop_str is not None:
            raise ValueError("stop_str needs a tokenizer; this engine takes and gives token ids only")
        if not packet.tokens:
            raise ValueError(f"request {packet.thread_id!r} has no prompt tokens")
        for tok in packet.tokens:
            if not 0 <= int(tok) < self.model.vocab_size:
                raise ValueError(f"request {packet.thread_id!r}: token id {tok} is outside the vocabulary")
        max_gen = packet.max_gen if packet.max_gen is not None else self.args.max_gen
        max_len = self.max_seq if max_gen is None else min(len(packet.tokens) + max_gen, self.max_seq)
        temperature = packet.temperature if packet.temperature is not None else self.args.temperature
        top_p = packet.top_p if packet.top_p is not None else self.args.top_p
        request = Request(
            rid=packet.thread_id,
            prompt=[int(t) for t in packet.tokens],
            max_len=max_len,
            temperature=effective_temperature(self.args.use_sampling, temperature),
            top_p=float(top_p),
            rng=RequestStream(self.seed, packet.seed if packet.seed is not None else packet.thread_id),
            want_logprobs=self.args.logprobs or self.args.prompt_logprobs,
            want_prompt_logprobs=self.args.prompt_logprobs,
        )
        self.scheduler.add(request)

    def _packet(self, request: Request) -> Packet:
        self.n_sequences += 1
        return Packet(
            thread_id=request.rid,
            tokens=list(request.generated),
            # with prompt_logprobs the prompt's scores come first (cwm/fastgen/generate.py:719-724)
            logprobs=(list(request.prompt_logprobs) + list(request.logprobs)) if request.want_logprobs else None,
            sample_logprobs=list(request.sample_logprobs) if request.want_logprobs else None,
            max_gen=len(request.generated),
            finish_reason=request.finish_reason,
        )

    # ---- events and profiles ----------------------------------------------------------- #
    def _scheduler_event(self, kind: str, request: Request) -> None:
        if kind == "admit" and request.preemptions > 0:
            self.metrics.record("unpark", tokens=len(request))
        elif kind == "preempt":
            self.metrics.record("preempt", tokens=len(request))

    def install_profile_signal(self, profile_sig: int = signal.SIGUSR2) -> bool:
        """Make `profile_sig` (SIGUSR2, as the reference's default) call `request_profile`, so that a window
        of steps can be traced from outside the process (`kill -USR2 PID`); cwm/fastgen/generate.py:139,
        159-169,405-406.  As there, a handler that is already set is left alone (returns False).  Only the
        main thread can set a handler.  The handler holds the engine weakly."""
        log = logging.getLogger("cwm_amd")
        if signal.getsignal(profile_sig) is not signal.SIG_DFL:
            log.warning("Signal handler for %s is set; the profile handler was not installed", profile_sig)
            return False
        ref = weakref.ref(self)

        def handler(_signum: int, _frame: Any) -> None:
            engine = ref()
            if engine is not None:
                engine.request_profile()

        signal.signal(profile_sig, handler)
        log.info("Profiling signal handler set for signal %s", profile_sig)
        return True

    def request_profile(self) -> None:
        """Trace the next `profile_iters` steps (FG_PROFILE_ITERS, default 8) with torch's
        profiler and write a Chrome trace into `profile_dir` (FG_PROFILE_DIR, default /tmp);
        cwm/fastgen/generate.py:397-434."""
        if self._profile_state == "inactive":
            self._profile_state = "requested"

    def _profile_step(self) -> None:
        if self._profile_state == "active":
            self._profile_iter += 1
            if self._profile_iter >= self.profile_iters:
                self._profile_done()
            return
        if self._profile_state != "requested":
            return
        from torch.profiler import ProfilerActivity, profile

        activities = [ProfilerActivity.CPU]
        if self.device.type == "cuda":
            activities.append(ProfilerActivity.CUDA)
        self._profile_iter = 0
        self._profile_ctx = profile(activities=activities)
        self._profile_ctx.__enter__()
        self._profile_state = "active"

    def _profile_done(self) -> None:
        if self._profile_state != "active":
            self._profile_state = "inactive"
            return
        self._profile_state = "inactive"
        ctx, self._profile_ctx = self._profile_ctx, None
        ctx.__exit__(None, None, None)
        path = os.path.join(self.profile_dir, f"cwm_amd_{time.strftime('%y%m%d-%H%M%S')}_{os.getpid()}.json.gz")
        ctx.export_chrome_trace(path)
        self.last_profile_path = path

    # ---- one step -------------------------------------------------------------------- #
    def step(self) -> List[Packet]:
        """Schedule, run and sample one step; returns the requests it finished."""
        sched = self.scheduler
        self.n_iterations += 1
        if self._profile_state != "inactive":
            self._profile_step()
        already = 0 if not sched.finished else len(sched.finished)
        # a request that may not grow at all is done before it starts
        for request in list(sched.waiting):
            if request.max_len <= len(request.prompt):
                sched.waiting.remove(request)
                sched._finish(request, "length")
        batch = sched.schedule()
        if len(sched.running) != self._last_active:
            self._last_active = len(sched.running)
            if self.metrics.enabled():
                self.metrics.record(
                    "nactive", lanes=self._last_active, free_pages=self.manager.free_pages(),
                    pages=[g.pool.num_pages for g in self.manager.groups],
                )
        for item in batch:
            if item.start == 0 and item.request.cached == 0:
                self.storage.zero_state(self.manager.slot(item.request.rid))
        self.last_step_sequences = len(batch)
        self.last_step_tokens = sum(item.count for item in batch)
        burst = 1
        if batch and self.args.sync_freq > 1 and all(item.count == 1 and item.wants_logits for item in batch):
            if not any(item.request.want_prompt_logprobs and len(item.request.prompt_logprobs) < len(item.request.prompt) - 1 for item in batch):
                burst = sched.reserve_burst(batch, self.args.sync_freq)
        self.last_step_burst = burst
        if burst > 1:
            self._decode_burst(batch, burst)
        elif batch:
            logits = self.runner.step(sched.portions(batch))
            self.n_steps += 1
            # rows of `logits`: per entry its prompt places, then its sampling place
            wanting, sample_rows = [], []
            score_rows, score_targets, score_owner = [], [], []
            row = 0
            for item in batch:
                request = item.request
                for place in item.prompt_places:
                    score_rows.append(row)
                    score_targets.append(request.prompt[item.start + place + 1])
                    score_owner.append(request)
                    row += 1
                if item.wants_logits:
                    wanting.append(request)
                    sample_rows.append(row)
                    row += 1
            if score_rows:
                from .. import ops

                packed = torch.tensor([score_rows, score_targets], dtype=torch.int32).to(self.device)
                scores = ops.token_logprobs(logits, packed[0].contiguous(), packed[1].contiguous()).tolist()
                for request, value in zip(score_owner, scores):
                    request.prompt_logprobs.append(float(value))
            if wanting:
                rows_logits = logits if len(sample_rows) == logits.shape[0] else logits[sample_rows]
                tokens, logprobs, sample_logprobs = self.sampler.sample(
                    rows_logits,
                    [r.temperature for r in wanting],
                    [r.top_p for r in wanting],
                    [r.rng.next_uniform() if r.temperature > 0 else 0.0 for r in wanting],
                )
                self.n_generated += len(tokens)
            else:
                tokens, logprobs, sample_logprobs = [], [], []
            sched.step_done(batch, tokens, self.stop_tokens, logprobs, sample_logprobs)
        out = [self._packet(r) for r in sched.finished[already:]]
        for packet in out:
            self.metrics.record("yield", tokens=len(packet.tokens))
        # what has been handed back is not kept: a long-lived generate(q) would collect every request
        del sched.finished[:]
        return out

    def _decode_burst(self, batch: List[Any], steps: int) -> None:
        """`steps` decode steps of the same requests without a word from the host in between
        (cwm/fastgen/generate.py:729-809): each step's tokens are sampled on the device and feed
        the next step from there; tokens and log-probabilities come to the host once, at the end.
        Pages for all the steps are reserved (`Scheduler.reserve_burst`)."""
        from .batch import Portion

        requests = [item.request for item in batch]
        n = len(requests)
        params = torch.tensor(
            [[r.temperature for r in requests], [r.top_p for r in requests]]
            + [[r.rng.next_uniform() if r.temperature > 0 else 0.0 for r in requests] for _ in range(steps)],
            dtype=torch.float32,
        )
        if self.device.type == "cuda":
            params = params.pin_memory()
        params = params.to(self.device, non_blocking=True)
        first = self.scheduler.portions(batch)
        results = []
        tokens_device = None
        for k in range(steps):
            portions = first if k == 0 else [Portion(rid=r.rid, tokens=[0], want=[0]) for r in requests]
            logits = self.runner.step(portions, tokens_device)
            packed = self.sampler.sample_packed(logits, params[0], params[1], params[2 + k])
            tokens_device = packed[0]
            results.append(packed)
        self.n_steps += steps
        host = torch.stack(results).cpu()  # [steps, 3, requests]: one copy for the whole burst
        tokens, logprobs, sample_logprobs = [], [], []
        for k in range(steps):
            t, a, b = self.sampler.unpack(host[k])
            tokens.append(t)
            logprobs.append(a)
            sample_logprobs.append(b)
        before = sum(len(r.generated) for r in requests)
        self.scheduler.burst_done(batch, tokens, self.stop_tokens, logprobs, sample_logprobs)
        self.n_generated += sum(len(r.generated) for r in requests) - before

    # ---- the reference's generator interface ------------------------------------------ #
    def generate(self, q: "queue.Queue[Optional[Packet]]") -> Generator[Optional[Packet], None, None]:
        eoq = False
        iterations = 0
        while not eoq or self.scheduler.has_work():
            while not eoq:
                try:
                    packet = q.get(block=not self.scheduler.has_work())
                except queue.Empty:
                    break
                if packet is None:
                    eoq = True
                    break
                self.submit(packet)
            if not self.scheduler.has_work():
                continue
            for packet in self.step():
                yield packet
            iterations += 1
            if self.args.handover_frequency > 0 and iterations % self.args.handover_frequency == 0:
                yield None
        self._profile_done()

    def generate_tokens(
        self,
        prompts: Sequence[Sequence[int]],
        max_gen: Optional[int] = None,
        temperature: Optional[float] = None,
        top_p: Optional[float] = None,
    ) -> List[List[int]]:
        """Generated token ids for each prompt, in the order of the prompts."""
        q: "queue.Queue[Optional[Packet]]" = queue.Queue()
        for i, prompt in enumerate(prompts):
            q.put(Packet(thread_id=i, tokens=list(prompt), max_gen=max_gen, temperature=temperature, top_p=top_p))
        q.put(None)
        results: Dict[int, List[int]] = {}
        for packet in self.generate(q):
            if packet is not None:
                results[packet.thread_id] = packet.tokens
        return [results[i] for i in range(len(prompts))]
