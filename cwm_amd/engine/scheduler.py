"""Continuous batching: admits requests, cuts prompts into portions under a token
budget, puts single decoded tokens beside them, finishes requests and frees their
pages; decides what happens when pages run out.

Host logic only (it talks to the `CacheManager`, not to the device), so its
decisions are tested without a GPU.

Differences from the reference's scheduler (cwm/fastgen/generate.py:446-658,
811-994) are those of having one mixed step: the reference alternates a decode
burst with a chunked prefill and holds admissions back until enough prompt tokens
have gathered (:645-653); here every step takes one token from each decoding
request first and fills the rest of the budget (`max_prefill`, :55) with prompt
portions in arrival order, so no such threshold is needed.

A request joins running ones only when every group has free pages for all of its known
tokens and `headroom` more (the reference admits a lane when prompt + 128 tokens fit,
:596-597,627-640): one that was let in with part of its prompt would be the shortest
when pages run out, lose what it has computed and come back, over and over.

When pages run out (`CacheManager.extend` fails):
  * for a decoding request, the shortest running request is preempted, as the
    reference parks the shortest lane (:540-566): its pages are given back, it goes
    to the back of the parked queue and is later recomputed from prompt + generated
    tokens (:107-109,841); parked requests are admitted before new ones (:604-606);
  * a prompt portion is shortened to what fits, or waits for the next step;
  * a request that cannot fit even alone in an empty cache ends with
    finish_reason "cache" (the reference asserts instead, :240-243,757).
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Any, Callable, Deque, Hashable, List, Optional, Sequence, Set

from ..cache.manager import CacheManager
from .batch import Portion

WAITING, RUNNING, PARKED, FINISHED = "waiting", "running", "parked", "finished"


@dataclass
class Request:
    rid: Hashable
    prompt: List[int]
    max_len: int  # the sequence ends when it holds this many tokens
    temperature: float = 0.0
    top_p: float = 1.0
    rng: Any = None
    want_logprobs: bool = False
    want_prompt_logprobs: bool = False
    prompt_logprobs: List[float] = field(default_factory=list)  # entry p: log P(prompt[p + 1] | prompt[: p + 1])
    generated: List[int] = field(default_factory=list)
    logprobs: List[float] = field(default_factory=list)
    sample_logprobs: List[float] = field(default_factory=list)
    state: str = WAITING
    cached: int = 0  # tokens whose keys and values are in the cache
    preemptions: int = 0
    finish_reason: Optional[str] = None
    arrival: int = 0

    def all_tokens(self) -> List[int]:
        """cwm/fastgen/generate.py:107-109."""
        return self.prompt + self.generated

    def __len__(self) -> int:
        return len(self.prompt) + len(self.generated)

    def tokens_between(self, start: int, end: int) -> List[int]:
        """all_tokens()[start:end] without joining the two lists (a decoded token is one element)."""
        n = len(self.prompt)
        if end <= n:
            return self.prompt[start:end]
        if start >= n:
            return self.generated[start - n : end - n]
        return self.prompt[start:] + self.generated[: end - n]

    @property
    def pending(self) -> int:
        """Known tokens not yet in the cache."""
        return len(self) - self.cached


@dataclass
class Scheduled:
    request: Request
    start: int  # index of the portion's first token in all_tokens()
    count: int
    wants_logits: bool  # the portion ends the known tokens: its last place yields the next token
    prompt_places: List[int] = field(default_factory=list)  # places whose logits score the prompt's own next token


class Scheduler:
    def __init__(self, manager: CacheManager, max_batch: int, max_tokens_per_step: int, headroom: int = 0) -> None:
        self.manager = manager
        self.max_batch = max_batch
        self.max_tokens_per_step = max_tokens_per_step
        self.headroom = headroom  # tokens of room to decode that a request needs beside its known tokens to join others
        self.waiting: Deque[Request] = deque()
        self.parked: Deque[Request] = deque()
        self.running: List[Request] = []
        self.finished: List[Request] = []  # the caller may empty it once it has taken what it needs
        self._arrivals = 0
        self._preempted_now = False
        self.events: Deque[str] = deque(maxlen=4096)  # the latest admit / preempt / finish events, in order
        self.n_preemptions = 0
        self.on_event: Optional[Callable[[str, Request], None]] = None  # called as on_event("admit" | "preempt" | "finish", request)

    def _event(self, kind: str, request: Request, detail: str = "") -> None:
        self.events.append(f"{kind} {request.rid}{detail}")
        if self.on_event is not None:
            self.on_event(kind, request)

    # ---- queue ---------------------------------------------------------------- #
    def add(self, request: Request) -> None:
        if not request.prompt:
            raise ValueError(f"request {request.rid!r} has an empty prompt")
        request.arrival = self._arrivals
        self._arrivals += 1
        request.state = WAITING
        self.waiting.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.parked or self.running)

    # ---- helpers ---------------------------------------------------------------- #
    def _tokens_that_fit(self, request: Request, wanted: int) -> int:
        """Largest count <= wanted whose pages every group can supply now."""
        if not self.manager.groups:
            return wanted
        page = self.manager.page_size
        reserved = len(self.manager.table(0, request.rid))  # logical pages, the same in every group
        free = min(self.manager.free_pages())
        room = (reserved + free) * page - self.manager.length(request.rid)
        return max(0, min(wanted, room))

    def _fits_whole(self, request: Request) -> bool:
        """Whether every group has free pages for the request's known tokens and the headroom
        (capped by the request's own longest length).  A window group never holds more of a
        request than its window and one step's tokens."""
        total = max(len(request), min(len(request) + self.headroom, request.max_len))
        page = self.manager.page_size
        for group, free in zip(self.manager.groups, self.manager.free_pages()):
            if group.most_pages(total, self.max_tokens_per_step, page) > free:
                return False
        return True

    def _preempt(self, victim: Request) -> None:
        """Give back a running request's pages; it is recomputed later."""
        self.manager.release(victim.rid)
        self.running.remove(victim)
        victim.state = PARKED
        victim.cached = 0
        victim.preemptions += 1
        self._preempted_now = True
        self.parked.append(victim)
        self.n_preemptions += 1
        self._event("preempt", victim)

    def _finish(self, request: Request, reason: str) -> None:
        if request.rid in self.manager:
            self.manager.release(request.rid)
        if request in self.running:
            self.running.remove(request)
        request.state = FINISHED
        request.finish_reason = reason
        self.finished.append(request)
        self._event("finish", request, f" {reason}")

    # ---- one step's batch ------------------------------------------------------ #
    def schedule(self) -> List[Scheduled]:
        """Choose this step's portions and reserve their pages."""
        budget = self.max_tokens_per_step
        self._preempted_now = False
        batch: List[Scheduled] = []
        in_batch: Set[Hashable] = set()

        # 1. one token for every decoding request
        for request in sorted([r for r in self.running if r.pending == 1 and r.cached > 0], key=lambda r: r.arrival):
            if request.state != RUNNING or budget <= 0:
                continue
            while not self.manager.extend(request.rid, 1):
                others = [r for r in self.running if r.rid not in in_batch]
                if len(self.running) == 1:
                    # alone and the cache is full: it ends here (cwm/fastgen/generate.py:572-577)
                    self._finish(request, "cache")
                    break
                victim = min(others, key=lambda r: (len(r), -r.arrival)) if others else request
                self._preempt(victim)
                if victim is request:
                    break
            if request.state != RUNNING:
                continue
            batch.append(Scheduled(request, request.cached, 1, True))
            in_batch.add(request.rid)
            budget -= 1

        # 2. prompt portions of running requests, in arrival order
        for request in sorted([r for r in self.running if r.rid not in in_batch and r.pending >= 1], key=lambda r: r.arrival):
            if budget <= 0:
                break
            count = self._tokens_that_fit(request, min(request.pending, budget))
            if count <= 0:
                continue
            if not self.manager.extend(request.rid, count):
                continue
            batch.append(Scheduled(request, request.cached, count, count == request.pending))
            in_batch.add(request.rid)
            budget -= count

        # 3. admissions: parked requests first, then new ones
        # (not in a step that had to preempt: the pages just freed are for those who run)
        while budget > 0 and len(self.running) < self.max_batch and self.manager.has_free_slot() and not self._preempted_now:
            source = self.parked if self.parked else self.waiting
            if not source:
                break
            request = source[0]
            if self.running and not self._fits_whole(request):
                break  # it waits until it fits beside those who run (alone, it takes what there is)
            self.manager.admit(request.rid)
            count = self._tokens_that_fit(request, min(request.pending, budget))
            if count <= 0 or not self.manager.extend(request.rid, count):
                self.manager.release(request.rid)
                if not self.running:
                    # an empty cache cannot hold even its first token
                    source.popleft()
                    self._finish(request, "cache")
                    continue
                break
            source.popleft()
            request.state = RUNNING
            self.running.append(request)
            self._event("admit", request)
            batch.append(Scheduled(request, request.cached, count, count == request.pending))
            in_batch.add(request.rid)
            budget -= count

        # 4. nothing could be scheduled although requests run: they all wait for pages
        #    that only they themselves hold.  Preempt the shortest and let the rest go on.
        if not batch and self.running:
            if len(self.running) == 1:
                self._finish(self.running[0], "cache")
            else:
                self._preempt(min(self.running, key=lambda r: (len(r), -r.arrival)))
            return self.schedule()
        return batch

    def reserve_burst(self, batch: Sequence[Scheduled], steps: int) -> int:
        """`batch` holds one decoded token per request and its pages are reserved.  Reserve pages
        for up to `steps` tokens each (the reference grows every lane to len + sync_freq before a
        burst of decode steps, cwm/fastgen/generate.py:545-580), no further than any request may
        grow; all or nothing: returns the steps reserved, 1 if the further pages are not there."""
        steps = min([steps] + [item.request.max_len - len(item.request) for item in batch])
        if steps <= 1:
            return 1
        # pages for `steps` tokens from each request's length on (the first token's are held already): do the
        # pools have them, all requests together?
        need = [0] * len(self.manager.groups)
        for item in batch:
            for g, missing in enumerate(self.manager.pages_missing(item.request.rid, steps)):
                need[g] += missing
        if any(n > free for n, free in zip(need, self.manager.free_pages())):
            return 1
        for item in batch:
            if not self.manager.extend(item.request.rid, steps):
                raise AssertionError("pages that were counted free are not there")
        return steps

    def burst_done(
        self,
        batch: Sequence[Scheduled],
        tokens: Sequence[Sequence[int]],
        stop_tokens: Set[int],
        logprobs: Optional[Sequence[Sequence[float]]] = None,
        sample_logprobs: Optional[Sequence[Sequence[float]]] = None,
    ) -> None:
        """`tokens[k][i]` is the token that step k of a burst sampled for the i-th request of
        `batch`; step k + 1 has already run on it.  A request that stops inside the burst keeps
        the tokens up to its stop token (cwm/fastgen/generate.py:681-727); what ran after it is
        dropped with its pages."""
        for i, item in enumerate(batch):
            request = item.request
            for k in range(len(tokens)):
                request.cached += 1
                token = int(tokens[k][i])
                request.generated.append(token)
                if logprobs is not None:
                    request.logprobs.append(float(logprobs[k][i]))
                if sample_logprobs is not None:
                    request.sample_logprobs.append(float(sample_logprobs[k][i]))
                if token in stop_tokens:
                    self._finish(request, "stop")
                    break
                if len(request) >= request.max_len:
                    self._finish(request, "length")
                    break

    def portions(self, batch: Sequence[Scheduled]) -> List[Portion]:
        out = []
        for item in batch:
            request = item.request
            toks = request.tokens_between(item.start, item.start + item.count)
            item.prompt_places = []
            if request.want_prompt_logprobs:
                # prompt positions not scored yet (a recomputed request has its scores already)
                first = max(item.start, len(request.prompt_logprobs))
                last = min(item.start + item.count, len(request.prompt) - 1)
                item.prompt_places = [p - item.start for p in range(first, last)]
            want = list(item.prompt_places)
            if item.wants_logits:
                want.append(item.count - 1)
            out.append(Portion(rid=request.rid, tokens=toks, want=want))
        return out

    # ---- after the step ---------------------------------------------------------- #
    def step_done(
        self,
        batch: Sequence[Scheduled],
        next_tokens: Sequence[int],
        stop_tokens: Set[int],
        logprobs: Optional[Sequence[float]] = None,
        sample_logprobs: Optional[Sequence[float]] = None,
    ) -> List[Request]:
        """`next_tokens[i]` is the token sampled for the i-th entry of `batch` that
        wanted logits.  Returns the requests that finished with this step."""
        done: List[Request] = []
        k = 0
        for item in batch:
            request = item.request
            request.cached += item.count
            if not item.wants_logits:
                continue
            token = int(next_tokens[k])
            request.generated.append(token)
            if logprobs is not None:
                request.logprobs.append(float(logprobs[k]))
            if sample_logprobs is not None:
                request.sample_logprobs.append(float(sample_logprobs[k]))
            k += 1
            # cwm/fastgen/generate.py:681-727: a stop token ends the request and is kept
            if token in stop_tokens:
                self._finish(request, "stop")
                done.append(request)
            elif len(request) >= request.max_len:
                self._finish(request, "length")
                done.append(request)
        return done
