"""The scheduler above the step function: admits requests, cuts prompts into
portions under a token budget, decodes, finishes and frees, and decides what
happens when pages run out.

The reference runs its prompts strictly one after another, each as one whole
prefill and a token-by-token loop (src/core/runtime/InferRuntime.cu:281-292,
:348-375), truncates prompts longer than the context with a warning
(:399-403), and ignores a failed page allocation
(src/core/runtime/KVCache.cpp:23-27, InferRuntime.cu:525-527).  Continuous
batching is named there only as future work (docs/TFFInfer-1.md:1419-1429).

Rules of a step, in this order:

1. every running request that waits for one token (decoding) gets it; if the
   pool cannot give a page for it, the most recently admitted running request
   is preempted — its pages are freed, its tokens (prompt and output) are kept
   and it goes to the front of the waiting queue to be computed again — until
   the page is there;
2. running requests with more of their prompt to compute get a portion of at
   most ``prefill_chunk`` tokens, cut down to the token budget and to what the
   free pages hold, oldest first;
3. waiting requests are admitted in arrival order while a slot is free, budget
   is left and pages for a first portion are free; the queue is not overtaken;
4. if nothing at all could be scheduled although requests are running, the most
   recently admitted one is preempted and the step is planned again;
5. with a ``token_quantum`` (the row tile of the products, 256 rows on the
   matrix cores): a step whose tokens exceed a multiple of the quantum by a
   little (a quarter of it at most) is cut down to the multiple, by shortening
   the last prompt portion that does not end its prompt.  A step's time is a
   staircase in its rows: at the 8B shape 512 rows take 9.0 ms and 520 rows
   10.9 ms, so a portion of 512 beside 24 decoding requests is better cut to
   488 tokens (the step a sixth shorter for a twentieth fewer prompt tokens).

A request that could never fit the pool or the model's length is refused when
it is added, with an error, not truncated: a group that keeps every key must
hold all its tokens, a group with a window the pages that one more token
touches (portions are cut to what the free pages hold, however large the token
budget lets them grow).  A request that passes this check and still does not
fit the cache when it is alone is taken out of the queue and finished with the
reason "refused" (``Scheduler.refused`` holds such requests until the engine
reports them), so that the requests behind it run.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

from ..cache.manager import CacheManager
from ..cache.sizing import min_window_pages
from ..sampling.params import SamplingConfig


class RequestRefused(ValueError):
    """A request that can never run on this engine."""


@dataclass
class Request:
    id: object
    prompt: list
    sampling: SamplingConfig = field(default_factory=SamplingConfig)
    max_new_tokens: int = 64
    eos_token_id: int | None = None
    ignore_eos: bool = False
    output: list = field(default_factory=list)
    num_computed: int = 0           # tokens whose keys and values are in the cache
    status: str = "waiting"         # waiting | running | finished
    finish_reason: str | None = None
    num_preemptions: int = 0

    @property
    def tokens(self) -> list:
        return self.prompt + self.output

    @property
    def num_pending(self) -> int:
        return len(self.prompt) + len(self.output) - self.num_computed


@dataclass
class ScheduledPortion:
    request: Request
    start: int
    count: int
    samples: bool   # the portion reaches the request's last token: its logits pick the next one


@dataclass
class SchedulerOptions:
    max_num_seqs: int = 8
    max_num_batched_tokens: int = 2048
    prefill_chunk: int = 512
    #: > 0: steps a little over a multiple of this many tokens are cut down to the multiple (rule 5)
    token_quantum: int = 0


@dataclass
class SchedulerStats:
    steps: int = 0
    tokens: int = 0
    preemptions: int = 0
    finished: int = 0


class Scheduler:
    def __init__(self, cache: CacheManager, options: SchedulerOptions, max_model_len: int):
        if options.max_num_seqs > cache.max_seqs:
            raise ValueError(f"max_num_seqs={options.max_num_seqs} exceeds the cache's {cache.max_seqs} slots")
        if options.max_num_batched_tokens < options.max_num_seqs:
            raise ValueError("the token budget must allow one token for every running request")
        self.cache = cache
        self.opt = options
        self.max_model_len = int(max_model_len)
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []   # in order of admission
        self.refused: list[Request] = []   # finished as "refused" by schedule(), not yet reported
        self.stats = SchedulerStats()

    # ---- requests --------------------------------------------------------
    def add_request(self, req: Request) -> None:
        n = len(req.prompt)
        if n == 0:
            raise RequestRefused(f"request {req.id!r} has an empty prompt")
        if req.max_new_tokens < 1:
            raise RequestRefused(f"request {req.id!r} asks for no new token")
        total = n + req.max_new_tokens
        if total > self.max_model_len:
            raise RequestRefused(
                f"request {req.id!r}: {n} prompt tokens + {req.max_new_tokens} new tokens exceed the "
                f"length limit of {self.max_model_len}")
        ps = self.cache.page_size
        # the last token chosen is never fed back, so total - 1 tokens reach the cache
        pages = -(-(total - 1) // ps)
        for g in self.cache.groups:
            # a group with a window must hold what one more token touches; portions are cut to
            # what the free pages hold (_fit), so no larger bound is needed for the request to run
            need = pages if g.spec.window <= 0 else min(pages, min_window_pages(g.spec.window, ps))
            if need > g.pool.num_pages:
                raise RequestRefused(
                    f"request {req.id!r} needs {need} cache pages, the pool has {g.pool.num_pages} in all")
        req.status = "waiting"
        self.waiting.append(req)

    def abort(self, req_id) -> bool:
        for r in list(self.waiting):
            if r.id == req_id:
                self.waiting.remove(r)
                self._finish(r, "abort", live=False)
                return True
        for r in self.running:
            if r.id == req_id:
                self.running.remove(r)
                self._finish(r, "abort", live=True)
                return True
        return False

    @property
    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- planning a step -------------------------------------------------
    def _fit(self, req: Request, want: int, free: list[int]) -> int:
        """Most tokens up to ``want`` whose pages the free counts allow."""
        ps = self.cache.page_size
        st_tokens = self.cache.num_tokens(req.id)
        n = want
        for gi, g in enumerate(self.cache.groups):
            have = len(g.tables[req.id]) * ps - st_tokens
            n = min(n, have + free[gi] * ps)
        return max(0, n)

    def _take(self, req: Request, n: int, free: list[int]) -> None:
        need = self.cache.pages_needed(req.id, n)
        self.cache.reserve(req.id, n)
        for gi, k in enumerate(need):
            free[gi] -= k

    def _preempt_last(self) -> Request:
        victim = self.running.pop()
        self.cache.release(victim.id)
        victim.num_computed = 0
        victim.status = "waiting"
        victim.num_preemptions += 1
        self.stats.preemptions += 1
        self.waiting.appendleft(victim)
        return victim

    def schedule(self) -> list[ScheduledPortion]:
        """Plans one step and reserves its pages.  Empty when nothing is left to do."""
        while True:
            plan = self._plan()
            if plan or not (self.running or self.waiting):
                return plan
            if self.running:
                self._preempt_last()
            else:
                # nothing runs and the head of the queue still does not fit: it never will
                head = self.waiting.popleft()
                self._finish(head, "refused", live=False)
                self.refused.append(head)

    def _plan(self) -> list[ScheduledPortion]:
        budget = self.opt.max_num_batched_tokens
        free = [g.pool.num_free for g in self.cache.groups]
        plan: list[ScheduledPortion] = []
        # 1. decoding requests, oldest first
        i = 0
        while i < len(self.running):
            req = self.running[i]
            if req.num_pending == 1:
                while self._fit(req, 1, free) < 1:
                    victim = self._preempt_last()
                    plan = [p for p in plan if p.request is not victim]
                    free = [g.pool.num_free for g in self.cache.groups]
                    if victim is req:
                        break
                if req.status != "running":
                    continue  # it was itself the last one; the list is shorter now
                self._take(req, 1, free)
                plan.append(ScheduledPortion(req, req.num_computed, 1, True))
                budget -= 1
            i += 1
        # 2. running requests still computing their prompt
        for req in self.running:
            if req.num_pending > 1 and budget > 0:
                n = self._fit(req, min(req.num_pending, self.opt.prefill_chunk, budget), free)
                if n >= 1:
                    self._take(req, n, free)
                    plan.append(ScheduledPortion(req, req.num_computed, n, n == req.num_pending))
                    budget -= n
        # 3. admissions in arrival order
        while self.waiting and budget > 0 and len(self.running) < self.opt.max_num_seqs \
                and self.cache.slots.num_free > 0:
            req = self.waiting[0]
            want = min(req.num_pending, self.opt.prefill_chunk, budget)
            ps = self.cache.page_size
            n = min([want] + [f * ps for f in free])
            if n < 1:
                break
            self.waiting.popleft()
            self.cache.add_request(req.id)
            req.status = "running"
            self.running.append(req)
            self._take(req, n, free)
            plan.append(ScheduledPortion(req, req.num_computed, n, n == req.num_pending))
            budget -= n
        # 4. prefill_chunk bounds the time of a step for the sake of the requests that decode in it.
        #    In a step in which none does, what is left of the budget goes to the prompts, in their order.
        if budget > 0 and plan and not any(p.samples and p.count == 1 and p.start > 0 for p in plan):
            for i, p in enumerate(plan):
                rest = p.request.num_pending - p.count
                if rest <= 0 or budget <= 0:
                    continue
                n = self._fit(p.request, p.count + min(rest, budget), free)
                if n > p.count:
                    self._take(p.request, n, free)
                    budget -= n - p.count
                    plan[i] = ScheduledPortion(p.request, p.start, n, n == p.request.num_pending)
        # 5. a step a little over a multiple of the quantum is cut down to the multiple
        q = self.opt.token_quantum
        total = sum(p.count for p in plan)
        if q > 0 and total > q and 0 < total % q <= q // 4:
            cut = total % q
            for i in range(len(plan) - 1, -1, -1):
                p = plan[i]
                if not p.samples and p.count > cut:
                    n = p.count - cut
                    self.cache.rollback(p.request.id, keep_new=n)      # the pages of the tokens cut away
                    plan[i] = ScheduledPortion(p.request, p.start, n, False)
                    break
        return plan

    # ---- after the step --------------------------------------------------
    def update(self, plan: list[ScheduledPortion], sampled: dict) -> list[Request]:
        """The step ran (the runner committed the tokens to the cache).
        ``sampled`` maps request id -> token for portions that sample.
        Returns the requests that finished."""
        self.stats.steps += 1
        finished = []
        for p in plan:
            req = p.request
            req.num_computed += p.count
            self.stats.tokens += p.count
            if not p.samples:
                continue
            tok = int(sampled[req.id])
            req.output.append(tok)
            reason = None
            if not req.ignore_eos and req.eos_token_id is not None and tok == req.eos_token_id:
                reason = "stop"
            elif len(req.output) >= req.max_new_tokens:
                reason = "length"
            elif len(req.prompt) + len(req.output) >= self.max_model_len:
                reason = "length"
            if reason:
                self.running.remove(req)
                self._finish(req, reason, live=True)
                finished.append(req)
        return finished

    def _finish(self, req: Request, reason: str, live: bool) -> None:
        if live:
            self.cache.release(req.id)
        req.status = "finished"
        req.finish_reason = reason
        self.stats.finished += 1
