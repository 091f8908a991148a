"""The engine: model, step function, cache, scheduler and sampler together.

``LLMEngine`` is the Python entry point for generation from token ids;
``LLMInferRuntime`` (tffinfer_amd/runtime.py) wraps it in the reference's own
call sequence.
"""
from __future__ import annotations

import itertools
from dataclasses import dataclass, field

import numpy as np
import torch

from ..kernels import staging as _staging
from ..models import load_model
from ..sampling import Sampler, SamplingConfig, SeenTokens
from .batch import StepEntry
from .runner import ModelRunner
from .scheduler import Request, Scheduler, SchedulerOptions

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32,
           "fp32": torch.float32, torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


@dataclass
class EngineOptions:
    """Run-time options.  The reference fixes these at compile time
    (PAGE_SIZE 32 in src/core/runtime/KVCache.h:16; MAX_SEQ_LENGTH 8192 and
    MAX_BATCH_SIZE 512 in src/core/global/GlobalDefine.h:39-40)."""
    dtype: object = "bfloat16"
    device: str = "cuda:0"
    page_size: int = 16
    #: pages per cache group; if None, sized from ``kv_tokens``
    num_pages: int | None = None
    #: tokens the cache holds; if None too, max_num_seqs * max_model_len capped by free memory
    kv_tokens: int | None = None
    #: or bytes of device memory for keys and values, all layers together (whole pages of it are used)
    kv_bytes: int | None = None
    max_num_seqs: int = 8
    max_num_batched_tokens: int = 2048
    prefill_chunk: int = 512
    #: steps a little over a multiple of this many tokens are cut down to the multiple (the
    #: scheduler's rule 5); None: 256 for bfloat16 (the row tile of the matrix-core products), off for float32
    token_quantum: int | None = None
    max_model_len: int | None = None
    memory_fraction: float = 0.85
    use_graphs: bool = True
    #: launch a decode step before the host has read the tokens of the one before it
    run_ahead: bool = True
    #: capture the decode graphs of all batch sizes when the engine is made (some 50 ms each)
    #: instead of at the first step that wants one
    warm_up: bool = False


@dataclass
class _Launched:
    """A step whose kernels are queued and whose tokens the host has not read yet."""
    plan: list
    rows: list                      # the requests that sample, in the order of the logit rows
    tokens: torch.Tensor | None     # int32 [rows] on the device
    host: torch.Tensor | None       # the same in pinned host memory, valid after ``ready``
    ready: torch.cuda.Event | None
    logits: torch.Tensor | None = None   # float32 [rows, vocab] in pinned host memory, if kept


@dataclass
class GenerationResult:
    id: object
    prompt: list
    output: list
    finish_reason: str
    num_preemptions: int = 0
    logits: list = field(default_factory=list)   # float32 rows at sampled positions, if kept


def resolve_dtype(d) -> torch.dtype:
    try:
        return _DTYPES[d]
    except KeyError:
        raise ValueError(f"dtype {d!r} is not supported (bfloat16 or float32)") from None


class LLMEngine:
    def __init__(self, model, options: EngineOptions | None = None):
        self.options = opt = options or EngineOptions()
        self.model = model
        cfg = model.config
        max_len = min(opt.max_model_len or cfg.max_position_embeddings, cfg.max_position_embeddings)
        if sum(x is not None for x in (opt.num_pages, opt.kv_tokens, opt.kv_bytes)) > 1:
            raise ValueError("give one of num_pages, kv_tokens and kv_bytes")
        num_pages = opt.num_pages
        if num_pages is None:
            num_pages = self.plan_cache(model, opt, max_len)
        self.runner = ModelRunner(model, page_size=opt.page_size, num_pages=num_pages,
                                  max_seqs=opt.max_num_seqs, max_model_len=max_len,
                                  use_graphs=opt.use_graphs)
        quantum = opt.token_quantum
        if quantum is None:
            quantum = 256 if model.dtype == torch.bfloat16 else 0
        self.scheduler = Scheduler(self.runner.cache,
                                   SchedulerOptions(opt.max_num_seqs, opt.max_num_batched_tokens,
                                                    opt.prefill_chunk, int(quantum)), max_len)
        self.sampler = Sampler(model.device)
        self._ids = itertools.count()
        self.keep_logits = False
        self._results: dict = {}
        self._requests: dict = {}
        self._ahead: _Launched | None = None   # a decode step launched ahead of its predecessor's tokens
        self.steps_ahead = 0                   # how many steps were launched that way
        if opt.warm_up:
            self.warm_up()

    @classmethod
    def from_model_dir(cls, model_dir: str, options: EngineOptions | None = None) -> "LLMEngine":
        opt = options or EngineOptions()
        model = load_model(model_dir, resolve_dtype(opt.dtype), opt.device)
        return cls(model, opt)

    @staticmethod
    def plan_cache(model, opt: "EngineOptions", max_len: int, free_bytes: int | None = None) -> dict:
        """Pages for every group of layers (``cache.sizing.plan_pages``): from ``kv_bytes``, or from
        ``kv_tokens`` (by default what ``max_num_seqs`` requests of the longest length hold)
        capped by ``memory_fraction`` of the free device memory, of which the per-request state
        tensors come off first.  A group with a window gets the pages its window and a step's
        tokens need, not the full pool."""
        from ..cache.sizing import plan_pages
        reqs = model.call_requirements()
        esz = 2 if model.dtype == torch.bfloat16 else 4
        budget = max(opt.max_num_batched_tokens, opt.prefill_chunk)
        try:
            if opt.kv_bytes is not None:
                return plan_pages(reqs, opt.page_size, esz, opt.max_num_seqs, budget, kv_bytes=int(opt.kv_bytes))
            if free_bytes is None:
                free_bytes = int(torch.cuda.mem_get_info(model.device)[0] * opt.memory_fraction)
            tokens = opt.kv_tokens or opt.max_num_seqs * max_len
            return plan_pages(reqs, opt.page_size, esz, opt.max_num_seqs, budget, tokens=tokens,
                              free_bytes=free_bytes)
        except ValueError as e:
            raise ValueError(f"{e} (kv_bytes={opt.kv_bytes}, kv_tokens={opt.kv_tokens}, page_size={opt.page_size})") from None

    def warm_up(self) -> int:
        """What a server does before it takes requests: the decode graphs of all batch sizes are
        captured now and not at the first step that wants one.  Returns the number of captures."""
        n = self.runner.capture_graphs()
        # torch loads a kernel's code when it is first launched (the row selection below took
        # 0.2 s once): the one torch kernel of the decode loop is launched here, on nothing
        dev = self.model.device
        if torch.device(dev).type == "cuda":
            self._take_rows(torch.zeros(2, dtype=torch.int32, device=dev), np.zeros(1, dtype=np.int32))
            torch.cuda.synchronize(dev)
        return n

    @staticmethod
    def _take_rows(tokens: torch.Tensor, keep: np.ndarray) -> torch.Tensor:
        """tokens[keep] on the device; the indices go through pinned memory without a wait (a copy
        from pageable memory would hold the host until the step in flight has ended, and the
        device idle for as long afterwards)."""
        return torch.index_select(tokens, 0, _staging.send(tokens.device, [keep])[0])

    # ---- requests --------------------------------------------------------
    def add_request(self, prompt_ids, sampling: SamplingConfig | None = None, max_new_tokens: int = 64,
                    eos_token_id: int | None = None, ignore_eos: bool = False, request_id=None):
        rid = next(self._ids) if request_id is None else request_id
        prompt = [int(t) for t in prompt_ids]
        V = self.model.config.vocab_size
        for t in prompt:
            if not 0 <= t < V:
                raise ValueError(f"token id {t} is outside the vocabulary of {V}")
        if eos_token_id is None and not ignore_eos:
            eos_token_id = getattr(self.model.config, "eos_token_id", None)
        req = Request(rid, prompt, sampling or SamplingConfig(), int(max_new_tokens), eos_token_id, ignore_eos)
        if rid in self._requests and self._requests[rid].status != "finished":
            raise ValueError(f"request id {rid!r} is in use")
        self.scheduler.add_request(req)
        self._requests[rid] = req
        self._results.pop(rid, None)
        return rid

    def pop_result(self, request_id) -> GenerationResult:
        """The result of a request that has finished (by length, stop token or abort); the
        engine forgets the request."""
        r = self._requests[request_id]
        if r.status != "finished":
            raise ValueError(f"request {request_id!r} has not finished")
        del self._requests[request_id]
        return GenerationResult(r.id, r.prompt, r.output, r.finish_reason, r.num_preemptions,
                                self._results.pop(r.id, []))

    def abort(self, request_id) -> bool:
        return self.scheduler.abort(request_id)

    @property
    def has_work(self) -> bool:
        return self.scheduler.has_work or self._ahead is not None

    # ---- one step --------------------------------------------------------
    # Decoding one token per request leaves the device idle from the moment the host reads the
    # sampled tokens until the next step's kernels are queued: a quarter of a millisecond of
    # planning, table writing and graph launch per step.  While the batch only decodes, the
    # next step is therefore launched *before* the tokens of the step in flight are read: its
    # input tokens go from the sampler's output to the step's token table on the device, and
    # everything else about it (positions, pages, random draws) the host knows beforehand.
    # A request that turns out to have ended with the token just read (end of sequence) has
    # one token computed in vain; it is dropped when that step completes.
    def _launch(self, plan, token_source=None) -> _Launched:
        entries, rows = [], []
        for p in plan:
            if token_source is None:
                toks = p.request.tokens[p.start:p.start + p.count]
            else:
                toks = [0]            # in token_source
            entries.append(StepEntry(p.request.id, toks, [p.count - 1] if p.samples else []))
            if p.samples:
                rows.append(p.request)
        logits = self.runner.step(entries, token_source)
        if not rows:
            return _Launched(plan, rows, None, None, None)
        kept = None
        if self.keep_logits:
            # copied on the stream, before a penalty changes the rows and before the next
            # replay of a decode graph writes its logits tensor again
            kept = torch.empty(logits.shape, dtype=torch.float32, pin_memory=True)
            kept.copy_(logits, non_blocking=True)
        ahead = 0 if token_source is None else 1      # outputs the host has not appended yet
        seen = None
        if any(r.sampling.repetition_penalty != 1.0 for r in rows):
            seen = [self._seen_tokens(r) if r.sampling.repetition_penalty != 1.0 else None for r in rows]
        tokens = self.sampler.sample_on_device(
            logits, [r.sampling for r in rows], [len(r.output) + ahead for r in rows], seen)
        host = torch.empty(len(rows), dtype=torch.int32, pin_memory=True)
        host.copy_(tokens, non_blocking=True)
        ready = torch.cuda.Event()
        ready.record()
        return _Launched(plan, rows, tokens, host, ready, kept)

    @staticmethod
    def _seen_tokens(req):
        """The distinct tokens of the request's prompt and output, kept with the request and
        brought up to date with the tokens it got since."""
        tracker = getattr(req, "_seen_tokens", None)
        if tracker is None:
            tracker = req._seen_tokens = SeenTokens()
        return tracker.update(req.tokens)

    def _complete(self, st: _Launched) -> list[tuple]:
        """Reads the step's tokens and tells the scheduler.  Requests that ended
        or were taken away while the step ran are passed over."""
        plan = [p for p in st.plan if p.request.status == "running"]
        sampled = {}
        if st.rows:
            st.ready.synchronize()
            for r, (req, t) in enumerate(zip(st.rows, st.host.tolist())):
                if req.status == "running":
                    sampled[req.id] = t
                    if st.logits is not None:
                        self._results.setdefault(req.id, []).append(st.logits[r].clone())
        finished = self.scheduler.update(plan, sampled)
        done = {r.id for r in finished}
        return [(rid, tok, rid in done) for rid, tok in sampled.items()]

    def _plan_ahead(self, st: _Launched):
        """The decode step after ``st``, planned without its tokens: every request
        of ``st`` that its length does not end goes on.  None when the step after
        needs the scheduler (admissions, prompts, pages running out, a penalty on
        seen tokens)."""
        if not self.options.run_ahead or not st.rows:
            return None
        sch = self.scheduler
        if any(p.count != 1 or not p.samples for p in st.plan) or len(st.plan) != len(sch.running):
            return None
        if sch.waiting and len(sch.running) < sch.opt.max_num_seqs and self.runner.cache.slots.num_free > 0:
            return None     # somebody may be admitted
        plan = []
        for p in st.plan:
            req = p.request
            if req.status != "running" or req.sampling.repetition_penalty != 1.0:
                return None
            n_out = len(req.output) + 1           # with the token in flight
            if n_out >= req.max_new_tokens or len(req.prompt) + n_out >= sch.max_model_len:
                continue                          # that token is its last
            plan.append(type(p)(req, p.start + 1, 1, True))
        if not plan:
            return None
        need = [0] * len(self.runner.cache.groups)
        for p in plan:
            for gi, k in enumerate(self.runner.cache.pages_needed(p.request.id, 1)):
                need[gi] += k
        if any(k > g.pool.num_free for k, g in zip(need, self.runner.cache.groups)):
            return None
        return plan

    def step(self) -> list[tuple]:
        """Plans and runs one step.  Returns (request id, new token, finished)
        for every request that got a token, and (request id, None, True) for a
        request that was dropped because the cache cannot hold it even alone
        (finish reason "refused")."""
        st = self._ahead
        self._ahead = None
        dropped = []
        if st is None:
            plan = self.scheduler.schedule()
            # requests that turned out not to fit the cache even alone: finished without a token
            dropped = [(r.id, None, True) for r in self.scheduler.refused]
            self.scheduler.refused.clear()
            if not plan:
                return dropped
            st = self._launch(plan)
        nxt = self._plan_ahead(st)
        failed = None
        if nxt is not None:
            src = st.tokens
            if len(nxt) != len(st.rows):          # some requests end with the token in flight
                going = {id(p.request) for p in nxt}
                src = self._take_rows(st.tokens, np.asarray([i for i, r in enumerate(st.rows) if id(r) in going],
                                                            dtype=np.int32))
            try:
                self._ahead = self._launch(nxt, src)
                self.steps_ahead += 1
            except Exception as e:
                # The step ahead did not run (its pages went back); the step in flight did and is
                # completed first, so that scheduler and cache agree before the error is raised.
                failed = e
        done = dropped + self._complete(st)
        if failed is not None:
            raise failed
        return done

    # ---- whole generations ----------------------------------------------
    def generate(self, prompts, sampling=None, max_new_tokens: int = 64, eos_token_id: int | None = None,
                 ignore_eos: bool = False) -> list[GenerationResult]:
        """Generates for every prompt (a list of token ids each) and returns the
        results in the order of the prompts.  ``sampling`` is one SamplingConfig
        for all or a list with one per prompt."""
        if sampling is None or isinstance(sampling, SamplingConfig):
            sampling = [sampling or SamplingConfig()] * len(prompts)
        ids = [self.add_request(prompt, sc, max_new_tokens, eos_token_id, ignore_eos)
               for prompt, sc in zip(prompts, sampling)]
        while self.has_work:
            self.step()
        return [self.pop_result(rid) for rid in ids]
