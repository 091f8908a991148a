"""The engine: model, step function, cache, scheduler and sampler together.

``LLMEngine`` is the Python entry point for generation from token ids;
``LLMInferRuntime`` (tffinfer_amd/runtime.py) wraps it in the reference's own
call sequence.
"""
from __future__ import annotations

import itertools
from dataclasses import dataclass, field

import torch

from ..models import load_model
from ..sampling import Sampler, SamplingConfig
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
    max_num_seqs: int = 8
    max_num_batched_tokens: int = 2048
    prefill_chunk: int = 512
    max_model_len: int | None = None
    memory_fraction: float = 0.85
    use_graphs: bool = True


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
        num_pages = opt.num_pages
        if num_pages is None:
            tokens = opt.kv_tokens or opt.max_num_seqs * max_len
            num_pages = -(-tokens // opt.page_size) + opt.max_num_seqs
            num_pages = self._cap_pages_by_memory(model, num_pages, opt)
        self.runner = ModelRunner(model, page_size=opt.page_size, num_pages=num_pages,
                                  max_seqs=opt.max_num_seqs, max_model_len=max_len,
                                  use_graphs=opt.use_graphs)
        self.scheduler = Scheduler(self.runner.cache,
                                   SchedulerOptions(opt.max_num_seqs, opt.max_num_batched_tokens,
                                                    opt.prefill_chunk), max_len)
        self.sampler = Sampler(model.device)
        self._ids = itertools.count()
        self.keep_logits = False
        self._results: dict = {}

    @classmethod
    def from_model_dir(cls, model_dir: str, options: EngineOptions | None = None) -> "LLMEngine":
        opt = options or EngineOptions()
        model = load_model(model_dir, resolve_dtype(opt.dtype), opt.device)
        return cls(model, opt)

    @staticmethod
    def _cap_pages_by_memory(model, num_pages: int, opt: EngineOptions) -> int:
        free, _ = torch.cuda.mem_get_info(model.device)
        esz = 2 if model.dtype == torch.bfloat16 else 4
        per_page = 0
        seen = set()
        for cache_id, _, kv, _ in model.call_requirements():
            if kv is not None and cache_id not in seen:
                seen.add(cache_id)
                per_page += 2 * kv.num_kv_heads * kv.head_dim * opt.page_size * esz
        if per_page == 0:
            return max(1, num_pages)
        fit = int(free * opt.memory_fraction) // per_page
        return max(1, min(num_pages, fit))

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
        self.scheduler.add_request(req)
        return rid

    def abort(self, request_id) -> bool:
        return self.scheduler.abort(request_id)

    @property
    def has_work(self) -> bool:
        return self.scheduler.has_work

    # ---- one step --------------------------------------------------------
    def step(self) -> list[tuple]:
        """Plans and runs one step.  Returns (request id, new token, finished)
        for every request that got a token."""
        plan = self.scheduler.schedule()
        if not plan:
            return []
        entries, sampling_rows = [], []
        for p in plan:
            toks = p.request.tokens[p.start:p.start + p.count]
            entries.append(StepEntry(p.request.id, toks, [p.count - 1] if p.samples else []))
            if p.samples:
                sampling_rows.append(p.request)
        logits = self.runner.step(entries)
        sampled = {}
        if sampling_rows:
            if self.keep_logits:
                host = logits.float().cpu()
                for r, req in enumerate(sampling_rows):
                    self._results.setdefault(req.id, []).append(host[r].clone())
            toks = self.sampler.sample(
                logits, [r.sampling for r in sampling_rows], [len(r.output) for r in sampling_rows],
                [r.tokens for r in sampling_rows])
            sampled = {req.id: t for req, t in zip(sampling_rows, toks)}
        finished = self.scheduler.update(plan, sampled)
        done = {r.id for r in finished}
        return [(rid, tok, rid in done) for rid, tok in sampled.items()]

    # ---- whole generations ----------------------------------------------
    def generate(self, prompts, sampling=None, max_new_tokens: int = 64, eos_token_id: int | None = None,
                 ignore_eos: bool = False) -> list[GenerationResult]:
        """Generates for every prompt (a list of token ids each) and returns the
        results in the order of the prompts.  ``sampling`` is one SamplingConfig
        for all or a list with one per prompt."""
        if sampling is None or isinstance(sampling, SamplingConfig):
            sampling = [sampling or SamplingConfig()] * len(prompts)
        reqs = []
        for prompt, sc in zip(prompts, sampling):
            rid = self.add_request(prompt, sc, max_new_tokens, eos_token_id, ignore_eos)
            reqs.append(self.scheduler.waiting[-1])
            assert reqs[-1].id == rid
        while self.scheduler.has_work:
            self.step()
        return [GenerationResult(r.id, r.prompt, r.output, r.finish_reason, r.num_preemptions,
                                 self._results.pop(r.id, [])) for r in reqs]
