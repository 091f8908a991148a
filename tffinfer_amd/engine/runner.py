"""The step function: runs a batch of (request, its next tokens) through the
model from the cache and returns the logits at the wanted places.

It replaces the reference's ``prefill()`` + the body of ``decode()``'s loop +
``update_kv_cache`` (src/core/runtime/InferRuntime.cu:294-323, :348-375,
:523-529) and its kernel-launch task graph (src/core/runtime/TaskFlowManager.cu:15-56)
by straight-line code on one stream.  A step runs only the tokens it is given;
everything earlier comes from the cache.
"""
from __future__ import annotations

import torch

from ..cache.block_pool import OutOfPages
from ..cache.manager import CacheManager
from ..kernels import ops as _ops
from .batch import KVView, PinnedTables, StepBatch, StepEntry, build_step_batch
from .graphs import DecodeGraph, graph_buckets


class StepError(ValueError):
    """A batch the step function cannot run as given."""


class LayerContext:
    """What a part sees during one layer call of one step."""
    __slots__ = ("ops", "act_dtype", "batch", "max_positions", "kv", "state", "call_index")

    def __init__(self, ops, act_dtype, batch, max_positions):
        self.ops = ops
        self.act_dtype = act_dtype
        self.batch = batch
        self.max_positions = max_positions
        self.kv = None
        self.state = None
        self.call_index = -1


class StepContext(LayerContext):
    __slots__ = ("_calls", "_cache")

    def __init__(self, ops, act_dtype, batch, max_positions, calls, cache):
        super().__init__(ops, act_dtype, batch, max_positions)
        self._calls = calls
        self._cache = cache

    def for_call(self, idx: int) -> LayerContext:
        c = LayerContext(self.ops, self.act_dtype, self.batch, self.max_positions)
        c.call_index = idx
        cache_id, writes, group, k, v, state = self._calls[idx]
        if group is not None:
            gt = self.batch.groups[group]
            c.kv = KVView(k, v, gt.block_tables, gt.slot_mapping if writes else gt.no_slot_mapping,
                          self._cache.page_size, group, gt.key_runs, gt.run_start, gt.runs_window,
                          gt.runs_for_blocks, gt.runs_merge)
        c.state = state
        return c


class ModelRunner:
    def __init__(self, model, page_size: int = 16, num_pages=256, max_seqs: int = 8,
                 max_model_len: int | None = None, ops=_ops, use_graphs: bool = False):
        if model.device is None or model.device.type != "cuda":
            raise StepError("the model has no weights on a GPU; there is no CPU path")
        self.model = model
        self.ops = ops
        self.use_graphs = bool(use_graphs)
        self.device = model.device
        self.act_dtype = model.dtype
        cfg = model.config
        self.max_model_len = min(int(max_model_len or cfg.max_position_embeddings),
                                 cfg.max_position_embeddings)
        self.vocab_size = cfg.vocab_size
        reqs = model.call_requirements()
        self.cache = CacheManager(reqs, page_size, num_pages, max_seqs, dtype=self.act_dtype,
                                  device=self.device)
        self._calls = []
        for cache_id, writes, kv_spec, state_spec in reqs:
            group = self.cache.group_index(cache_id) if kv_spec is not None else None
            k = v = None
            if group is not None:
                k, v = self.cache.kv_tensors(cache_id)
            self._calls.append((cache_id, writes, group, k, v, self.cache.state_tensors.get(cache_id)))
        self._pinned = PinnedTables()     # the tables of steps that run eagerly leave through it
        # decode-only steps replay HIP graphs of the pieces of the model that can be captured
        self._graphs = {}
        self._graph_wanted = {}         # bucket -> steps that would have run in it had it been captured
        self._graph_buckets = graph_buckets(max_seqs) if (self.use_graphs and model.graph_pieces()) else []

    # ---- requests --------------------------------------------------------
    def add_request(self, req) -> int:
        return self.cache.add_request(req)

    def free_request(self, req) -> None:
        self.cache.release(req)

    def has_request(self, req) -> bool:
        return self.cache.has_request(req)

    # ---- the step --------------------------------------------------------
    def _validate(self, entries) -> None:
        seen = set()
        for e in entries:
            if not self.cache.has_request(e.req):
                raise StepError(f"request {e.req!r} is not live (add_request first)")
            if e.req in seen:
                raise StepError(f"request {e.req!r} appears twice in one step")
            seen.add(e.req)
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.req!r} brings no tokens")
            for t in e.tokens:
                if not isinstance(t, int) or not 0 <= t < self.vocab_size:
                    raise StepError(f"request {e.req!r}: token id {t!r} is outside the vocabulary "
                                    f"of {self.vocab_size}")
            for w in e.want:
                if not isinstance(w, int) or not 0 <= w < n:
                    raise StepError(f"request {e.req!r}: wanted place {w!r} is not among its {n} tokens")
            end = self.cache.num_tokens(e.req) + n
            if end > self.max_model_len:
                raise StepError(f"request {e.req!r} would reach {end} tokens, the limit is {self.max_model_len}")

    def reserve(self, entries) -> None:
        """Takes the pages the step's new tokens need, for all entries or none."""
        free = [g.pool.num_free for g in self.cache.groups]
        for e in entries:
            need = self.cache.pages_needed(e.req, len(e.tokens))
            for i, n in enumerate(need):
                free[i] -= n
        if any(f < 0 for f in free):
            short = [-f for f in free if f < 0]
            raise OutOfPages(f"the step needs {max(short)} more pages than the pool has free")
        for e in entries:
            self.cache.reserve(e.req, len(e.tokens))

    @torch.no_grad()
    def step(self, entries: list[StepEntry], token_source: torch.Tensor | None = None) -> torch.Tensor:
        """Logits (float32 [wanted, vocab], on the device) at the wanted places,
        in the order of the entries and of their ``want``.

        ``token_source`` (int32 [len(entries)], on the device) serves a step in
        which every entry brings one token that the host does not know yet (it
        was sampled by a step still running): entry i's token is
        token_source[i], whatever ``entries[i].tokens`` holds in its place."""
        if not entries:
            return torch.empty(0, self.vocab_size, dtype=torch.float32, device=self.device)
        self._validate(entries)
        if token_source is not None:
            if any(len(e.tokens) != 1 for e in entries):
                raise StepError("tokens can come from the device only in a step of one token per request")
            if token_source.dtype != torch.int32 or tuple(token_source.shape) != (len(entries),) \
                    or token_source.device != torch.device(self.device):
                raise StepError("token_source must be int32 [entries] on the runner's device")
        self.reserve(entries)
        try:
            if self._graph_buckets and len(entries) <= self._graph_buckets[-1] \
                    and all(len(e.tokens) == 1 for e in entries):
                return self._step_graph(entries, token_source)
            with torch.cuda.device(self.device):
                batch = build_step_batch(entries, self.cache, self.device, self._pinned)
                if token_source is not None:
                    batch.token_ids[:len(entries)].copy_(token_source)
                ctx = StepContext(self.ops, self.act_dtype, batch, self.max_model_len, self._calls, self.cache)
                logits = self.model.forward(ctx)
        except BaseException:
            # The step did not run to its end: its tokens are not in the cache, so the pages taken
            # for them (here or by a scheduler beforehand) go back and the requests stand where
            # they stood; the caller may run the same step again.
            for e in entries:
                self.cache.rollback(e.req)
            raise
        for e in entries:
            self.cache.commit(e.req, len(e.tokens))
        return logits

    #: steps a bucket has to be wanted for before it is captured while a graph of less than twice
    #: its rows can stand in: a capture holds the device up for some 60 ms, which the rows saved
    #: (a few percent of a step) pay back over a few hundred steps
    CAPTURE_AFTER = 64

    def _pick_bucket(self, R: int) -> int:
        """The bucket a decode step of R requests runs in: the smallest that holds it, if its
        graph exists or no existing graph of less than twice its rows can stand in for it
        (then it is captured now); otherwise that stand-in, until the smaller bucket has been
        wanted often enough to be worth its capture.  A batch that shrinks request by request
        passes through every size once and should not stop for a capture at each."""
        want = next(b for b in self._graph_buckets if b >= R)
        if want in self._graphs:
            return want
        have = min((b for b in self._graphs if want < b < 2 * want), default=None)
        if have is None:
            return want
        n = self._graph_wanted[want] = self._graph_wanted.get(want, 0) + 1
        return want if n >= self.CAPTURE_AFTER else have

    def capture_graphs(self) -> int:
        """Captures the decode graph of every bucket that has none yet (some 50 ms a variant: with
        and without the merge of partial attention results on single waves, and for blocks of eight
        waves where the bucket's rows may get them), so that no step stops for a capture later;
        returns for how many buckets it did."""
        n = 0
        with torch.cuda.device(self.device):
            for bucket in self._graph_buckets:
                if bucket not in self._graphs:
                    g = self._graphs[bucket] = DecodeGraph(self, bucket)
                    for variant in g.possible_variants():
                        g.capture(variant)
                    n += 1
        return n

    def _step_graph(self, entries, token_source=None) -> torch.Tensor:
        """A decode-only step through the HIP graph of its batch size bucket.
        The logits live in a tensor the next such step overwrites."""
        R = len(entries)
        bucket = self._pick_bucket(R)
        with torch.cuda.device(self.device):
            g = self._graphs.get(bucket)
            if g is None:
                g = self._graphs[bucket] = DecodeGraph(self, bucket)
            logits = g.run(entries, token_source)       # (captures the variant the step needs, if it is new)
            rows = [r for r, e in enumerate(entries) if e.want]
            if len(rows) == R:
                out = logits[:R]
            elif rows:
                out = logits[torch.tensor(rows, device=self.device)]
            else:
                out = logits[:0]
        for e in entries:
            self.cache.commit(e.req, 1)
        return out
