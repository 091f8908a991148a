"""Decode steps as HIP graphs.

A step in which every request brings exactly one token launches some four
hundred small kernels; at small batches the time to launch them from Python
exceeds the time they run.  Such steps are therefore captured once per batch
size bucket into a HIP graph (through torch's CUDAGraph, which records the
launches made on its capture stream, ours included) and replayed: the step's
tables are written into fixed device buffers, the graph runs, the logits
appear in a fixed tensor.  Rows beyond the live requests are padding: token 0
at position 0 that writes no key, whose state slot is a row of the state
tensors that no request holds, and whose logits nobody reads.

Nothing in a captured step clears memory with a memset node, and the kernels
take every size from the tables, so one graph serves any mix of context
lengths.  Among the tables are the runs of keys that the host deals the
requests' keys into for the attention (``kernels.key_runs``); what the dealing
finds (rows of several runs or none; single waves or blocks of eight) selects
among a few captured variants of the step.

A model may hold parts that cannot be captured (a mixer that loops on the host
over the step's entries).  The step is then cut into pieces at those layer
calls (``DecoderModel.graph_pieces``): the pieces that can be captured are one
graph each, the others run eagerly between the replays, on the live rows only
(never on padding: such a part may keep state per request), and hand their
result to the next graph through a fixed tensor.
"""
from __future__ import annotations

import gc
import weakref

import numpy as np
import torch

from .batch import GroupTables, StepBatch
from ..kernels.key_runs import deal_key_runs, max_key_runs


def _pad4(n: int) -> int:
    return (n + 3) & ~3


def table_layout(bucket: int, widths: list[int], run_caps: list[int]) -> tuple[list[int], int]:
    """Offsets of the sections of a decode step's packed tables (the order of
    build_step_batch) and their total length, for ``bucket`` rows; per cache group a block table
    of ``widths`` pages a row, the slots of the new tokens, ``run_caps`` runs of keys (four ints
    each) and the rows' first runs."""
    B = bucket
    sizes = [B, B, B, B + 1, B, B, B, B, B]
    for w, cap in zip(widths, run_caps):
        sizes += [B * w, B, 4 * cap, B + 1]
    offs, total = [], 0
    for n in sizes:
        offs.append(total)
        total += _pad4(n)
    return offs, total


class DecodeTables:
    """The host side of a decode graph: the packed tables of a step of one token
    per request, kept between steps in one int32 array so that a step writes
    only what changed.  Pure host code (numpy), no device.

    A row remembers whose block table it holds as (request id, the request's
    *life* in the cache, table lengths).  Only for the same life may the row be
    extended instead of rewritten: a request that was released and added again
    (preempted and computed again, or an id used twice) comes back under the
    same id with other pages.  The reference looks every location up in the
    page table itself and keeps no copy (src/core/runtime/KVCache.h:221-240);
    this copy must behave as if it did."""

    def __init__(self, cache, bucket: int, max_model_len: int, hv: np.ndarray | None = None):
        self.cache = cache
        self.B = B = int(bucket)
        ps = cache.page_size
        self.widths = [-(-max_model_len // ps) for _ in cache.groups]
        self.run_caps = [max_key_runs(B, g.spec.num_kv_heads) for g in cache.groups]
        self.offs, self.total = table_layout(B, self.widths, self.run_caps)
        if hv is None:
            hv = np.zeros(self.total, dtype=np.int32)
        if hv.dtype != np.int32 or hv.shape != (self.total,):
            raise ValueError(f"the table buffer must be int32 [{self.total}]")
        self.hv = hv
        o = self.offs
        hv[:] = 0
        hv[o[2]:o[2] + B] = np.arange(B)            # token_req
        hv[o[3]:o[3] + B + 1] = np.arange(B + 1)    # cu_tokens
        hv[o[7]:o[7] + B] = np.arange(B)            # logit rows: every row
        hv[o[8]:o[8] + B] = -1                      # no-slot mapping
        self._row_state = [None] * B                # (request, life, table lengths) last written per row
        self.host_start_pos, self.host_state_slots = [], []    # of the live rows of the last fill
        self.variant = (False, ())                  # (some row has several runs, per group: dealt for blocks) at the last fill
        self._pad_rows(0)
        self._deal_runs(0)

    def block_table_row(self, group: int, row: int) -> np.ndarray:
        w = self.widths[group]
        base = self.offs[9 + 4 * group] + row * w
        return self.hv[base:base + w]

    def _pad_rows(self, first: int) -> None:
        o, hv, B = self.offs, self.hv, self.B
        if first >= B:
            return
        hv[o[0] + first:o[0] + B] = 0               # token
        hv[o[1] + first:o[1] + B] = 0               # position
        hv[o[4] + first:o[4] + B] = 0               # start_pos
        hv[o[5] + first:o[5] + B] = 1               # context length
        hv[o[6] + first:o[6] + B] = self.cache.padding_slot   # a state row that no request holds
        for gi, w in enumerate(self.widths):
            hv[o[10 + 4 * gi] + first:o[10 + 4 * gi] + B] = -1   # writes no key
            for r in range(first, B):
                if self._row_state[r] is not None:
                    hv[o[9 + 4 * gi] + r * w:o[9 + 4 * gi] + (r + 1) * w] = 0
        for r in range(first, B):
            self._row_state[r] = None

    def fill(self, entries) -> None:
        """Writes the step's tables for ``entries`` (one token each, pages reserved)."""
        cache, o, hv = self.cache, self.offs, self.hv
        ps = cache.page_size
        R = len(entries)
        if R > self.B:
            raise ValueError(f"{R} entries do not fit a graph of {self.B} rows")
        self.host_start_pos, self.host_state_slots = [], []
        for r, e in enumerate(entries):
            P = cache.num_tokens(e.req)
            life = cache.life(e.req)
            self.host_start_pos.append(P)
            self.host_state_slots.append(cache.slot(e.req))
            hv[o[0] + r] = e.tokens[0]
            hv[o[1] + r] = P
            hv[o[4] + r] = P
            hv[o[5] + r] = P + 1
            hv[o[6] + r] = cache.slot(e.req)
            prev = self._row_state[r]
            lens = []
            for gi, w in enumerate(self.widths):
                table = cache.block_table(gi, e.req)
                base = o[9 + 4 * gi] + r * w
                n = len(table)
                old = prev[2][gi] if prev is not None else 0
                grown = prev is not None and prev[0] == e.req and prev[1] == life and n >= old
                if grown:
                    # The same stay in the cache: the table only grew at its end.  (A window gives
                    # pages back at the table's front; those entries stay as they are, no kernel
                    # reads before the window's first key.)
                    if n > old:
                        hv[base + old:base + n] = [p if p >= 0 else 0 for p in table[old:]]
                else:
                    hv[base:base + n] = [p if p >= 0 else 0 for p in table]
                    if old > n:
                        hv[base + n:base + old] = 0
                lens.append(n)
                hv[o[10 + 4 * gi] + r] = table[P // ps] * ps + P % ps
            self._row_state[r] = (e.req, life, lens)
        self._pad_rows(R)
        self._deal_runs(R)

    def _deal_runs(self, live: int) -> None:
        """The keys of all rows (a padding row has the one key of position 0) dealt into runs for
        the attention, per cache group; the first ``live`` rows are requests."""
        o, hv, B = self.offs, self.hv, self.B
        positions = hv[o[4]:o[4] + B]
        merge, blocks = False, []
        for gi, g in enumerate(self.cache.groups):
            dealt = deal_key_runs(positions, g.spec.window, g.spec.num_kv_heads,
                                  runs_out=hv[o[11 + 4 * gi]:o[11 + 4 * gi] + 4 * self.run_caps[gi]],
                                  start_out=hv[o[12 + 4 * gi]:o[12 + 4 * gi] + B + 1], live=live)
            merge = merge or dealt.merge        # some row's keys are several runs, in some group
            blocks.append(dealt.blocks)
        #: what the last fill's dealing found: the variant of the captured step that fits these tables
        self.variant = (merge, tuple(blocks))


class DecodeGraph:
    def __init__(self, runner, bucket: int):
        self._runner = weakref.ref(runner)   # the runner owns its graphs; no reference cycle
        self.B = B = int(bucket)
        cache = runner.cache
        widths = [-(-runner.max_model_len // cache.page_size) for _ in cache.groups]
        _, total = table_layout(B, widths, [max_key_runs(B, g.spec.num_kv_heads) for g in cache.groups])
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.tables = DecodeTables(cache, B, runner.max_model_len, self.host.numpy())
        self.widths = self.tables.widths
        self.offs = o = self.tables.offs
        self.dev = torch.zeros(total, dtype=torch.int32, device=runner.device)

        def sl(i, n):
            return self.dev[o[i]:o[i] + n]

        b = StepBatch()
        b.num_tokens = b.num_reqs = b.num_logit_rows = B
        b.max_new_tokens = 1
        b.max_context = runner.max_model_len
        b.token_ids, b.positions, b.token_req = sl(0, B), sl(1, B), sl(2, B)
        b.cu_tokens, b.start_pos, b.context_lens = sl(3, B + 1), sl(4, B), sl(5, B)
        b.state_slots, b.logit_rows = sl(6, B), sl(7, B)
        no_slot = sl(8, B)
        for gi, w in enumerate(self.widths):
            bt = self.dev[o[9 + 4 * gi]:o[9 + 4 * gi] + B * w].view(B, w)
            b.groups.append(GroupTables(bt, sl(10 + 4 * gi, B), no_slot,
                                        sl(11 + 4 * gi, 4 * self.tables.run_caps[gi]).view(-1, 4),
                                        sl(12 + 4 * gi, B + 1), cache.groups[gi].spec.window))
        b.host_cu_tokens = list(range(B + 1))
        b.host_start_pos = [0] * B
        b.host_state_slots = [cache.padding_slot] * B
        b.reqs = [None] * B
        self.batch = b
        # The step is captured in variants, by what the host finds when it deals the rows' keys into
        # runs: whether some row has several runs (else the kernel that merges partial attention
        # results is left out), and, per cache group, whether a run gets a block of eight waves or a
        # single one.  Each variant is captured when it is first wanted, on tables of padding rows.
        self._variants: dict[tuple, list[_Piece]] = {}
        self._padding = self.host.clone()           # the tables as they are with no live row
        self._copied = torch.cuda.Event()

    @property
    def runner(self):
        return self._runner()

    @property
    def pieces(self) -> list:
        """The pieces of the variant captured first (all variants are cut alike)."""
        return next(iter(self._variants.values())) if self._variants else []

    def fill(self, entries) -> None:
        self._copied.synchronize()      # the last copy out of the host buffer is done
        self.tables.fill(entries)

    def possible_variants(self) -> list:
        """The variants that steps in this bucket can ask for (for a warm-up that captures them
        all): single waves with and without the merge, and blocks of eight waves in the groups
        where some number of requests that runs in this bucket gets them."""
        from ..kernels.key_runs import wants_blocks
        heads = [g.spec.num_kv_heads for g in self.runner.cache.groups]
        out = [(True, (False,) * len(heads)), (False, (False,) * len(heads))]
        for r in range(self.B // 2 + 1, self.B + 1):
            v = (False, tuple(wants_blocks(r, h) for h in heads))
            if any(v[1]) and v not in out:
                out.append(v)
        return out

    def _context(self, batch):
        from .runner import StepContext
        rn = self.runner
        return StepContext(rn.ops, rn.act_dtype, batch, rn.max_model_len, rn._calls, rn.cache)

    def capture(self, variant: tuple | None = None) -> None:
        """Captures a variant of the step, unless it exists: ``variant`` = (whether partial
        attention results are merged, per cache group whether a run of keys gets a block of eight
        waves); None: with the merge, single waves."""
        if variant is None:
            variant = (True, (False,) * len(self.batch.groups))
        if variant in self._variants:
            return
        rn = self.runner
        pieces = [_Piece(safe, items) for safe, items in rn.model.graph_pieces()]
        for gt, blocks in zip(self.batch.groups, variant[1]):
            gt.runs_merge, gt.runs_for_blocks = variant[0], blocks
        # (the decode attention's launch is sized by the tables of runs of keys, whose size depends
        # on the bucket's rows only: the same launch whatever the requests hold)
        side = torch.cuda.Stream(device=rn.device)
        side.wait_stream(torch.cuda.current_stream(rn.device))
        # No collection of garbage may run while the stream records: the finaliser of an old
        # graph or tensor would make a HIP call that is illegal during capture and abort.
        gc.collect()
        gc_was_on = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.stream(side):
                # every row is padding while the step runs to warm up and to be recorded: a part
                # may keep state per request, which these runs must not touch
                self.dev.copy_(self._padding.to(rn.device))
                ctx = self._context(self.batch)
                resid = pending = None
                for piece in pieces:
                    if not piece.safe:
                        # Not run here: every row is padding now, and such a part may keep state per
                        # request.  At every step it runs on the live rows and leaves its result in
                        # this tensor, which the next graph was captured to read.
                        # (a pending term is added to the residual stream: it has the stream's shape)
                        piece.pending = torch.zeros_like(resid)
                        piece.resid, pending = resid, piece.pending
                        continue

                    def body(piece=piece, resid=resid, pending=pending):
                        r, p, logits = rn.model.run_items(ctx, piece.items, resid, pending)
                        if logits is None and p is not None:
                            p = rn.ops.as_tensor(p)     # handed on as a plain tensor
                        return r, p, logits

                    for _ in range(2):          # warm up: allocations, rotation tables
                        body()
                    side.synchronize()
                    piece.graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(piece.graph, stream=side):
                        piece.resid, piece.pending, piece.logits = body()
                    resid, pending = piece.resid, piece.pending
        finally:
            if gc_was_on:
                gc.enable()
        torch.cuda.current_stream(rn.device).wait_stream(side)
        torch.cuda.synchronize(rn.device)
        self._variants[variant] = pieces

    def _live_batch(self, R: int) -> StepBatch:
        """The first R rows of the graph's tables as a step of their own, with the host's
        copies that parts looping over entries read."""
        g, t = self.batch, self.tables
        b = StepBatch()
        b.num_tokens = b.num_reqs = b.num_logit_rows = R
        b.max_new_tokens = 1
        b.max_context = max(t.host_start_pos) + 1
        b.token_ids, b.positions, b.token_req = g.token_ids[:R], g.positions[:R], g.token_req[:R]
        b.cu_tokens, b.start_pos, b.context_lens = g.cu_tokens[:R + 1], g.start_pos[:R], g.context_lens[:R]
        b.state_slots, b.logit_rows = g.state_slots[:R], g.logit_rows[:R]
        for gt in g.groups:
            # (no runs of keys: those of the graph's tables cover its padding rows too)
            b.groups.append(GroupTables(gt.block_tables[:R], gt.slot_mapping[:R], gt.no_slot_mapping[:R]))
        b.host_cu_tokens = list(range(R + 1))
        b.host_start_pos = list(t.host_start_pos)
        b.host_state_slots = list(t.host_state_slots)
        b.reqs = [s[0] for s in t._row_state[:R]]
        return b

    def run(self, entries, token_source: torch.Tensor | None = None) -> torch.Tensor:
        """``token_source``: int32 [len(entries)] on the device with the step's tokens, for a
        step that is launched before the host knows them.  Returns the logits of the graph's
        rows ([bucket, vocab], or [len(entries), vocab] if the step's last piece ran eagerly)."""
        self.fill(entries)
        variant = self.tables.variant
        if variant not in self._variants:
            self.capture(variant)
        pieces = self._variants[variant]
        self.dev.copy_(self.host, non_blocking=True)
        self._copied.record()
        R = len(entries)
        if token_source is not None:
            self.dev[self.offs[0]:self.offs[0] + R].copy_(token_source)
        rn = self.runner
        logits = live = None
        for i, piece in enumerate(pieces):
            if piece.safe:
                piece.graph.replay()
                logits = piece.logits
                continue
            if live is None:
                live = self._context(self._live_batch(R))
            # the piece before left the residual stream and its pending term in fixed tensors;
            # this one adds to the stream's live rows in place
            before = pieces[i - 1]
            _, p, lg = rn.model.run_items(live, piece.items, piece.resid[:R],
                                          None if before.pending is None else before.pending[:R])
            if lg is not None:
                logits = lg
            else:
                piece.pending[:R].copy_(rn.ops.as_tensor(p))
        return logits


class _Piece:
    """A run of consecutive items of the step: one captured graph, or eager code."""
    __slots__ = ("safe", "items", "graph", "resid", "pending", "logits")

    def __init__(self, safe: bool, items: list):
        self.safe, self.items = safe, items
        self.graph = self.resid = self.pending = self.logits = None


def graph_buckets(max_seqs: int) -> list[int]:
    """Batch sizes that get a graph of their own: the powers of two and the sizes half way
    between them (1, 2, 3, 4, 6, 8, 12, 16, 24, ...), and the largest batch.  A step runs in
    the smallest bucket that holds it and pays for the bucket's rows: with powers of two alone
    twelve requests ran as sixteen (a tenth slower) and twenty-four as thirty-two.  A graph is
    captured when its bucket is first used."""
    out, p = set(), 1
    while p < max_seqs:
        out.add(p)
        if p >= 2 and p + p // 2 < max_seqs:
            out.add(p + p // 2)
        p *= 2
    out.add(max_seqs)
    return sorted(out)
