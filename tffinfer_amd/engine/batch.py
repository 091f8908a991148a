"""A step's batch: entries as the caller gives them, and the flat device tables
the kernels read.

The reference's LLMBatch is a flat token list with positions, sequence ids and
a logits flag per token (src/core/runtime/BatchManager.h:77-99), but a forward
there holds one whole prompt or one decode token of one sequence
(src/core/runtime/InferRuntime.cu:415-416, :429).  Here any number of entries
of any length share a step.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..kernels.key_runs import deal_key_runs


@dataclass
class StepEntry:
    """The next tokens of one request and the places among them whose logits
    are wanted (indices into ``tokens``; may be empty)."""
    req: object
    tokens: list
    want: list = field(default_factory=list)


class KVView:
    """What a mixer sees of the cache in one layer call."""
    __slots__ = ("k_cache", "v_cache", "block_tables", "slot_mapping", "page_size", "group", "key_runs",
                 "run_start", "runs_window", "runs_for_blocks", "runs_merge")

    def __init__(self, k_cache, v_cache, block_tables, slot_mapping, page_size, group, key_runs=None,
                 run_start=None, runs_window=0, runs_for_blocks=False, runs_merge=True):
        self.k_cache = k_cache
        self.v_cache = v_cache
        self.block_tables = block_tables
        self.slot_mapping = slot_mapping     # per token; -1: not written (a call that only reads, padding)
        self.page_size = page_size
        self.group = group
        # a step of one token per request: the requests' visible keys dealt into runs of similar
        # length (kernels.key_runs), for a window of runs_window, for single waves or for blocks
        # of eight; else None
        self.key_runs = key_runs
        self.run_start = run_start
        self.runs_window = runs_window
        self.runs_for_blocks = runs_for_blocks
        self.runs_merge = runs_merge         # False: every request is one run, no result is partial


class GroupTables:
    __slots__ = ("block_tables", "slot_mapping", "no_slot_mapping", "key_runs", "run_start", "runs_window",
                 "runs_for_blocks", "runs_merge")

    def __init__(self, block_tables, slot_mapping, no_slot_mapping, key_runs=None, run_start=None, runs_window=0,
                 runs_for_blocks=False, runs_merge=True):
        self.block_tables = block_tables        # int32 [R, max_blocks]
        self.slot_mapping = slot_mapping        # int32 [T]: page * page_size + offset of each new token
        self.no_slot_mapping = no_slot_mapping  # int32 [T] of -1: for calls that only read a cache
        self.key_runs = key_runs                # int32 [runs, 4] or None (kernels.key_runs)
        self.run_start = run_start              # int32 [R + 1] or None
        self.runs_window = runs_window
        self.runs_for_blocks = runs_for_blocks
        self.runs_merge = runs_merge            # False: the host knows that every request is one run


class StepBatch:
    """Flat tables of one step, on the device (int32) and on the host.

    token_ids[T], positions[T], token_req[T] (row of the token's request in
    this step's tables), cu_tokens[R+1], start_pos[R] (tokens cached before
    the step), context_lens[R] (after it), state_slots[R], logit_rows[K].
    """

    def __init__(self):
        self.num_tokens = 0
        self.num_reqs = 0
        self.num_logit_rows = 0
        self.max_new_tokens = 0          # longest entry
        self.max_context = 0
        self.token_ids = self.positions = self.token_req = None
        self.cu_tokens = self.start_pos = self.context_lens = None
        self.state_slots = self.logit_rows = None
        self.groups: list[GroupTables] = []
        # host copies for parts that loop over entries
        self.host_cu_tokens: list = []
        self.host_start_pos: list = []
        self.host_state_slots: list = []
        self.reqs: list = []


def _pad4(n: int) -> int:
    return (n + 3) & ~3


class PinnedTables:
    """A pinned host buffer for the step's tables that is used again step after step: to pin
    memory anew for every step costs more than the copy it speeds up.  The copy out of it is
    asynchronous, so the next step waits for that copy (an event) before it writes."""

    def __init__(self, ints: int = 1 << 16):
        self._buf = torch.empty(int(ints), dtype=torch.int32, pin_memory=True)
        self._copied = torch.cuda.Event()
        self._busy = False

    def take(self, ints: int) -> torch.Tensor:
        if self._busy:
            self._copied.synchronize()
            self._busy = False
        if ints > self._buf.numel():
            self._buf = torch.empty(max(int(ints), 2 * self._buf.numel()), dtype=torch.int32, pin_memory=True)
        return self._buf[:ints]

    def copied(self) -> None:
        """To be called right after the copy to the device was queued."""
        self._copied.record()
        self._busy = True


def build_step_batch(entries, cache, device, pinned: PinnedTables | None = None) -> StepBatch:
    """Packs all tables of a step into one host buffer and sends it with one
    copy.  ``cache`` is the CacheManager; pages for the new tokens must have
    been reserved.  ``pinned``: the caller's reusable pinned buffer (else pageable
    memory, and a copy that waits)."""
    b = StepBatch()
    R = len(entries)
    tok, pos, treq, cu, start, ctxl, slots, rows = [], [], [], [0], [], [], [], []
    for r, e in enumerate(entries):
        P = cache.num_tokens(e.req)
        n = len(e.tokens)
        tok.extend(e.tokens)
        pos.extend(range(P, P + n))
        treq.extend([r] * n)
        base = cu[-1]
        rows.extend(base + w for w in e.want)
        cu.append(base + n)
        start.append(P)
        ctxl.append(P + n)
        slots.append(cache.slot(e.req))
        b.max_new_tokens = max(b.max_new_tokens, n)
        b.max_context = max(b.max_context, P + n)
    T = cu[-1]
    sections = [tok, pos, treq, cu, start, ctxl, slots, rows, [-1] * T]
    group_meta = []
    for gi, g in enumerate(cache.groups):
        tables = [cache.block_table(gi, e.req) for e in entries]
        width = max(1, max((len(t) for t in tables), default=1))
        flat = []
        for t in tables:
            flat.extend(p if p >= 0 else 0 for p in t)
            flat.extend([0] * (width - len(t)))
        sm = []
        for e, P in zip(entries, start):
            sm.extend(cache.slot_mapping(gi, e.req, P, len(e.tokens)))
        group_meta.append((len(sections), width))
        sections.append(flat)
        sections.append(sm)
        # a step of one token per request: the requests' keys dealt into runs for the attention
        if b.max_new_tokens == 1:
            dealt = deal_key_runs(start, g.spec.window, g.spec.num_kv_heads)
            sections.append(dealt.runs.reshape(-1))
            sections.append(dealt.run_start)
            group_meta[-1] += (dealt.blocks, dealt.merge)
    offs, total = [], 0
    for s in sections:
        offs.append(total)
        total += _pad4(len(s))
    host = pinned.take(max(total, 4)) if pinned is not None else torch.empty(max(total, 4), dtype=torch.int32)
    hv = host.numpy()
    for s, o in zip(sections, offs):
        if len(s):
            hv[o:o + len(s)] = s
    dev = host.to(device, non_blocking=True)
    if pinned is not None:
        pinned.copied()

    def sl(i, n):
        return dev[offs[i]:offs[i] + n]

    b.num_tokens, b.num_reqs, b.num_logit_rows = T, R, len(rows)
    b.token_ids, b.positions, b.token_req = sl(0, T), sl(1, T), sl(2, T)
    b.cu_tokens, b.start_pos, b.context_lens = sl(3, R + 1), sl(4, R), sl(5, R)
    b.state_slots, b.logit_rows = sl(6, R), sl(7, len(rows))
    no_slot = sl(8, T)
    for (si, width, *dealt), g in zip(group_meta, cache.groups):
        bt = dev[offs[si]:offs[si] + R * width].view(R, width)
        gt = GroupTables(bt, sl(si + 1, T), no_slot)
        if dealt:
            gt.key_runs = sl(si + 2, len(sections[si + 2])).view(-1, 4)
            gt.run_start = sl(si + 3, R + 1)
            gt.runs_window = g.spec.window
            gt.runs_for_blocks, gt.runs_merge = dealt
        b.groups.append(gt)
    b.host_cu_tokens, b.host_start_pos, b.host_state_slots = cu, start, slots
    b.reqs = [e.req for e in entries]
    return b
