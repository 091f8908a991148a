"""The cache manager: keys and values in pages with a block table per request,
one pool per group of layers with the same needs, and slots for per-request
state of fixed size.

A *cache id* names one layer call's cache (``LayerCall.cache``).  Cache ids
whose mixers ask for the same ``KVCacheSpec`` (kv heads, head size, window)
form a *group*: the group has its own pool of pages, and a request has one
block table per group, shared by all cache ids of the group — page p holds the
same token slots in each of them.  A group that keeps all keys gives pages back
when the request ends; a group with a window also gives back every page the
window has passed, after each step.

Device layout per group: one tensor ``kv[cache index, 0 = K / 1 = V, page, ...]``;
a key page is ``[kv head, slot in page, head element]``, a value page is kept
transposed, ``[kv head, head element, slot in page]``, so that the slots of one
element lie side by side as a matrix-core operand of P.V wants them.

Reference: LLMKVCache / PageManager / LayerKVContext
(src/core/runtime/KVCache.h:24-31, :36-184, :189-262, :267-473): pages of 32
tokens per (sequence, layer), location = (page_table[i / bs], i % bs)
(:221-226), a new page when the count reaches pages * bs (:232-240); kernels
there see a table of raw addresses per token (src/kernel/cuda/get_row.cu:73-109),
here block ids and arithmetic.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..parts.base import KVCacheSpec, StateSpec
from .block_pool import BlockPool, OutOfPages
from .state_slots import StateSlots


@dataclass
class CacheGroup:
    spec: KVCacheSpec
    page_size: int
    pool: BlockPool
    cache_ids: list = field(default_factory=list)
    tables: dict = field(default_factory=dict)   # request -> [page id or -1 per logical block]
    kv: torch.Tensor | None = None

    def index_of(self, cache_id: int) -> int:
        return self.cache_ids.index(cache_id)


@dataclass
class RequestCacheState:
    slot: int
    num_tokens: int = 0
    #: unique to this stay of the request in the cache: a request that is released and added
    #: again under the same id (preemption, an id used twice) gets another one
    life: int = 0


class CacheManager:
    def __init__(self, requirements, page_size: int, num_pages, max_seqs: int,
                 dtype: torch.dtype | None = None, device=None):
        """``requirements``: (cache id, writes, KVCacheSpec | None, StateSpec | None)
        per layer call.  ``num_pages``: pages of every group's pool, or a dict
        {KVCacheSpec: pages}.  Device memory is taken only if ``device`` is given."""
        if page_size <= 0 or page_size % 8:
            raise ValueError(f"page size {page_size} must be a positive multiple of 8")
        self.page_size = int(page_size)
        self.max_seqs = int(max_seqs)
        self.slots = StateSlots(max_seqs)
        self.requests: dict = {}
        self._lives = 0
        self.groups: list[CacheGroup] = []
        self._group_of_cache: dict[int, int] = {}
        self._state_specs: dict[int, StateSpec] = {}
        self.state_tensors: dict[int, torch.Tensor] = {}
        spec_of: dict[int, KVCacheSpec] = {}
        writers = set()
        for cache_id, writes, kv_spec, state_spec in requirements:
            if kv_spec is not None:
                if cache_id in spec_of and spec_of[cache_id] != kv_spec:
                    raise ValueError(f"layer calls sharing cache {cache_id} ask for different caches: "
                                     f"{spec_of[cache_id]} and {kv_spec}")
                spec_of[cache_id] = kv_spec
                if writes:
                    writers.add(cache_id)
            if state_spec is not None:
                if cache_id in self._state_specs and self._state_specs[cache_id] != state_spec:
                    raise ValueError(f"layer calls sharing state {cache_id} ask for different states")
                self._state_specs[cache_id] = state_spec
        for cache_id in spec_of:
            if cache_id not in writers:
                raise ValueError(f"cache {cache_id} is read but no layer call writes it")
        by_spec: dict[KVCacheSpec, CacheGroup] = {}
        for cache_id in sorted(spec_of):
            spec = spec_of[cache_id]
            g = by_spec.get(spec)
            if g is None:
                n = num_pages[spec] if isinstance(num_pages, dict) else num_pages
                g = CacheGroup(spec, self.page_size, BlockPool(int(n)))
                by_spec[spec] = g
                self.groups.append(g)
            g.cache_ids.append(cache_id)
            self._group_of_cache[cache_id] = self.groups.index(g)
        if device is not None:
            for g in self.groups:
                g.kv = torch.zeros(len(g.cache_ids), 2, g.pool.num_pages, g.spec.num_kv_heads,
                                   self.page_size, g.spec.head_dim, dtype=dtype, device=device)
            # one row more than there are requests: the row of the padding rows of a decode graph,
            # which no request ever holds (``padding_slot``)
            for cache_id, st in self._state_specs.items():
                self.state_tensors[cache_id] = torch.zeros(self.max_seqs + 1, *st.shape, dtype=st.dtype,
                                                           device=device)

    # ---- lookups ---------------------------------------------------------
    def group_index(self, cache_id: int) -> int | None:
        return self._group_of_cache.get(cache_id)

    def kv_tensors(self, cache_id: int):
        g = self.groups[self._group_of_cache[cache_id]]
        i = g.index_of(cache_id)
        k = g.kv[i, 0]
        pages, nkv, ps, d = k.shape
        return k, g.kv[i, 1].view(pages, nkv, d, ps)   # values are kept transposed

    def num_tokens(self, req) -> int:
        return self.requests[req].num_tokens

    def slot(self, req) -> int:
        return self.requests[req].slot

    @property
    def padding_slot(self) -> int:
        """The state slot of rows that stand for no request (the padding rows of a decode
        graph): a row of its own in every state tensor, so that a part that updates its state
        for every row of a step never touches a live request's."""
        return self.max_seqs

    def life(self, req) -> int:
        """A number that no other stay of any request in this cache has had.  Whoever keeps
        a copy of a request's block table keys it on this, never on the request's id alone:
        the id comes back with other pages after a preemption."""
        return self.requests[req].life

    def has_request(self, req) -> bool:
        return req in self.requests

    def block_table(self, group: int, req) -> list[int]:
        return self.groups[group].tables[req]

    # ---- life of a request ----------------------------------------------
    def add_request(self, req) -> int:
        if req in self.requests:
            raise ValueError(f"request {req!r} is already live")
        slot = self.slots.acquire()
        self._lives += 1
        self.requests[req] = RequestCacheState(slot, life=self._lives)
        for g in self.groups:
            g.tables[req] = []
        for t in self.state_tensors.values():
            t[slot].zero_()
        return slot

    def pages_needed(self, req, n_new: int) -> list[int]:
        """Pages each group must still take so that ``n_new`` more tokens fit."""
        st = self.requests[req]
        blocks = -(-(st.num_tokens + n_new) // self.page_size)
        return [max(0, blocks - len(g.tables[req])) for g in self.groups]

    def can_reserve(self, req, n_new: int, spare: list[int] | None = None) -> bool:
        need = self.pages_needed(req, n_new)
        free = spare if spare is not None else [g.pool.num_free for g in self.groups]
        return all(n <= f for n, f in zip(need, free))

    def reserve(self, req, n_new: int) -> None:
        """Takes the pages for ``n_new`` more tokens in every group, or none."""
        need = self.pages_needed(req, n_new)
        for n, g in zip(need, self.groups):
            if n > g.pool.num_free:
                raise OutOfPages(
                    f"request {req!r} needs {n} more pages for {n_new} tokens, "
                    f"{g.pool.num_free} of {g.pool.num_pages} free (group {g.spec})")
        for n, g in zip(need, self.groups):
            g.tables[req].extend(g.pool.allocate(n))

    def rollback(self, req, keep_new: int = 0) -> int:
        """Gives back the pages that ``reserve`` took beyond what ``keep_new`` more tokens need
        (none: a step that failed between ``reserve`` and ``commit``; some: a portion that was
        cut down after its pages were taken); returns how many."""
        st = self.requests[req]
        keep = -(-(st.num_tokens + keep_new) // self.page_size)
        n = 0
        for g in self.groups:
            table = g.tables[req]
            gone = [p for p in table[keep:] if p >= 0]
            if gone:
                g.pool.free(gone)
                n += len(gone)
            del table[keep:]
        return n

    def commit(self, req, n_new: int) -> None:
        """``n_new`` tokens have been written.  Gives back the pages of window
        groups that no later query can reach: a query at position p >= count
        reads keys j >= p - window + 1, so block b is dead once
        (b + 1) * page_size <= count - window + 1."""
        st = self.requests[req]
        st.num_tokens += n_new
        ps = self.page_size
        for g in self.groups:
            if st.num_tokens > len(g.tables[req]) * ps:
                raise RuntimeError(f"request {req!r} holds {st.num_tokens} tokens but pages for "
                                   f"{len(g.tables[req]) * ps}")
            w = g.spec.window
            if w > 0:
                dead = max(0, (st.num_tokens - w + 1) // ps)
                table = g.tables[req]
                gone = [table[b] for b in range(min(dead, len(table))) if table[b] >= 0]
                if gone:
                    g.pool.free(gone)
                    for b in range(min(dead, len(table))):
                        table[b] = -1

    def release(self, req) -> None:
        """The request ends (or is preempted): all its pages and its slot go back."""
        st = self.requests.pop(req)
        for g in self.groups:
            g.pool.free([p for p in g.tables.pop(req) if p >= 0])
        self.slots.release(st.slot)

    def slot_mapping(self, group: int, req, start: int, n: int) -> list[int]:
        """Flat slot (page * page_size + offset) of tokens start .. start+n-1."""
        table = self.groups[group].tables[req]
        ps = self.page_size
        out = []
        for j in range(start, start + n):
            page = table[j // ps]
            if page < 0:
                raise RuntimeError(f"request {req!r}: token {j} lies in a page already given back")
            out.append(page * ps + j % ps)
        return out

    def check(self) -> None:
        """Invariants: no page lost, none held twice, counts add up."""
        self.slots.check()
        for g in self.groups:
            g.pool.check()
            held = [p for t in g.tables.values() for p in t if p >= 0]
            assert len(held) == len(set(held)), "a page is held by two requests"
            assert len(held) == g.pool.num_used, "pages in tables and used count differ"
        assert set(self.requests) == set().union(*[set(g.tables) for g in self.groups]) or not self.groups
