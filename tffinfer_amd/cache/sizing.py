"""How many pages each group of layers gets.

A group that keeps every key needs pages for all the tokens the engine is to
hold.  A group with a window needs, per request, only the pages its window and
the step's new tokens touch, whatever the length of the request; giving it the
full pool would pay for the cache twice.  The reference has one geometry for
all layers and sizes its pool from the free device memory
(src/core/runtime/KVCache.h:267-281, src/core/runtime/InferRuntime.cu:123-136).
"""
from __future__ import annotations

import math

from ..parts.base import KVCacheSpec


def group_layers(requirements) -> dict[KVCacheSpec, int]:
    """Cache spec -> number of caches (layer calls that write one) of that spec, in the
    order the cache manager forms its groups."""
    spec_of = {}
    for cache_id, _writes, kv_spec, _state in requirements:
        if kv_spec is not None:
            spec_of[cache_id] = kv_spec
    out: dict[KVCacheSpec, int] = {}
    for cache_id in sorted(spec_of):
        out[spec_of[cache_id]] = out.get(spec_of[cache_id], 0) + 1
    return out


def state_bytes(requirements, max_seqs: int) -> int:
    """Device bytes of the per-request state tensors (one row more than there are requests)."""
    seen, total = set(), 0
    for cache_id, _writes, _kv, st in requirements:
        if st is not None and cache_id not in seen:
            seen.add(cache_id)
            total += (max_seqs + 1) * math.prod(st.shape) * st.dtype.itemsize
    return total


def min_window_pages(window: int, page_size: int) -> int:
    """Pages a request must be able to hold in a group with a window to advance by one token:
    the window's tokens, wherever the window's start falls in its page."""
    return -(-max(window - 1, 0) // page_size) + 1


def window_pool_pages(window: int, page_size: int, max_seqs: int, token_budget: int) -> int:
    """Pages with which a group with a window never runs short: a request that brings n tokens to
    a step touches the n + window - 1 tokens that end with them, at most ceil((n + window - 1) /
    page) + 1 pages, and a step's portions hold ``token_budget`` tokens between them."""
    return max_seqs * (-(-max(window - 1, 0) // page_size) + 2) + -(-token_budget // page_size)


def bytes_per_page(spec: KVCacheSpec, layers: int, page_size: int, elem_size: int) -> int:
    return 2 * layers * spec.num_kv_heads * spec.head_dim * page_size * elem_size


def plan_pages(requirements, page_size: int, elem_size: int, max_seqs: int, token_budget: int,
               tokens: int | None = None, kv_bytes: int | None = None,
               free_bytes: int | None = None) -> dict[KVCacheSpec, int]:
    """Pages per group.  ``tokens``: what the groups that keep every key shall hold (plus a page
    a request for the last, partly filled one); ``kv_bytes``: or the device bytes that all groups
    may take together; ``free_bytes``: a cap on those bytes (the state tensors come off it
    first).  Groups with a window get what :func:`window_pool_pages` says, never more than a
    group that keeps every key."""
    groups = group_layers(requirements)
    if not groups:
        return {}
    full = [s for s in groups if s.window <= 0]
    want_full = None if tokens is None else -(-tokens // page_size) + max_seqs
    pages = {}
    for s in groups:
        if s.window > 0:
            n = window_pool_pages(s.window, page_size, max_seqs, token_budget)
            pages[s] = n if want_full is None else min(n, want_full)
    budget = None
    if kv_bytes is not None:
        budget = int(kv_bytes)
    if free_bytes is not None:
        cap = max(0, int(free_bytes) - state_bytes(requirements, max_seqs))
        budget = cap if budget is None else min(budget, cap)

    def cost(spec, n):
        return n * bytes_per_page(spec, groups[spec], page_size, elem_size)

    if budget is None and want_full is None:
        raise ValueError("the cache needs a size: tokens, bytes or the free memory")
    if budget is not None:
        # the groups with a window first (they are small); if even they do not fit, they shrink alike
        win_cost = sum(cost(s, n) for s, n in pages.items())
        if win_cost > budget:
            pages = {s: int(n * budget / win_cost) for s, n in pages.items()}
            win_cost = sum(cost(s, n) for s, n in pages.items())
        per_full = sum(cost(s, 1) for s in full)
        fit = int((budget - win_cost) // per_full) if per_full else 0
        for s in full:
            pages[s] = fit if want_full is None else min(want_full, fit)
    else:
        for s in full:
            pages[s] = want_full
    bad = [s for s, n in pages.items() if n < 1]
    if bad:
        raise ValueError(f"the memory given to the cache holds no page of {page_size} tokens for {bad[0]}")
    return pages
