"""Runs of keys for a decode step's attention, dealt on the host.

An attention kernel that gives every (request, kv head) the same number of
waves is as slow as its longest request: sixty-three requests of a thousand
tokens beside one of thirty thousand wait for the waves of that one, five times
as long as the bytes of the step need.  The host knows every request's length
when it writes the step's tables, so it cuts each request's visible keys into
runs of about the same length and the kernel gives a wave to every (run, kv
head): a short request is one run, a long one many, and all waves end
together.  The tables are written anew for every step, captured or not; their
size depends only on the number of rows, so a captured launch serves any mix of
lengths.

How many runs: the kernel's waves fill a SIMD's registers alone, so the GPU
holds RESIDENT_WAVES of them at once, and a wave that streams alone is bound by
latency, not by bandwidth.  Measured on decode steps of 1 to 128 requests: some
TARGET_WAVES waves, none beyond what is resident, runs of LONG_STEPS steps and
more as long as BUSY_WAVES waves have work, never under MIN_STEPS; with so many
requests that the waves' fair share is most of a request, a run a request.

With as many pairs of request and kv head as BLOCK_PAIRS says (most of a round
of a block a CU, or of two), and requests of about one length (the longest no
more than some two times the average, see BLOCK_RATE_SHARE), a block of eight
waves per request and kv head, which merges its waves' results in LDS, is
faster than single waves whose results a second kernel merges: every request
is one run then, and ``blocks`` says so.  A CU holds one such block, and a
block is as slow as its request is long, so uneven lengths go to single waves.

Pure host code (numpy).  The reference has one sequence per forward and no such
table (src/core/runtime/InferRuntime.cu:415-429).
"""
from __future__ import annotations

from typing import NamedTuple

import numpy as np

#: keys a wave works through at a time: a run begins a multiple of this after its request's
#: first visible key rounded down to a multiple of it
KEY_STEP = 32
#: waves of one wave a block that the GPU holds at once (256 CUs, four SIMDs a CU, a wave a SIMD)
RESIDENT_WAVES = 1024
#: waves a launch aims at when single waves take the runs
TARGET_WAVES = 768
#: no run is shorter than this many steps of keys (a request that has fewer is one run) ...
MIN_STEPS = 4
#: ... nor shorter than this many while as many waves as BUSY_WAVES are left with work
LONG_STEPS = 8
BUSY_WAVES = 256
#: pairs of request and kv head between which requests of about one length get a block of eight
#: waves each (one round of a block a CU, or two full ones) ...
BLOCK_PAIRS = ((160, 256), (448, 512))
#: ... "about one length": a block's eight waves stream some 45 GB/s, all blocks together what HBM
#: gives (5 TB/s, 111 times as much), so the blocks are as fast as the bytes allow as long as the
#: longest request has no more than pairs / 111 times the average's keys (per round of blocks)
BLOCK_RATE_SHARE = 111
CUS = 256


class KeyRuns(NamedTuple):
    runs: np.ndarray         # int32 [max_key_runs, 4]: (row, first key, end of keys, the row's position); row -1: not in use
    run_start: np.ndarray    # int32 [rows + 1]: row r has the runs run_start[r] .. run_start[r + 1] - 1
    blocks: bool             # dealt for a block of eight waves per run
    merge: bool              # some row has several runs: partial results have to be merged


def wants_blocks(rows: int, waves_per_run: int) -> bool:
    """Whether ``rows`` requests, if they are of about one length, get a block of eight waves each."""
    pairs = int(rows) * max(1, int(waves_per_run))
    return any(lo <= pairs <= hi for lo, hi in BLOCK_PAIRS)


def max_key_runs(rows: int, waves_per_run: int) -> int:
    """Runs that :func:`deal_key_runs` makes at most for ``rows`` requests, whatever their lengths:
    the size of the tables.  A multiple of eight: the kernel's blocks go to the eight XCDs in turn,
    and run i is to be on XCD i % 8 with all its kv heads."""
    return (max(int(rows), RESIDENT_WAVES // max(1, int(waves_per_run))) + 7) & ~7


def deal_key_runs(positions, window: int, waves_per_run: int, runs_out: np.ndarray | None = None,
                  start_out: np.ndarray | None = None, blocks: bool | None = None,
                  target: int | None = None, min_steps: int | None = None, live: int | None = None) -> KeyRuns:
    """``positions`` [R]: the position of each request's one new token (as many tokens are cached
    before it); ``window`` > 0: a token sees only the last ``window`` keys, itself included;
    ``waves_per_run``: waves (or blocks) that the kernel starts per run: the kv heads.  ``blocks``:
    whether a run gets a block of eight waves (None: by the number of rows and their lengths).
    ``live``: the first so many rows are requests, the others padding (a captured step's), which
    does not count where the requests' number and lengths decide.  ``target`` and ``min_steps``
    override the number of waves (or blocks) aimed at and the shortest run (for tests).

    The runs of row r are ``run_start[r] .. run_start[r + 1] - 1``, in the order of their keys,
    without gap or overlap, from the row's first visible key rounded down to a multiple of
    KEY_STEP to its new token, all of one length but the last, which is no longer; runs beyond
    ``run_start[R]`` have row -1.  ``runs_out`` (flat, 4 ints a run) and ``start_out`` are
    written if given."""
    P = np.asarray(positions, dtype=np.int64)
    R = P.shape[0]
    wps = max(1, int(waves_per_run))
    cap = max_key_runs(R, wps)
    runs = np.empty(4 * cap, dtype=np.int32) if runs_out is None else runs_out
    start = np.empty(R + 1, dtype=np.int32) if start_out is None else start_out
    if runs.shape[0] < 4 * cap or start.shape[0] < R + 1:
        raise ValueError(f"tables of {runs.shape[0]} and {start.shape[0]} ints are too small for {R} rows "
                         f"({4 * cap} and {R + 1})")
    start[0] = 0
    if R == 0:
        runs[0:4 * cap:4] = -1
        return KeyRuns(runs[:4 * cap].reshape(-1, 4), start[:1], False, False)
    lo = np.maximum(0, P - window + 1) if window > 0 else np.zeros_like(P)
    first = lo // KEY_STEP * KEY_STEP
    steps = (P - first) // KEY_STEP + 1
    wave_steps = int(steps.sum()) * wps
    mine = steps if live is None else steps[:max(1, int(live))]
    if blocks is None:
        pairs = mine.shape[0] * wps
        spread = max(1.2, pairs / (BLOCK_RATE_SHARE * -(-pairs // CUS)))
        blocks = wants_blocks(mine.shape[0], wps) and int(mine.max()) * mine.shape[0] <= spread * int(mine.sum())
    if blocks:
        # a run a row, unless a test asks for more
        n = np.ones(R, dtype=np.int64)
        chunk = int(steps.max())
        if target is not None:
            chunk = max(1 if min_steps is None else int(min_steps), -(-wave_steps // int(target)))
            n = -(-steps // chunk)
    else:
        typical = int(np.median(mine))
        floor = max(MIN_STEPS, min(LONG_STEPS, -(-wave_steps // BUSY_WAVES))) if min_steps is None else int(min_steps)
        share = -(-wave_steps // max(1, TARGET_WAVES if target is None else int(target)))
        if target is None and share * 5 > typical * 3:
            # so many requests that the waves' fair share is most of a request: requests of about
            # one length stay a run each (nothing to merge then); a request much longer than the
            # others is cut to their measure
            chunk = max(share, -(-3 * typical // 2))
            n = -(-steps // chunk)
        elif share >= floor:
            chunk = share
            n = -(-steps // chunk)            # no run longer than the waves' fair share
        else:
            chunk = floor
            n = np.maximum(1, steps // chunk)  # no run shorter than the floor
    # within what the GPU holds at once (and the tables), where longer runs can make it so
    limit = min(RESIDENT_WAVES, cap * wps)
    while wps * int(n.sum()) > limit and int(n.max()) > 1:
        chunk += max(1, chunk // 4)
        n = -(-steps // chunk)
    # A row's runs are of one length but the last, which is the shorter for it: its wave (or block)
    # also rotates the new token's key and puts key and value into their page.
    per = -(-steps // n)
    n = -(-steps // per)
    np.cumsum(n, out=start[1:R + 1])
    total = int(start[R])
    row = np.repeat(np.arange(R), n)
    j = np.arange(total) - np.repeat(start[:R].astype(np.int64), n)
    kb = first[row] + KEY_STEP * j * per[row]
    runs[0:4 * total:4] = row
    runs[1:4 * total:4] = kb
    runs[2:4 * total:4] = np.minimum(P[row] + 1, kb + KEY_STEP * per[row])
    runs[3:4 * total:4] = P[row]
    runs[4 * total:4 * cap:4] = -1
    return KeyRuns(runs[:4 * cap].reshape(-1, 4), start[:R + 1], bool(blocks), total > R)
