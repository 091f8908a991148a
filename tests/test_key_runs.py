"""The runs of keys that the host deals for a decode step's attention: whatever the requests'
lengths, every visible key of every row lies in exactly one run, runs begin where the kernel's
steps of keys begin, a row's runs follow each other, their number stays within the tables, and no
run is much longer than the waves' fair share."""
import random

import numpy as np
import pytest

from tffinfer_amd.kernels.key_runs import (BLOCK_PAIRS, BUSY_WAVES, KEY_STEP, LONG_STEPS, MIN_STEPS, RESIDENT_WAVES,
                                          TARGET_WAVES, deal_key_runs, max_key_runs, wants_blocks)


def check_runs(runs, start, positions, window):
    runs, start = np.asarray(runs), np.asarray(start)
    R = len(positions)
    assert runs.ndim == 2 and runs.shape[1] == 4 and start.shape == (R + 1,)
    assert start[0] == 0 and np.all(np.diff(start) >= 1), "every row has a run"
    total = int(start[R])
    assert total <= runs.shape[0]
    assert np.all(runs[total:, 0] == -1), "runs beyond the last row's are marked unused"
    for r, P in enumerate(positions):
        P = int(P)
        lo = max(0, P - window + 1) if window > 0 else 0
        first = lo // KEY_STEP * KEY_STEP
        mine = runs[start[r]:start[r + 1]]
        assert np.all(mine[:, 0] == r) and np.all(mine[:, 3] == P)
        assert mine[0, 1] == first, f"row {r}: the first run begins at {mine[0, 1]}, the first step of keys at {first}"
        assert mine[-1, 2] == P + 1, f"row {r}: the last run ends at {mine[-1, 2]}, the new token is {P}"
        assert np.all((mine[:, 1] - first) % KEY_STEP == 0)
        assert np.all(mine[:, 2] > mine[:, 1]), "no empty run"
        assert np.all(mine[1:, 1] == mine[:-1, 2]), f"row {r}: a gap or an overlap between runs"
        lens = -(-(mine[:, 2] - mine[:, 1]) // KEY_STEP)
        assert np.all(lens[:-1] == lens[0]) and lens[-1] <= lens[0], f"row {r}: runs of {lens.tolist()} steps"


@pytest.mark.parametrize("window", [0, 1, 40, 1000])
@pytest.mark.parametrize("nkv", [1, 2, 8])
def test_every_key_in_exactly_one_run(window, nkv):
    rng = random.Random(17 * window + nkv)
    for trial in range(60):
        R = rng.choice([1, 2, 3, 8, 24, 64, 200])
        kind = rng.randrange(4)
        if kind == 0:
            pos = [rng.randrange(0, 40000) for _ in range(R)]
        elif kind == 1:
            pos = [rng.choice([0, 1, 30, 31, 32, 33, 63, 64, 127, 128]) for _ in range(R)]
        elif kind == 2:
            pos = [30000] + [rng.randrange(0, 600) for _ in range(R - 1)]
        else:
            pos = [2047] * R
        live = rng.choice([None, R, max(1, R - 3)])
        dealt = deal_key_runs(pos, window, nkv, live=live)
        assert dealt.runs.shape[0] == max_key_runs(R, nkv)
        check_runs(dealt.runs, dealt.run_start, pos, window)
        assert dealt.merge == (dealt.run_start[-1] > R)
        assert not (dealt.blocks and dealt.merge), "blocks of eight waves are for rows of one run each"
        assert dealt.run_start[-1] * nkv <= max(RESIDENT_WAVES, R * nkv), "more waves than the GPU holds at once"


def test_runs_are_of_similar_length():
    # one long request beside many short ones: the long one's runs are about as long as the
    # waves' fair share of all keys, not a fixed fraction of its own length
    pos = [32767] + [1023] * 63
    runs, start, blocks, merge = deal_key_runs(pos, 0, 8)
    steps = -(-(runs[:start[-1], 2] - runs[:start[-1], 1]) // KEY_STEP)
    fair = -(-sum((p // KEY_STEP + 1) for p in pos) * 8 // TARGET_WAVES)
    assert steps.max() <= 1.5 * fair, (steps.max(), fair)
    assert start[1] - start[0] >= 16, "the long request is many runs"
    assert np.all(np.diff(start)[1:] == 1), "a short request is one run"
    assert start[-1] * 8 <= RESIDENT_WAVES and merge and not blocks
    # few requests: runs no shorter than MIN_STEPS steps, and no shorter than LONG_STEPS while
    # BUSY_WAVES waves have work
    runs, start, _, _ = deal_key_runs([2047], 0, 8)
    assert start[1] == -(-64 // -(-64 // (64 // MIN_STEPS)))
    for P in (2047, 2099, 2111):
        runs, start, _, _ = deal_key_runs([P] * 8, 0, 8)
        n = start[1] - start[0]
        assert n == (P // KEY_STEP + 1) // LONG_STEPS and n * 8 * 8 >= BUSY_WAVES
    # a short request is one run whatever its neighbours
    runs, start, _, _ = deal_key_runs([5, 100000], 0, 8)
    assert start[1] == 1
    # requests of one length: the launch stays within the waves that the GPU holds at once
    assert deal_key_runs([2100] * 64, 0, 8).blocks
    for R, per_row in ((16, 6), (40, 3), (48, 2), (64, 1), (72, 1), (128, 1), (200, 1)):
        runs, start, blocks, merge = deal_key_runs([2100] * R, 0, 8, blocks=False)
        assert start[-1] == per_row * R, (R, start[-1])
        assert (per_row == 1 or start[-1] * 8 <= RESIDENT_WAVES) and merge == (per_row > 1)


def test_blocks_of_eight_waves_are_for_requests_of_about_one_length():
    rng = random.Random(5)
    for R in (20, 24, 32):
        assert wants_blocks(R, 8) and BLOCK_PAIRS[0][0] <= R * 8 <= BLOCK_PAIRS[0][1]
        # requests of one length, or of about one: a run each, the block's waves split it among them
        for pos in ([2100] * R, [2000 + 11 * i for i in range(R)], [2000 + (997 * i) % 1000 for i in range(R)]):
            runs, start, blocks, merge = deal_key_runs(pos, 0, 8)
            assert blocks and not merge and start[-1] == R
            check_runs(runs, start, pos, 0)
        # padding rows of a captured step do not count
        runs, start, blocks, merge = deal_key_runs([2100] * R + [0] * 4, 0, 8, live=R)
        assert blocks and not merge and start[-1] == R + 4
        # uneven lengths go to single waves, the long requests cut to the others' measure
        for pos in ([16383] * 3 + [1023] * (R - 3), [rng.choice([300, 300, 300, 4300]) for _ in range(R - 1)] + [4300]):
            runs, start, blocks, merge = deal_key_runs(pos, 0, 8)
            assert not blocks and merge and R < start[-1] <= RESIDENT_WAVES // 8
            check_runs(runs, start, pos, 0)
            lens = -(-(runs[:start[-1], 2] - runs[:start[-1], 1]) // KEY_STEP)
            steps = sorted(p // KEY_STEP + 1 for p in pos)
            fair = -(-sum(steps) * 8 // TARGET_WAVES)
            assert lens.max() <= 1.5 * max(fair, steps[R // 2]) + 1, "a run much longer than the fair share and the median request"
    assert not wants_blocks(19, 8) and not wants_blocks(33, 8) and wants_blocks(128, 2) and not wants_blocks(1, 8)
    # too few or too many requests: single waves whatever the lengths
    for R in (8, 19, 33, 48, 72):
        assert not deal_key_runs([2100] * R, 0, 8).blocks


def test_tables_too_small_are_refused():
    with pytest.raises(ValueError):
        deal_key_runs([5, 6], 0, 8, runs_out=np.zeros(8, dtype=np.int32), start_out=np.zeros(3, dtype=np.int32))
    with pytest.raises(ValueError):
        deal_key_runs([5, 6], 0, 8, runs_out=np.zeros(4 * max_key_runs(2, 8), dtype=np.int32), start_out=np.zeros(2, dtype=np.int32))


def test_no_rows():
    runs, start, blocks, merge = deal_key_runs([], 0, 8)
    assert start.tolist() == [0] and np.all(runs[:, 0] == -1) and not blocks and not merge
