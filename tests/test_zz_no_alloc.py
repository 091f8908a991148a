"""The decode attention entry point that allocates nothing
(tff_attention_decode_fused_static), called through ctypes as a caller without
torch would, against the entry points that take a workspace from the caller:
two calls in a row on the same GPU, the second with a smaller input (fewer
requests, fewer splits, shorter contexts), so that what the first call left in
the library's array must not show in the second; and the refusal of sizes
beyond the array."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

P, I, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float


def _library():
    from tffinfer_amd.kernels.build import ensure_built
    lib = ctypes.CDLL(ensure_built())
    lib.tff_last_error.restype = ctypes.c_char_p
    tail = [F, P, I, I, I, I, I, I, I, I, I, I, F, P]     # eps .. stream
    lib.tff_attention_decode_fused.argtypes = [P, I, P, P, P, P, P, P, I, P, P, P, P, P] + tail
    lib.tff_attention_decode_fused_static.argtypes = [P, I, P, P, P, P, I, P, P, P, P, P] + tail
    lib.tff_attention_split_reduce.argtypes = [P, P, P, I, I, I, I, P, I, P]
    for f in (lib.tff_attention_decode_fused, lib.tff_attention_decode_fused_static, lib.tff_attention_split_reduce):
        f.restype = I
    return lib


def _case(R, contexts, nq, nkv, d, page_size, seed):
    """A decode step of R requests with the given numbers of cached tokens: raw projections,
    norm weights, rotation table, a shuffled page pool filled with keys and values."""
    g = torch.Generator().manual_seed(seed)
    dev = "cuda:0"
    blocks = [-(-(c + 1) // page_size) for c in contexts]
    num_pages = sum(blocks) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    width = max(blocks)
    bt = torch.zeros(R, width, dtype=torch.int32)
    at = 0
    for r, nb in enumerate(blocks):
        bt[r, :nb] = torch.tensor(perm[at:at + nb], dtype=torch.int32)
        at += nb
    k_cache = (torch.randn(num_pages, nkv, page_size, d, generator=g) * 0.5).to(torch.bfloat16)
    v_cache = (torch.randn(num_pages, nkv, d, page_size, generator=g) * 0.5).to(torch.bfloat16)
    qkv = (torch.randn(R, (nq + 2 * nkv) * d, generator=g)).to(torch.bfloat16)
    max_pos = max(contexts) + 1
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * torch.exp(
        -(2.0 * torch.arange(d // 2, dtype=torch.float64) / d) * math.log(10000.0))[None, :]
    cos_sin = torch.stack([torch.cos(ang), torch.sin(ang)], -1).float().contiguous()
    slot = torch.tensor([int(bt[r, c // page_size]) * page_size + c % page_size for r, c in enumerate(contexts)],
                        dtype=torch.int32)
    t = dict(qkv=qkv, k=k_cache, v=v_cache, bt=bt, cu=torch.arange(R + 1, dtype=torch.int32),
             start=torch.tensor(contexts, dtype=torch.int32), slot=slot,
             qw=1 + 0.1 * torch.randn(d, generator=g), kw=1 + 0.1 * torch.randn(d, generator=g), cos_sin=cos_sin)
    t = {k: v.to(dev) for k, v in t.items()}
    t.update(R=R, nq=nq, nkv=nkv, d=d, page_size=page_size, num_pages=num_pages, max_pos=max_pos, width=width)
    return t


def _run(lib, t, splits, static):
    """Runs one of the two entry points on copies of the caches; returns (out, k cache, v cache)."""
    R, nq, nkv, d = t["R"], t["nq"], t["nkv"], t["d"]
    k, v = t["k"].clone(), t["v"].clone()
    out = torch.full((R, nq * d), float("nan"), dtype=torch.bfloat16, device="cuda:0")
    tail = (1e-6, t["cos_sin"].data_ptr(), t["max_pos"], 0, splits, R, nq, nkv, d, t["page_size"], t["num_pages"], 0,
            1.0 / math.sqrt(d), None)
    head = (t["bt"].data_ptr(), t["width"], t["cu"].data_ptr(), t["start"].data_ptr(), t["slot"].data_ptr(),
            t["qw"].data_ptr(), t["kw"].data_ptr())
    torch.cuda.synchronize()
    if static:
        rc = lib.tff_attention_decode_fused_static(t["qkv"].data_ptr(), t["qkv"].shape[1], out.data_ptr(),
                                                   k.data_ptr(), v.data_ptr(), *head, *tail)
        assert rc == 0, lib.tff_last_error().decode()
    else:
        part_o = torch.empty(splits, R, nq, d, dtype=torch.float32, device="cuda:0")
        part_ml = torch.empty(splits, R, nq, 2, dtype=torch.float32, device="cuda:0")
        rc = lib.tff_attention_decode_fused(t["qkv"].data_ptr(), t["qkv"].shape[1], out.data_ptr(), part_o.data_ptr(),
                                            part_ml.data_ptr(), k.data_ptr(), v.data_ptr(), *head, *tail)
        assert rc == 0, lib.tff_last_error().decode()
        if splits > 1:
            rc = lib.tff_attention_split_reduce(part_o.data_ptr(), part_ml.data_ptr(), out.data_ptr(), splits, R, nq,
                                                d, None, 0, None)
            assert rc == 0, lib.tff_last_error().decode()
    torch.cuda.synchronize()
    return out, k, v


def test_two_calls_in_a_row_the_second_smaller():
    lib = _library()
    big = _case(6, [700, 33, 1290, 5, 257, 999], nq=8, nkv=2, d=128, page_size=16, seed=1)
    small = _case(2, [40, 311], nq=8, nkv=2, d=128, page_size=16, seed=2)
    for t, splits in ((big, 7), (small, 3), (small, 1)):
        print(f"static decode attention: {t['R']} requests, {splits} splits", flush=True)
        want = _run(lib, t, splits, static=False)
        got = _run(lib, t, splits, static=True)
        assert not torch.isnan(got[0].float()).any()
        for a, b, what in zip(got, want, ("output", "key cache", "value cache")):
            assert torch.equal(a, b), f"{what} differs from the entry point with a caller's workspace"
        assert not torch.equal(got[1], t["k"])          # the step's keys did reach their pages


def test_sizes_beyond_the_array_are_refused():
    lib = _library()
    t = _case(2, [40, 311], nq=8, nkv=2, d=128, page_size=16, seed=3)
    # 256 splits x 600 entries x 8 heads x 130 floats = 639 MB of partial results
    rc = lib.tff_attention_decode_fused_static(
        t["qkv"].data_ptr(), t["qkv"].shape[1], t["qkv"].data_ptr(), t["k"].data_ptr(), t["v"].data_ptr(),
        t["bt"].data_ptr(), t["width"], t["cu"].data_ptr(), t["start"].data_ptr(), t["slot"].data_ptr(),
        t["qw"].data_ptr(), t["kw"].data_ptr(), 1e-6, t["cos_sin"].data_ptr(), t["max_pos"], 0, 256, 600, 8, 2, 128,
        16, t["num_pages"], 0, 0.1, None)
    assert rc != 0
    msg = lib.tff_last_error().decode()
    assert "bytes" in msg and "fewer splits" in msg
