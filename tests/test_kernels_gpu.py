"""Each kernel alone against a plain float64 computation of the same op, at
sizes other than the engine's."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _ops():
    from tffinfer_amd.kernels import ops
    return ops


def _w(w):
    """A weight as ops.linear takes it: row-major float32, fragment order bfloat16."""
    w = w.to(DEV)
    return _ops().pack_weight(w) if w.dtype == torch.bfloat16 else w


#: bfloat16 attention against float64 on the same bfloat16 inputs: the largest difference over the largest
#: value; about twice the worst seen over all the cases below (a run prints what it saw at its end)
ATTN_TOL = 1.1e-2


def _close(got, ref, tol, what=""):
    got, ref = got.double().cpu(), ref.double().cpu()
    err = float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))
    if tol == ATTN_TOL:
        from helpers import note_error
        note_error("kernels", "attention_bf16", err)
    assert err <= tol, f"{what}: rel. error {err:.3e} > {tol:.1e}"
    return err


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(0)
    table = torch.randn(77, 40, generator=g).to(dtype)
    ids = torch.tensor([0, 76, 5, 5, 33], dtype=torch.int32)
    out = ops.embed(table.to(DEV), ids.to(DEV))
    assert out.dtype == torch.float32
    assert torch.equal(out.cpu(), table.float()[ids.long()])


@pytest.mark.parametrize("H", [40, 96, 1000, 4096, 5120])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_add_rmsnorm(H, out_dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(H)
    n = 7
    resid = torch.randn(n, H, generator=g) * 3
    delta = torch.randn(n, H, generator=g)
    w = 1 + 0.1 * torch.randn(H, generator=g)
    eps = 1e-3
    v = (resid + delta).double()
    ref = v * torch.rsqrt((v * v).mean(-1, keepdim=True) + eps) * w.double()
    r = resid.to(DEV).clone()
    out = ops.add_rmsnorm(r, delta.to(DEV), w.to(DEV), eps, out_dtype)
    _close(out, ref, 1e-6 if out_dtype == torch.float32 else 8e-3, "norm")
    _close(r, v, 1e-6, "residual sum stored back")
    # gathered rows: residual untouched, norm of resid + delta of those rows
    rows = torch.tensor([5, 0, 5], dtype=torch.int32)
    r2 = resid.to(DEV).clone()
    out2 = ops.add_rmsnorm(r2, delta.to(DEV), w.to(DEV), eps, out_dtype, rows=rows.to(DEV))
    _close(out2, ref[rows.long()], 1e-6 if out_dtype == torch.float32 else 8e-3, "gathered norm")
    assert torch.equal(r2.cpu(), resid)
    # no delta
    out3 = ops.add_rmsnorm(r2, None, w.to(DEV), eps, out_dtype)
    v3 = resid.double()
    _close(out3, v3 * torch.rsqrt((v3 * v3).mean(-1, keepdim=True) + eps) * w.double(),
           1e-6 if out_dtype == torch.float32 else 8e-3, "norm without delta")


def test_rmsnorm_eps_position():
    """eps is added to the mean inside the root: a row of tiny values tells it
    from eps added to the sum or outside the root."""
    ops = _ops()
    H = 64
    x = torch.full((1, H), 1e-3)
    w = torch.ones(H)
    eps = 1e-5
    out = ops.add_rmsnorm(x.to(DEV).clone(), None, w.to(DEV), eps, torch.float32)
    want = 1e-3 / math.sqrt(1e-6 + eps)
    assert abs(float(out[0, 0]) - want) / want < 1e-5


@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (5, 320, 96), (33, 200, 200), (130, 130, 72), (257, 96, 256),
                                    (64, 4096, 512), (300, 1000, 1024), (50, 203, 1000), (40, 1024, 2056),
                                    (100, 203, 2048), (520, 264, 1544),
                                    # a little more groups of 16 columns than CUs: two groups a block (up to 16 rows)
                                    (5, 5000, 1096), (16, 4100, 264), (1, 6544, 520), (3, 6560, 512)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear(M, N, K, dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(M * 1000 + N)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.1).to(dtype)
    ref = x.double() @ w.double().T
    out = ops.linear(x.to(DEV), _w(w), out_dtype=torch.float32)
    _close(out, ref, 2e-6 if dtype == torch.float32 else 2e-5, f"linear {M}x{N}x{K} f32 out")
    if dtype == torch.bfloat16:
        out_b = ops.linear(x.to(DEV), _w(w))
        assert out_b.dtype == torch.bfloat16
        _close(out_b, ref, 6e-3, "linear bf16 out")
    # strided rows (a slice of a wider matrix)
    wide = torch.randn(M, K + 16, generator=g).to(dtype).to(DEV)
    out_s = ops.linear(wide[:, :K], _w(w), out_dtype=torch.float32)
    _close(out_s, wide[:, :K].double().cpu() @ w.double().T, 2e-6 if dtype == torch.float32 else 2e-5, "strided")


@pytest.mark.parametrize("M,N,K", [(16, 33000, 2560), (10, 40000, 4096), (3, 33000, 512)])
def test_linear_very_wide(M, N, K):
    """An output head's shape: thousands of groups of 16 columns; with many rows and a long K a block
    of the streaming kernel takes two groups (the last case: one)."""
    ops = _ops()
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) * 0.1).to(torch.bfloat16)
    ref = x.double() @ w.double().T
    out = ops.linear(x.to(DEV), _w(w), out_dtype=torch.float32)
    _close(out, ref, 2e-5, f"linear {M}x{N}x{K}")
    for m in range(M):
        _close(out[m], ref[m], 2e-5, f"row {m}")


@pytest.mark.parametrize("M,N,K", [(40, 1024, 2056), (520, 264, 1544), (8, 64, 64), (8, 5120, 8192), (16, 5120, 8200),
                                    (16, 5120, 17408), (12, 5120, 25600)])
def test_linear_partial_sums_feed_the_norm(M, N, K):
    """Where the product splits K over blocks it can hand out the partial sums; the fused
    residual sum and norm adds them up itself, in order, to what the whole product gives."""
    ops = _ops()
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) * 0.1).to(torch.bfloat16)
    pw = ops.pack_weight(w.to(DEV))
    whole = ops.linear(x, pw, out_dtype=torch.float32)
    parts = ops.linear(x, pw, out_dtype=torch.float32, partials=True)
    # 9 to 16 rows, 320 column groups and a long K: the whole product streams, the partial sums come
    # from tiles that split K; the two kernels add in different orders.  (Up to 8 rows, or with a
    # shorter K, the streaming kernel gives a block two column groups and runs both.)
    other_kernel = 8 < M <= 16 and N == 5120 and N * K >= 45e6
    same = (lambda a, b: torch.allclose(a.float(), b.float(), rtol=2e-2 if a.dtype == torch.bfloat16 else 1e-4,
                                        atol=2e-2 if a.dtype == torch.bfloat16 else 1e-3)) if other_kernel else torch.equal
    if M <= 16 and not other_kernel:
        assert isinstance(parts, ops.PendingProduct)   # a few rows: run by whoever consumes it
        assert torch.equal(parts.run(), whole)
    else:
        assert parts.dim() == 3 and parts.shape[0] > 1 and tuple(parts.shape[1:]) == (M, N)
        acc = parts[0].clone()
        for p in parts[1:]:
            acc += p
        assert same(acc, whole)
    resid = torch.randn(M, N, generator=g).to(DEV)
    nw = (1 + 0.1 * torch.randn(N, generator=g)).to(DEV)
    r1, r2 = resid.clone(), resid.clone()
    y1 = ops.add_rmsnorm(r1, whole, nw, 1e-6, torch.float32)
    y2 = ops.add_rmsnorm(r2, parts, nw, 1e-6, torch.float32)
    assert same(r1, r2) and same(y1, y2)
    rows = torch.tensor([M - 1, 0], dtype=torch.int32, device=DEV)
    z1 = ops.add_rmsnorm(resid.clone(), whole, nw, 1e-6, torch.bfloat16, rows=rows)
    z2 = ops.add_rmsnorm(resid.clone(), parts, nw, 1e-6, torch.bfloat16, rows=rows)
    assert same(z1, z2)


@pytest.mark.parametrize("glu", [False, True])
@pytest.mark.parametrize("M,H,K,N2", [(1, 64, 64, 96), (8, 4096, 4096, 6144), (5, 320, 96, 200), (16, 200, 1000, 72),
                                       (3, 1000, 256, 33000), (7, 4096, 12288, 24576), (16, 40, 8200, 136),
                                       (16, 5120, 512, 51200), (11, 5120, 256, 49138), (2, 5120, 256, 51200),
                                       # widths of a little more groups of 16 columns than CUs (two groups a block) and just past them
                                       # gated on tiles of 128 rows from fewer elements on where there are more rows
                                       (12, 5120, 256, 34816), (16, 4096, 128, 24576), (14, 4096, 128, 24576),
                                       (9, 4112, 1000, 64), (8, 6544, 8200, 40), (16, 6544, 520, 40), (4, 6560, 512, 48), (8, 5120, 17408, 96)])
def test_norm_taken_into_the_products_on_either_side(M, H, K, N2, glu):
    """Up to 16 rows: the product before a norm adds to the residual stream, writes (sum * norm
    weight) in bfloat16 and the sums of squares of its groups of 16 columns; the product after it
    multiplies by the row's factor.  Against the three steps done one after the other, in float64,
    with the norm's weights and a residual stream whose rows differ in size by orders of magnitude
    (a factor applied to the wrong row, or a norm left out, would show).  The last three cases, gated:
    a weight so large (or so many rows) that the product after the norm runs on tiles of 32 rows
    of the four-wave kernel, which takes the rows' factors into its epilogue too."""
    ops = _ops()
    g = torch.Generator().manual_seed(M * 7 + H)
    eps = 1e-5
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(H, K, generator=g) * 0.05).to(torch.bfloat16)
    resid = torch.randn(M, H, generator=g) * (10.0 ** torch.arange(M).remainder(4).float())[:, None]
    nw = 1 + 0.3 * torch.randn(H, generator=g)
    new_resid = resid.double() + x.double() @ w1.double().T
    normed = new_resid * torch.rsqrt((new_resid * new_resid).mean(-1, keepdim=True) + eps) * nw.double()
    if glu:
        I = N2 // 2
        gate = (torch.randn(I, H, generator=g) * 0.05).to(torch.bfloat16)
        up = (torch.randn(I, H, generator=g) * 0.05).to(torch.bfloat16)
        w2 = ops.pack_gate_up(gate.to(DEV), up.to(DEV))
        a, b = normed @ gate.double().T, normed @ up.double().T
        ref = a / (1 + torch.exp(-a)) * b
    else:
        w2d = (torch.randn(N2, H, generator=g) * 0.05).to(torch.bfloat16)
        w2 = ops.pack_weight(w2d.to(DEV))
        ref = normed @ w2d.double().T
    r = resid.to(DEV).clone()
    pending = ops.linear(x.to(DEV), ops.pack_weight(w1.to(DEV)), out_dtype=torch.float32, partials=True)
    assert isinstance(pending, ops.PendingProduct)
    rows = ops.add_rmsnorm(r, pending, nw.to(DEV), eps, torch.bfloat16, for_linear=True)
    assert isinstance(rows, ops.ScaledRows)
    _close(r, new_resid, 2e-5, "residual stream after the product")
    y = ops.linear(rows, w2, out_dtype=torch.float32)
    _close(y, ref, 1.2e-2, "product after the norm")
    for m in range(M):     # row by row: a row's factor is its own
        _close(y[m], ref[m], 1.5e-2, f"row {m}")
    # written out for a consumer that is no such product: rounded to bfloat16 once (2^-9 of an element)
    out = rows.materialize().double().cpu()
    assert float(((out - normed).abs() / normed.abs().clamp_min(1e-3)).max()) <= 2.0 ** -8
    # the same through the separate kernels, to rounding
    r2 = resid.to(DEV).clone()
    z = ops.add_rmsnorm(r2, pending.run(), nw.to(DEV), eps, torch.bfloat16)
    assert torch.allclose(r2, r, rtol=1e-6, atol=1e-6)
    y2 = ops.linear(z, w2, out_dtype=torch.float32)
    _close(y, y2.double().cpu(), 1.2e-2, "fused against separate kernels")
    # without for_linear (or with rows to gather) the norm gives a plain tensor
    r3 = resid.to(DEV).clone()
    z3 = ops.add_rmsnorm(r3, pending, nw.to(DEV), eps, torch.bfloat16)
    assert isinstance(z3, torch.Tensor) and torch.equal(z3, z) and torch.equal(r3, r2)


def _gemm_plan(M, N, K, glu=0, keep=0):
    import ctypes
    from tffinfer_amd.kernels import lib
    r, c, s = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    assert lib.load().tff_gemm_plan(M, N, K, glu, keep, ctypes.byref(r), ctypes.byref(c), ctypes.byref(s)) == 0
    return r.value, c.value, s.value


@pytest.mark.parametrize("M,N,K,glu", [(2000, 8100, 328, False), (1500, 8000, 1096, False), (2048, 4096, 12296, False),
                                         (2000, 16160, 328, True), (1024, 16000, 328, False),
                                         (2048, 6144, 520, False), (2000, 6100, 328, False)])
def test_linear_on_the_largest_tile(M, N, K, glu):
    """Shapes for which the plan takes the sixteen-wave 256 x 256 or 256 x 192 tiles (K no
    multiple of 64): an odd number of 32-k steps, a last step that is not whole, rows and columns
    that do not fill the tiles, K split over blocks with the partial sums added or handed on.  The
    float32 product of the same (bfloat16) numbers is the yardstick."""
    ops = _ops()
    g = torch.Generator().manual_seed(N)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    if glu:
        I = N // 2
        gate = (torch.randn(I, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
        up = (torch.randn(I, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
        assert _gemm_plan(M, 2 * I, K, 1)[:2] == (256, 256)
        y = ops.linear(x, ops.pack_gate_up(gate, up), out_dtype=torch.float32)
        a, b = ops.linear(x.float(), gate.float()), ops.linear(x.float(), up.float())
        ref = a / (1 + torch.exp(-a)) * b
        _close(y, ref, 3e-5, "gated product")
        return
    w = (torch.randn(N, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
    pw = ops.pack_weight(w)
    ref = ops.linear(x.float(), w.float())
    for keep in (0, 1):
        r, c, sp = _gemm_plan(M, N, K, 0, keep)
        if K < 12288 or keep:       # (the long K runs on this tile when its two halves are handed on)
            assert r == 256 and c in ((192,) if N in (6144, 6100) else (192, 256)), (r, c, sp)
        y = ops.linear(x, pw, out_dtype=torch.float32, partials=bool(keep))
        if keep and sp > 1:
            assert y.dim() == 3 and y.shape[0] == sp
        _close(ops.as_tensor(y), ref, 3e-5, f"product (keep={keep}, {sp} parts)")
    yb = ops.linear(x, pw)       # bfloat16 result
    _close(yb, ref, 8e-3, "bfloat16 result")


FOUR_WAVE_CASES = [
    # M, N, K, gated: K in units of 64, so tiles of 256 rows are the four-wave kernel's
    (2048, 6144, 256, False),      # 256 x 192, whole tiles
    (2000, 8100, 320, False),      # 256 x 256, ragged rows and columns, an odd number of units
    (2304, 2100, 64, False),       # 256 x 128, nine row tiles (a last group of one), a single unit of K
    (1999, 4100, 2048, False),     # 256 x 192, a last column tile of a few columns
    (2048, 4096, 1024, False),     # 256 x 128
    (1024, 4096, 12288, False),    # K split over blocks: added up, and handed on
    (700, 4096, 2048, False),      # three row tiles and K split, when the sums are handed on (smaller tiles otherwise)
    (3000, 12288, 64, False),      # twelve row tiles: a full group of eight and one of four
    (2048, 16384, 128, True),      # gated, 256 x 256
    (1100, 12288, 192, True),      # gated, ragged rows
    (1100, 12280, 192, True),      # gated, a result whose rows are no multiple of 16 bytes: element by element
    (2048, 12288, 1024, True),     # gated, 256 x 192: pairs of groups within a wave's six
]


@pytest.mark.parametrize("M,N,K,glu", FOUR_WAVE_CASES)
def test_linear_on_four_wave_tiles(M, N, K, glu):
    """The four-wave kernel (tiles of 256 rows, K in units of 64, A fetched as whole cache lines and
    read back through a swizzle): every tile width, gated or not, ragged edges, more than eight row
    tiles, a row stride beyond K, K split over blocks with the sums added or handed on."""
    ops = _ops()
    g = torch.Generator().manual_seed(N + K)
    wide = torch.randn(M, K + 72, generator=g).to(torch.bfloat16).to(DEV)
    x = wide[:, :K].contiguous()
    if glu:
        I = N // 2
        gate = (torch.randn(I, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
        up = (torch.randn(I, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
        assert _gemm_plan(M, 2 * I, K, 1)[0] == 256
        a, b = ops.linear(x.float(), gate.float()), ops.linear(x.float(), up.float())
        ref = a / (1 + torch.exp(-a)) * b
        pw = ops.pack_gate_up(gate, up)
        _close(ops.linear(x, pw, out_dtype=torch.float32), ref, 3e-5, "gated product")
        _close(ops.linear(wide[:, :K], pw), ref, 8e-3, "gated product, strided rows, bfloat16 result")
        return
    w = (torch.randn(N, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
    pw = ops.pack_weight(w)
    ref = ops.linear(x.float(), w.float())
    seen = set()
    for keep in (0, 1):
        r, c, sp = _gemm_plan(M, N, K, 0, keep)
        assert r == 256 or (M, keep) == (700, 0), (r, c, sp)
        seen.add(sp)
        y = ops.linear(x, pw, out_dtype=torch.float32, partials=bool(keep))
        if keep and sp > 1:
            assert y.dim() == 3 and y.shape[0] == sp
        _close(ops.as_tensor(y), ref, 3e-5, f"product (keep={keep}, {c} columns, {sp} parts)")
    if K >= 2048 and M <= 1024:
        assert max(seen) > 1, "a case meant to split K"
    _close(ops.linear(wide[:, :K], pw), ref, 8e-3, "strided rows, bfloat16 result")


def test_four_wave_cases_cover_every_tile_width():
    widths = {(_gemm_plan(M, N, K, int(glu))[1], glu) for M, N, K, glu in FOUR_WAVE_CASES}
    assert {(128, False), (192, False), (256, False), (192, True), (256, True)} <= widths, widths


ONE_BY_FOUR_CASES = [
    # M, N, K, gated: few rows and K in units of 64, so tiles of 128 rows on four waves side by side
    (100, 6150, 4096, False),      # 128 x 128, K split; rows of the result that are no multiple of 16 bytes
    (120, 24576, 4096, True),      # 128 x 128, gated
    (70, 51184, 1024, True),       # 128 x 256, gated, a last column tile of a few columns
    (70, 40000, 512, False),       # 128 x 256
    (36, 66752, 640, False),       # 128 x 384
    (102, 73088, 1216, True),      # 128 x 384, gated
    (100, 4096, 12288, False),     # 128 x 128, eight parts: added up, and handed on
    (300, 34816, 320, False),      # three row tiles of 128, the last one ragged
]


@pytest.mark.parametrize("M,N,K,glu", ONE_BY_FOUR_CASES)
def test_linear_on_tiles_of_128_rows(M, N, K, glu):
    """The four-wave kernel with its waves side by side (tiles of 128 rows: products of few rows, whose
    time is the weight's stream): every tile width, gated or not, ragged edges, a row stride beyond K,
    K split over blocks with the sums added or handed on."""
    ops = _ops()
    g = torch.Generator().manual_seed(N + K)
    wide = torch.randn(M, K + 72, generator=g).to(torch.bfloat16).to(DEV)
    x = wide[:, :K].contiguous()
    if glu:
        I = N // 2
        gate = (torch.randn(I, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
        up = (torch.randn(I, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
        assert _gemm_plan(M, 2 * I, K, 1)[0] == 128
        a, b = ops.linear(x.float(), gate.float()), ops.linear(x.float(), up.float())
        ref = a / (1 + torch.exp(-a)) * b
        pw = ops.pack_gate_up(gate, up)
        _close(ops.linear(x, pw, out_dtype=torch.float32), ref, 3e-5, "gated product")
        _close(ops.linear(wide[:, :K], pw), ref, 8e-3, "gated product, strided rows, bfloat16 result")
        return
    w = (torch.randn(N, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
    pw = ops.pack_weight(w)
    ref = ops.linear(x.float(), w.float())
    for keep in (0, 1):
        r, c, sp = _gemm_plan(M, N, K, 0, keep)
        assert r == 128, (r, c, sp)
        y = ops.linear(x, pw, out_dtype=torch.float32, partials=bool(keep))
        if keep and sp > 1:
            assert y.dim() == 3 and y.shape[0] == sp
        _close(ops.as_tensor(y), ref, 3e-5, f"product (keep={keep}, {c} columns, {sp} parts)")
        if K >= 4096:
            assert sp > 1, "a case meant to split K"
    _close(ops.linear(wide[:, :K], pw), ref, 8e-3, "strided rows, bfloat16 result")


def test_cases_of_128_rows_cover_every_tile_width():
    widths = {(_gemm_plan(M, N, K, int(glu))[1], glu) for M, N, K, glu in ONE_BY_FOUR_CASES}
    assert {(128, False), (256, False), (384, False), (128, True), (256, True), (384, True)} <= widths, widths


FEW_ROWS_CASES = [
    # M, N, K, gated: 17 to 64 rows and K in units of 64, so tiles of 64 or 32 rows on four waves side by side
    (40, 6150, 4096, False),       # 64 x 128, K split; handed on: 64 x 256; rows of the result that are no multiple of 16 bytes
    (20, 24576, 4096, True),       # 32 x 128, gated
    (64, 40000, 512, False),       # 64 x 256, every row of the tile
    (17, 34816, 5120, True),       # 32 x 256, gated
    (50, 34816, 320, True),        # 64 x 256, gated, an odd number of units of K
    (33, 4096, 12288, False),      # 64 x 128, eight parts: added up, and handed on
    (30, 5120, 5120, False),       # 32 x 128, four parts
    (24, 10240, 5120, False),      # 32 x 256, four parts
    (60, 24560, 192, True),        # 64 x 128, gated, a result whose rows are no multiple of 16 bytes
    (18, 300, 64, False),          # 32 x 128, a single unit of K, a last column tile of a few columns
    (32, 8200, 128, False),        # 32 x 128, every row of the tile
    (16, 51200, 5120, True),       # up to 16 rows, gated, a weight so large that the rows go on tiles, not the streaming kernel
    (3, 49152, 5120, True),
    (14, 24576, 4096, True),       # (a smaller weight goes there with more rows)
]


@pytest.mark.parametrize("M,N,K,glu", FEW_ROWS_CASES)
def test_linear_on_tiles_of_64_and_32_rows(M, N, K, glu):
    """The four-wave kernel with its waves side by side and four or two row groups a wave (17 to 64
    rows: a decode step of so many requests): both heights and widths, gated or not, ragged edges, a
    row stride beyond K, K split over blocks with the sums added or handed on."""
    ops = _ops()
    g = torch.Generator().manual_seed(N + K)
    wide = torch.randn(M, K + 72, generator=g).to(torch.bfloat16).to(DEV)
    x = wide[:, :K].contiguous()
    if glu:
        I = N // 2
        gate = (torch.randn(I, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
        up = (torch.randn(I, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
        assert _gemm_plan(M, 2 * I, K, 1)[0] == (32 if M <= 32 else 64)
        a, b = ops.linear(x.float(), gate.float()), ops.linear(x.float(), up.float())
        ref = a / (1 + torch.exp(-a)) * b
        pw = ops.pack_gate_up(gate, up)
        _close(ops.linear(x, pw, out_dtype=torch.float32), ref, 3e-5, "gated product")
        _close(ops.linear(wide[:, :K], pw), ref, 8e-3, "gated product, strided rows, bfloat16 result")
        return
    w = (torch.randn(N, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
    pw = ops.pack_weight(w)
    ref = ops.linear(x.float(), w.float())
    for keep in (0, 1):
        r, c, sp = _gemm_plan(M, N, K, 0, keep)
        assert r in (32, 64) and r >= min(M, 33), (r, c, sp)
        y = ops.linear(x, pw, out_dtype=torch.float32, partials=bool(keep))
        if keep and sp > 1:
            assert y.dim() == 3 and y.shape[0] == sp
        _close(ops.as_tensor(y), ref, 3e-5, f"product (keep={keep}, {r} x {c}, {sp} parts)")
        if K >= 4096:
            assert sp > 1, "a case meant to split K"
    _close(ops.linear(wide[:, :K], pw), ref, 8e-3, "strided rows, bfloat16 result")


def test_cases_of_few_rows_cover_every_tile():
    tiles = {(_gemm_plan(M, N, K, int(glu))[:2], glu) for M, N, K, glu in FEW_ROWS_CASES}
    assert {((r, c), glu) for r in (32, 64) for c in (128, 256) for glu in (False, True)} <= tiles, tiles


@pytest.mark.parametrize("M,N,K", [(2600, 6144, 264), (4500, 520, 200), (1100, 300, 96), (9000, 130, 64),
                                   (2304, 2100, 72)])
def test_linear_with_many_row_tiles(M, N, K):
    """More than eight row tiles: the blocks walk them in groups of eight, the last group
    smaller.  Every tile is computed exactly once."""
    ops = _ops()
    g = torch.Generator().manual_seed(M)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
    y = ops.linear(x, ops.pack_weight(w), out_dtype=torch.float32)
    _close(y, ops.linear(x.float(), w.float()), 3e-5, "product")


def test_gemm_plan():
    """The plan of the tiled product: large tiles where they fill the machine, smaller ones or K
    split over blocks where they would not; never more parts than K has tiles for."""
    import ctypes
    from tffinfer_amd.kernels import lib
    L = lib.load()

    def plan(M, N, K, glu=0, keep=0):
        r, c, s = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        assert L.tff_gemm_plan(M, N, K, glu, keep, ctypes.byref(r), ctypes.byref(c), ctypes.byref(s)) == 0
        return r.value, c.value, s.value

    assert plan(8, 4096, 4096) == (0, 0, 1)
    # 9 to 16 rows, 320 column groups (two rounds for 64 CUs, one for the rest), partial sums wanted
    # anyway and a weight large enough: tiles that split K instead of the streaming kernel; up to 8
    # rows, or with a weight that is not so large, the streaming kernel with two column groups a block
    assert plan(12, 5120, 17408, keep=1)[0] in (32, 64, 128) and plan(12, 5120, 17408, keep=1)[2] > 1
    assert plan(8, 5120, 17408, keep=1) == (0, 0, 1) and plan(16, 5120, 8192, keep=1) == (0, 0, 1)
    assert plan(8, 5120, 8192) == (0, 0, 1) and plan(8, 5120, 5120, keep=1) == (0, 0, 1)
    assert plan(8, 4096, 12288, keep=1) == (0, 0, 1)
    assert plan(64, 4096, 12288) == (64, 128, 8)
    assert plan(64, 151936, 4096)[0] in (64, 128) and plan(64, 151936, 4096)[2] == 1
    assert plan(32, 24576, 4096, 1) == (32, 128, 1) and plan(64, 34816, 5120, 1) == (64, 256, 1)   # up to 64 rows: tiles of so many
    assert plan(65, 24576, 4096, 1)[0] == 128 and plan(33, 24576, 4096, 1)[0] == 64
    assert plan(128, 24576, 4096, 1) == (128, 128, 1)    # few rows: tiles of 128 rows, as many blocks as the columns give
    assert plan(32, 51200, 5120, 1)[:2] == (32, 256)
    assert plan(2048, 24576, 4096, 1)[0] == 256 and plan(2048, 24576, 4096, 1)[2] == 1
    assert plan(2048, 24584, 4104, 1) == (256, 256, 1)  # K no multiple of 64: the sixteen-wave tiles, gated on 256 columns only
    assert plan(4096, 4096, 4096) == (256, 256, 1)
    assert plan(2048, 6144, 4096) == (256, 192, 1)     # 8 x 32 tiles are one block a CU; 8 x 24 leave a quarter idle
    assert plan(2048, 4096, 4096) == (256, 128, 1)     # 8 x 32 again, where 192 columns would leave a third of the CUs idle
    r, c, s = plan(1024, 4096, 12288)
    assert r >= 128 and s >= 2                        # few tiles, long K: split
    r, c, s = plan(256, 4096, 4096)
    assert r <= 128 and s >= 2
    for M, N, K in ((100, 203, 2048), (520, 264, 1544), (300, 1000, 64), (2000, 64, 8)):
        r, c, s = plan(M, N, K)
        assert r in (64, 128, 256) and c in (128, 192, 256, 384) and 1 <= s <= 8 and (s == 1 or (K + 63) // 64 // s >= 4)
        assert L.tff_gemm_workspace_bytes(M, N, K, 1, 0, 0) == (s * M * N * 4 if s > 1 else 0)
    assert plan(2048, 4096, 12288, keep=1)[2] >= plan(2048, 4096, 12288)[2]   # kept sums cost less


def test_linear_identity_and_layout():
    """[out, in] layout: a non-square weight picks input columns."""
    ops = _ops()
    x = torch.arange(24, dtype=torch.float32).reshape(3, 8)
    w = torch.zeros(2, 8)
    w[0, 3] = 1.0
    w[1, 7] = 2.0
    out = ops.linear(x.to(DEV), w.to(DEV)).cpu()
    assert torch.equal(out[:, 0], x[:, 3]) and torch.equal(out[:, 1], 2 * x[:, 7])


def test_linear_refuses_bad_inner_size():
    from tffinfer_amd.kernels.lib import KernelError
    ops = _ops()
    x = torch.zeros(4, 12, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(8, 12, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(KernelError, match="multiple of 8"):
        ops.pack_weight(w)
    with pytest.raises(KernelError, match="PackedWeight"):
        ops.linear(torch.zeros(4, 16, dtype=torch.bfloat16, device=DEV),
                   torch.zeros(8, 16, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize("N,K", [(16, 32), (5, 8), (320, 96), (200, 200), (33, 1000)])
def test_pack_weight_round_trip_and_embedding(N, K):
    """Fragment order: element (n, k) at ((n/16) * KB + k/32) * 512 + ((k%32)/8 * 16 + n%16) * 8 + k%8."""
    ops = _ops()
    w = torch.randn(N, K, generator=torch.Generator().manual_seed(N * 1000 + K)).to(torch.bfloat16)
    pw = ops.pack_weight(w.to(DEV))
    assert pw.shape == (N, K)
    assert torch.equal(pw.unpack().cpu(), w)
    flat = pw.data.cpu()
    KB = -(-K // 32)
    for n, k in ((0, 0), (N - 1, K - 1), (N // 2, K // 3), (min(N - 1, 17), min(K - 1, 41))):
        off = ((n // 16) * KB + k // 32) * 512 + (((k % 32) // 8) * 16 + n % 16) * 8 + k % 8
        assert flat[off] == w[n, k]
    assert float(flat.double().abs().sum()) == float(w.double().abs().sum())   # the padding is zero (sums exact in float64)
    ids = torch.tensor([0, N - 1, N // 2], dtype=torch.int32)
    out = ops.embed(pw, ids.to(DEV))
    assert torch.equal(out.cpu(), w.float()[ids.long()])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("I", [200, 64, 1023])
def test_swiglu(dtype, I):
    ops = _ops()
    g = torch.Generator().manual_seed(I)
    gu = (torch.randn(5, 2 * I, generator=g) * 3).to(dtype)
    gt, up = gu[:, :I].double(), gu[:, I:].double()
    ref = gt / (1 + torch.exp(-gt)) * up
    out = ops.swiglu(gu.to(DEV))
    _close(out, ref, 1e-6 if dtype == torch.float32 else 8e-3, "swiglu")
    # roles: zero up gives zero, zero gate gives zero; silu(x) -> x for large x
    z = torch.zeros(1, 2 * I, dtype=dtype)
    z[:, :I] = 30.0
    z[:, I:] = 1.0
    assert torch.allclose(ops.swiglu(z.to(DEV)).float().cpu(), torch.full((1, I), 30.0), rtol=1e-2)


def _paged_setup(T_ctx, nkv, d, ps, dtype, seed, extra_pages=3):
    """A cache whose pages are deliberately out of order."""
    g = torch.Generator().manual_seed(seed)
    nblk = -(-T_ctx // ps)
    num_pages = nblk + extra_pages
    perm = torch.randperm(num_pages, generator=g)[:nblk]
    k = torch.randn(T_ctx, nkv, d, generator=g).to(dtype)
    v = torch.randn(T_ctx, nkv, d, generator=g).to(dtype)
    kc = torch.zeros(num_pages, nkv, ps, d, dtype=dtype)
    vc = torch.zeros(num_pages, nkv, d, ps, dtype=dtype)     # values are kept transposed
    for j in range(T_ctx):
        kc[perm[j // ps], :, j % ps] = k[j]
        vc[perm[j // ps], :, :, j % ps] = v[j]
    return k, v, kc, vc, perm.to(torch.int32)


def _attn_ref(q, k, v, positions, window, scale):
    T, nq, d = q.shape
    G = nq // k.shape[1]
    out = torch.zeros(T, nq, d, dtype=torch.float64)
    for t in range(T):
        p = int(positions[t])
        lo = 0 if window <= 0 else max(0, p - window + 1)
        for h in range(nq):
            s = (k[lo:p + 1, h // G].double() @ q[t, h].double()) * scale
            w = torch.softmax(s, 0)
            out[t, h] = w @ v[lo:p + 1, h // G].double()
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,d,ps,window", [(4, 2, 16, 16, 0), (6, 3, 48, 8, 0), (8, 2, 32, 8, 24),
                                                (5, 5, 80, 32, 0), (16, 2, 128, 16, 100), (3, 1, 256, 64, 0)])
def test_attention_generic(dtype, nq, nkv, d, ps, window):
    ops = _ops()
    ctx = 150
    k, v, kc, vc, table = _paged_setup(ctx, nkv, d, ps, dtype, seed=nq * d)
    g = torch.Generator().manual_seed(1)
    # queries at scattered positions of one request, including the first and the last
    positions = torch.tensor([0, 1, ps - 1, ps, 63, 64, 65, 100, ctx - 1], dtype=torch.int32)
    T = positions.numel()
    q = torch.randn(T, nq, d, generator=g).to(dtype)
    scale = 1 / math.sqrt(d)
    ref = _attn_ref(q, k, v, positions, window, scale)
    out = ops.attention_generic(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kc.to(DEV), vc.to(DEV),
                                table[None].contiguous().to(DEV), torch.zeros(T, dtype=torch.int32, device=DEV),
                                positions.to(DEV), window, scale)
    _close(out.reshape(T, nq, d), ref, 2e-6 if dtype == torch.float32 else 1e-2, "attention")


def test_attention_far_key_stands_out():
    """One key among hundreds is made to dominate: the output must be its value."""
    ops = _ops()
    nq, nkv, d, ps, ctx = 4, 2, 32, 16, 700
    k, v, kc, vc, table = _paged_setup(ctx, nkv, d, ps, torch.float32, seed=5)
    far = 3
    q = torch.randn(1, nq, d)
    q[0, 1] = q[0, 0]   # the two heads of a group share a query, so one key can serve both
    q[0, 3] = q[0, 2]
    for gidx, h in ((0, 0), (1, 2)):
        kc[table[far // ps], gidx, far % ps] = 200 * q[0, h] / q[0, h].norm()
    out = ops.attention_generic(q.reshape(1, nq * d).to(DEV), nq, nkv, d, kc.to(DEV), vc.to(DEV),
                                table[None].contiguous().to(DEV), torch.zeros(1, dtype=torch.int32, device=DEV),
                                torch.tensor([ctx - 1], dtype=torch.int32, device=DEV), 0, 1 / math.sqrt(d))
    out = out.reshape(nq, d).cpu()
    for h in range(nq):
        assert torch.allclose(out[h], v[far, h // 2], atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pairing", ["half", "interleaved"])
@pytest.mark.parametrize("T", [9, 139])
@pytest.mark.parametrize("nq,nkv,d,rot", [(4, 2, 16, 16), (3, 1, 48, 48), (8, 2, 128, 128), (2, 2, 64, 32),
                                           (5, 1, 32, 32), (3, 2, 256, 256), (9, 3, 64, 64)])
def test_qk_norm_rope_kv(dtype, pairing, nq, nkv, d, rot, T):
    """T = 75 takes the path for prompt portions (16-byte accesses, values written by runs of
    8 tokens): runs of slots that are aligned, that are not, single slots and a token without."""
    ops = _ops()
    from tffinfer_amd.parts.position import RotaryEmbedding
    ps, eps, theta = 8, 1e-5, 5000.0
    g = torch.Generator().manual_seed(d)
    qkv = torch.randn(T, (nq + 2 * nkv) * d, generator=g).to(dtype)
    qw = 1 + 0.1 * torch.randn(d, generator=g)
    kw = 1 + 0.1 * torch.randn(d, generator=g)
    if T == 9:
        num_pages = 6
        positions = torch.tensor([0, 1, 2, 17, 18, 40, 41, 42, 99], dtype=torch.int32)
        slots = torch.tensor([3, 47, 8, 9, 10, -1, 0, 1, 2], dtype=torch.int32)
    else:
        num_pages = 40
        positions = torch.cat([torch.arange(5, 45), torch.tensor([0]), torch.arange(100, 120),
                               torch.tensor([7, 99, 3, 64, 65, 66, 67, 68, 69, 70, 71, 2, 1, 127]),
                               torch.arange(30, 94)]).to(torch.int32)
        slots = torch.cat([torch.arange(16, 56), torch.tensor([-1]), torch.arange(59, 79),
                           torch.tensor([0, 9, 150, 96, 97, 98, 99, 100, 101, 102, 103, 159, 5, 88]),
                           torch.arange(200, 264)]).to(torch.int32)
        assert len(positions) == T and len(slots) == T
    rope = RotaryEmbedding(d, theta, pairing, rotary_dim=rot)
    table = rope.table(128, DEV)
    kc = torch.zeros(num_pages, nkv, ps, d, dtype=dtype, device=DEV)
    vc = torch.zeros(num_pages, nkv, d, ps, dtype=dtype, device=DEV)
    dq = qkv.to(DEV).clone()
    ops.qk_norm_rope_kv(dq, nq, nkv, d, qw.to(DEV), kw.to(DEV), eps, table, 1 if pairing == "interleaved" else 0,
                        positions.to(DEV), slots.to(DEV), kc, vc)
    x = qkv.double()
    q = x[:, :nq * d].reshape(T, nq, d)
    k = x[:, nq * d:(nq + nkv) * d].reshape(T, nkv, d)
    v = x[:, (nq + nkv) * d:].reshape(T, nkv, d)

    def norm(a, w):
        return a * torch.rsqrt((a * a).mean(-1, keepdim=True) + eps) * w.double()

    def rotate(a):
        ang = positions.double()[:, None] * torch.exp(-(2.0 * torch.arange(rot // 2).double() / rot) * math.log(theta))
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        out = a.clone()
        if pairing == "half":
            lo, hi = a[..., :rot // 2], a[..., rot // 2:rot]
            out[..., :rot // 2] = lo * c - hi * s
            out[..., rot // 2:rot] = lo * s + hi * c
        else:
            ev, od = a[..., 0:rot:2], a[..., 1:rot:2]
            out[..., 0:rot:2] = ev * c - od * s
            out[..., 1:rot:2] = ev * s + od * c
        return out

    tol = 2e-6 if dtype == torch.float32 else 8e-3
    qr, kr = rotate(norm(q, qw)), rotate(norm(k, kw))
    _close(dq[:, :nq * d].reshape(T, nq, d), qr, tol, "q")
    kc_h, vc_h = kc.cpu(), vc.cpu()
    written = set()
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        written.add(s)
        _close(kc_h[s // ps, :, s % ps], kr[t], tol, f"k of token {t}")
        _close(vc_h[s // ps, :, :, s % ps], v[t], tol if dtype == torch.bfloat16 else 0.0, f"v of token {t}")
    for s in range(num_pages * ps):
        if s not in written:
            assert float(kc_h[s // ps, :, s % ps].abs().max()) == 0.0, f"slot {s} was written"
            assert float(vc_h[s // ps, :, :, s % ps].abs().max()) == 0.0, f"value slot {s} was written"


def test_argmax_first_maximum():
    ops = _ops()
    x = torch.randn(6, 5000)
    x[0, 77] = x[0, 4000] = 100.0
    x[1, 4999] = 50.0
    x[2, 0] = 50.0
    out = ops.argmax(x.to(DEV)).cpu()
    assert out[0] == 77 and out[1] == 4999 and out[2] == 0
    assert torch.equal(out[3:].long(), x[3:].argmax(-1))
    # few rows of a large vocabulary: a row cut into runs over several blocks, then the first of their maxima
    V = 151937
    y = torch.randn(5, V)
    y[0, 100] = y[0, 100000] = 50.0          # equal maxima in different runs: the first one
    y[1, V - 1] = 50.0                       # the last element of the last run
    y[2, 4748] = y[2, 4749] = 50.0           # at a run's edge
    y[3] = float("nan")                      # nothing compares: index 0
    got = ops.argmax(y.to(DEV)).cpu()
    assert got.tolist()[:4] == [100, V - 1, 4748, 0] and got[4] == y[4].argmax()
    one = ops.argmax(y[4:5, 1:40000].contiguous().to(DEV)).cpu()     # rows off 16 bytes
    assert one[0] == y[4, 1:40000].argmax()


@pytest.mark.parametrize("V", [320, 5000, 151936, 600001])
def test_sample_distribution_and_draw(V):
    from plain_qwen3 import plain_inverse_cdf, plain_probs
    ops = _ops()
    g = torch.Generator().manual_seed(V)
    R = 6
    logits = torch.randn(R, V, generator=g) * 3
    temp = torch.tensor([0.8, 1.0, 0.5, 1.3, 0.0, 0.7])
    top_k = torch.tensor([0, 50, 0, 10, 5, 0], dtype=torch.int32)
    top_p = torch.tensor([1.0, 1.0, 0.9, 0.8, 0.5, 1.0])
    min_p = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.0, 0.05])
    u = torch.tensor([0.3, 0.999, 0.0, 0.5, 0.7, 0.42])
    tok, probs = ops.sample(logits.to(DEV), temp.to(DEV), u.to(DEV), top_k.to(DEV), top_p.to(DEV),
                            min_p.to(DEV), return_probs=True)
    tok, probs = tok.cpu(), probs.cpu()
    for r in range(R):
        if temp[r] == 0:
            assert tok[r] == logits[r].argmax()
            continue
        ref = plain_probs(logits[r], float(temp[r]), int(top_k[r]), float(top_p[r]), float(min_p[r]))
        assert int((ref > 0).sum()) == int((probs[r] > 0).sum()), f"row {r}: kept sets differ"
        assert float((probs[r].double() - ref).abs().max()) < 1e-6
        assert tok[r] == plain_inverse_cdf(ref, float(u[r]))


def test_sample_ties_rows_off_alignment_and_batch_position():
    """More equal logits at a threshold than the kernel keeps in LDS (it then goes through the row
    again for the lower bits); ties at the top-k and top-p thresholds are all kept, as in the plain
    implementation; rows of an odd vocabulary start off 16 bytes; a row's token does not depend on
    where in the batch the row stands."""
    from plain_qwen3 import plain_inverse_cdf, plain_probs
    ops = _ops()
    g = torch.Generator().manual_seed(5)
    V = 20001
    base = torch.randn(V, generator=g) * 2
    tied = torch.randperm(V, generator=g)[:6000]
    rows, params = [], []
    for k, p in ((100, 1.0), (0, 0.6), (7000, 0.9)):
        x = base.clone()
        x[tied] = 1.5 if k else 3.5      # some 3,200 other logits above 1.5: the 100th largest is not a tie, the 7000th is
        rows.append(x)
        params.append((0.9, k, p, 0.0))
    for V2 in (1, 3, 5, 67):
        x = torch.full((V,), float("-inf"))
        x[:V2] = torch.randn(V2, generator=g)
        rows.append(x)
        params.append((1.0, 0, 1.0, 0.0))
    logits = torch.stack(rows)
    R = len(rows)
    temp = torch.tensor([q[0] for q in params])
    top_k = torch.tensor([q[1] for q in params], dtype=torch.int32)
    top_p = torch.tensor([q[2] for q in params])
    min_p = torch.tensor([q[3] for q in params])
    u = torch.linspace(0.05, 0.95, R)
    tok, probs = ops.sample(logits.to(DEV), temp.to(DEV), u.to(DEV), top_k.to(DEV), top_p.to(DEV), min_p.to(DEV),
                            return_probs=True)
    tok, probs = tok.cpu(), probs.cpu()
    for r in range(R):
        ref = plain_probs(logits[r], *params[r])
        assert int((ref > 0).sum()) == int((probs[r] > 0).sum()), f"row {r}: kept sets differ"
        assert float((probs[r].double() - ref).abs().max()) < 1e-6
        assert tok[r] == plain_inverse_cdf(ref, float(u[r])), f"row {r}"
    assert int((probs[2] > 0).sum()) > 7000          # the ties at the 7000th were kept
    # the same rows in another order, and alone
    order = [3, 0, 6, 2, 5, 1, 4]
    again = ops.sample(logits[order].to(DEV), temp[order].to(DEV), u[order].to(DEV), top_k[order].to(DEV),
                       top_p[order].to(DEV), min_p[order].to(DEV)).cpu()
    assert torch.equal(again, tok[order])
    for r in (0, 2):
        alone = ops.sample(logits[r:r + 1].to(DEV), temp[r:r + 1].to(DEV), u[r:r + 1].to(DEV), top_k[r:r + 1].to(DEV),
                           top_p[r:r + 1].to(DEV), min_p[r:r + 1].to(DEV)).cpu()
        assert alone[0] == tok[r]


def test_sample_refuses_a_vocabulary_beyond_its_layout():
    ops = _ops()
    from tffinfer_amd.kernels.lib import KernelError
    V = (1 << 20) + 1
    with pytest.raises(KernelError, match="vocabulary"):
        ops.sample(torch.zeros(1, V, device=DEV), torch.ones(1, device=DEV), torch.zeros(1, device=DEV))


def test_repetition_penalty():
    from plain_qwen3 import plain_repetition_penalty
    ops = _ops()
    logits = torch.randn(2, 100)
    seen = [[3, 7, 50], [99, 0]]
    flat = torch.tensor(seen[0] + seen[1], dtype=torch.int32)
    cu = torch.tensor([0, 3, 5], dtype=torch.int32)
    pen = torch.tensor([1.3, 2.0])
    d = logits.to(DEV).clone()
    ops.repetition_penalty(d, flat.to(DEV), cu.to(DEV), pen.to(DEV))
    for r in range(2):
        assert torch.allclose(d[r].cpu(), plain_repetition_penalty(logits[r], seen[r], float(pen[r])))


def _fake_step(entries, ps, nkv, d, dtype, seed, extra_pages=2):
    """entries: (cached tokens P, new tokens n) per request.  Builds per-request
    keys/values, a shuffled page pool holding all of them, block tables and the
    step's flat tables, as the engine's batch builder would."""
    from types import SimpleNamespace
    g = torch.Generator().manual_seed(seed)
    R = len(entries)
    blocks = [-(-(P + n) // ps) for P, n in entries]
    num_pages = sum(blocks) + extra_pages
    perm = torch.randperm(num_pages, generator=g).tolist()
    kc = torch.zeros(num_pages, nkv, ps, d, dtype=dtype)
    vc = torch.zeros(num_pages, nkv, d, ps, dtype=dtype)
    width = max(blocks)
    bt = torch.zeros(R, width, dtype=torch.int32)
    ks, vs = [], []
    for r, (P, n) in enumerate(entries):
        k = torch.randn(P + n, nkv, d, generator=g).to(dtype)
        v = torch.randn(P + n, nkv, d, generator=g).to(dtype)
        ks.append(k)
        vs.append(v)
        for b in range(blocks[r]):
            bt[r, b] = perm.pop()
        for j in range(P + n):
            kc[bt[r, j // ps], :, j % ps] = k[j]
            vc[bt[r, j // ps], :, :, j % ps] = v[j]
    cu = [0]
    for P, n in entries:
        cu.append(cu[-1] + n)
    T = cu[-1]
    positions = torch.tensor([P + i for P, n in entries for i in range(n)], dtype=torch.int32)
    token_req = torch.tensor([r for r, (P, n) in enumerate(entries) for _ in range(n)], dtype=torch.int32)
    batch = SimpleNamespace(
        num_reqs=R, num_tokens=T, max_new_tokens=max(n for _, n in entries),
        max_context=max(P + n for P, n in entries), host_cu_tokens=cu,
        host_start_pos=[P for P, _ in entries],
        cu_tokens=torch.tensor(cu, dtype=torch.int32, device=DEV),
        start_pos=torch.tensor([P for P, _ in entries], dtype=torch.int32, device=DEV),
        positions=positions.to(DEV), token_req=token_req.to(DEV))
    kv = SimpleNamespace(k_cache=kc.to(DEV), v_cache=vc.to(DEV), block_tables=bt.to(DEV))
    return batch, kv, ks, vs, positions, token_req


@pytest.mark.parametrize("nq,nkv,d,ps,window", [
    (4, 2, 16, 16, 0), (8, 2, 32, 8, 24), (6, 3, 48, 8, 0), (32, 8, 128, 16, 0), (5, 5, 80, 32, 0),
    (12, 2, 64, 16, 40), (3, 1, 256, 64, 0), (40, 2, 96, 8, 0), (7, 7, 112, 16, 5), (4, 1, 192, 8, 0)])
def test_attention_mfma_prompt_portions_and_mixed(nq, nkv, d, ps, window):
    ops = _ops()
    # whole prompts, portions after a cached prefix (ending off page edges), single tokens
    entries = [(0, 37), (50, 13), (129, 1), (0, 1), (63, 2), (7, 70)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=nq + d)
    T = batch.num_tokens
    g = torch.Generator().manual_seed(2)
    q = torch.randn(T, nq, d, generator=g).to(torch.bfloat16)
    scale = 1 / math.sqrt(d)
    ref = torch.zeros(T, nq, d, dtype=torch.float64)
    for r in range(len(entries)):
        sel = (token_req == r).nonzero().flatten()
        ref[sel] = _attn_ref(q[sel], ks[r], vs[r], positions[sel], window, scale)
    # a wider row, as the fused projection output has
    wide = torch.zeros(T, nq * d + 2 * nkv * d, dtype=torch.bfloat16)
    wide[:, :nq * d] = q.reshape(T, nq * d)
    out = ops.attention_mfma(wide.to(DEV), nq, nkv, d, kv, batch, window, scale)
    _close(out.reshape(T, nq, d), ref, ATTN_TOL, "mfma attention")
    gen = ops.attention_generic(wide.to(DEV), nq, nkv, d, kv.k_cache, kv.v_cache, kv.block_tables,
                                batch.token_req, batch.positions, window, scale)
    _close(gen.reshape(T, nq, d), ref, ATTN_TOL, "generic attention on the same step")


@pytest.mark.parametrize("bins,groups", [(None, None), (3, 2), (1, 2), (None, 1), (3, 1), (1, 1)])
@pytest.mark.parametrize("nq,nkv,d,ps,window", [
    (32, 8, 128, 16, 0), (8, 2, 32, 8, 300), (6, 3, 48, 8, 0), (5, 1, 128, 32, 0), (40, 2, 96, 8, 77),
    (4, 2, 16, 16, 0), (3, 1, 256, 64, 0)])
def test_attention_mfma_long_portions(nq, nkv, d, ps, window, bins, groups):
    """Portions long enough for the kernel whose blocks share keys through LDS:
    several blocks per request, a cached prefix, windows that start mid-page."""
    ops = _ops()
    entries = [(0, 700), (333, 200), (5, 1), (1000, 130)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=nq * 7 + d)
    T = batch.num_tokens
    g = torch.Generator().manual_seed(4)
    q = torch.randn(T, nq, d, generator=g).to(torch.bfloat16)
    scale = 1 / math.sqrt(d)
    # bins: with fewer blocks than runs of 128 columns a block works through several runs in turn
    # groups: a block of two groups of waves that take every other slice, or of one
    out = ops.attention_mfma(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kv, batch, window, scale, block_bins=bins,
                             key_groups=groups)
    # the general kernel is the yardstick here (it is checked against float64 above)
    gen = ops.attention_generic(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kv.k_cache, kv.v_cache, kv.block_tables,
                                batch.token_req, batch.positions, window, scale)
    _close(out, gen.double(), ATTN_TOL, "block attention against the general kernel")
    sel = torch.tensor([0, 1, 31, 32, 127, 128, 699, 700, 899, 900, 901, T - 1])
    for r in range(len(entries)):
        mine = sel[(token_req[sel] == r)]
        if len(mine):
            ref = _attn_ref(q[mine], ks[r], vs[r], positions[mine], window, scale)
            _close(out.reshape(T, nq, d)[mine], ref, ATTN_TOL, f"block attention, request {r}")


@pytest.mark.parametrize("bins", [None, 3, 1])
@pytest.mark.parametrize("nq,nkv,d,ps,window", [
    (32, 8, 128, 16, 0), (8, 2, 32, 8, 300), (6, 3, 48, 8, 0), (5, 1, 128, 32, 0), (40, 2, 96, 8, 77),
    (4, 2, 16, 16, 0), (7, 7, 112, 16, 130)])
def test_attention_mfma_blocks_of_256_columns(nq, nkv, d, ps, window, bins):
    """The blocks for long prompts, whose waves take two column tiles each, forced here on
    portions of a few hundred tokens: requests whose columns end inside a wave's first or
    second tile, a cached prefix, windows, one query head to a key head and twenty."""
    ops = _ops()
    entries = [(0, 700), (333, 200), (5, 1), (1000, 130), (64, 37)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=nq * 5 + d)
    T = batch.num_tokens
    g = torch.Generator().manual_seed(14)
    q = torch.randn(T, nq, d, generator=g).to(torch.bfloat16)
    scale = 1 / math.sqrt(d)
    out = ops.attention_mfma(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kv, batch, window, scale, block_bins=bins,
                             block_cols=256)
    gen = ops.attention_generic(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kv.k_cache, kv.v_cache, kv.block_tables,
                                batch.token_req, batch.positions, window, scale)
    _close(out, gen.double(), ATTN_TOL, "blocks of 256 columns against the general kernel")
    sel = torch.tensor([0, 1, 31, 32, 63, 64, 127, 128, 699, 700, 899, 900, 901, 1030, 1031, T - 1])
    for r in range(len(entries)):
        mine = sel[(token_req[sel] == r)]
        if len(mine):
            ref = _attn_ref(q[mine], ks[r], vs[r], positions[mine], window, scale)
            _close(out.reshape(T, nq, d)[mine], ref, ATTN_TOL, f"blocks of 256 columns, request {r}")


def test_attention_mfma_picks_its_blocks_by_the_work():
    """A prompt of 2,048 tokens goes to the blocks of 128 columns, one of 32,768 tokens to those
    of 256; head sizes beyond 128 never do.  A prompt of 6,000 tokens through either gives
    what the general kernel gives."""
    from types import SimpleNamespace
    ops = _ops()
    nq, nkv, d, ps = 32, 8, 128, 16
    G = nq // nkv
    for T, want in ((2048, 128), (6000, 128), (32768, 256)):
        b = SimpleNamespace(host_cu_tokens=[0, T], host_start_pos=[0])
        assert ops._pick_block_cols(b, G, nkv, 0, DEV, "all", 128) == want
        assert ops._pick_block_cols(SimpleNamespace(host_cu_tokens=[0, T], host_start_pos=[0]), G, nkv, 0, DEV, "all", 256) == 128
    entries = [(0, 6000)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=3)
    T = batch.num_tokens
    q = torch.randn(T, nq, d, generator=torch.Generator().manual_seed(15)).to(torch.bfloat16)
    gen = ops.attention_generic(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kv.k_cache, kv.v_cache, kv.block_tables,
                                batch.token_req, batch.positions, 0, 1 / math.sqrt(d))
    for cols in (None, 256):
        out = ops.attention_mfma(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kv, batch, 0, 1 / math.sqrt(d), block_cols=cols)
        _close(out, gen.double(), ATTN_TOL, f"a long prompt against the general kernel (blocks: {cols})")
    assert ("blocks", G, nkv, 256, 0, _ops()._num_cus(DEV) // nkv, "all", 1, d, None) in batch._attn_work


@pytest.mark.parametrize("nq,nkv,d,ps,window,splits", [
    (32, 8, 128, 16, 0, None), (32, 8, 128, 16, 0, 1), (32, 8, 128, 16, 0, 7), (4, 2, 16, 16, 0, 3),
    (8, 2, 32, 8, 24, 4), (40, 2, 96, 8, 0, 5), (6, 3, 48, 8, 100, None), (16, 1, 64, 32, 0, 64),
    (4, 2, 192, 16, 0, 3), (2, 1, 256, 8, 0, None)])
def test_attention_mfma_decode_split_keys(nq, nkv, d, ps, window, splits):
    ops = _ops()
    entries = [(0, 1), (1, 1), (31, 1), (32, 1), (700, 1), (255, 1), (64, 1)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=d + ps)
    T = batch.num_tokens
    g = torch.Generator().manual_seed(3)
    q = torch.randn(T, nq, d, generator=g).to(torch.bfloat16)
    scale = 1 / math.sqrt(d)
    ref = torch.stack([_attn_ref(q[r:r + 1], ks[r], vs[r], positions[r:r + 1], window, scale)[0]
                       for r in range(T)])
    out = ops.attention_mfma(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kv, batch, window, scale, splits=splits)
    _close(out.reshape(T, nq, d), ref, ATTN_TOL, "split-key decode attention")
    if splits is None:
        # with the keys dealt into runs by the step's tables, as the engine brings them
        from tffinfer_amd.kernels.key_runs import deal_key_runs
        for target in (None, 40):
            dealt = deal_key_runs([P for P, _ in entries], window, nkv, blocks=False, target=target, min_steps=1 if target else None)
            kv.key_runs, kv.run_start = torch.from_numpy(dealt.runs.copy()).to(DEV), torch.from_numpy(dealt.run_start.copy()).to(DEV)
            kv.runs_window, kv.runs_merge, kv.runs_for_blocks = window, dealt.merge, False
            assert dealt.merge or target is None
            out = ops.attention_mfma(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kv, batch, window, scale)
            _close(out.reshape(T, nq, d), ref, ATTN_TOL, "decode attention over runs of keys, q finished")


@pytest.mark.parametrize("with_norm,with_rope", [(True, True), (False, True), (True, False)])
@pytest.mark.parametrize("nq,nkv,d,ps,window,splits,pairing", [
    (32, 8, 128, 16, 0, None, "half"), (32, 8, 128, 16, 0, 1, "interleaved"), (4, 2, 16, 16, 0, 3, "interleaved"),
    (8, 2, 32, 8, 24, 4, "interleaved"), (40, 2, 96, 8, 0, 5, "interleaved"), (6, 3, 48, 8, 100, None, "interleaved"),
    (16, 1, 64, 32, 0, 64, "half"), (4, 2, 192, 16, 0, 3, "half"), (2, 1, 256, 8, 0, None, "half"),
    # splits 0: a block of eight waves per entry and kv head, merged in LDS
    (32, 8, 128, 16, 0, 0, "half"), (4, 2, 16, 16, 0, 0, "interleaved"), (8, 2, 32, 8, 24, 0, "interleaved"),
    (40, 2, 96, 8, 0, 0, "interleaved"), (6, 3, 48, 8, 100, 0, "interleaved"), (16, 1, 112, 32, 0, 0, "interleaved"),
    # the entries' keys dealt into runs by the host, for so many waves
    (32, 8, 128, 16, 0, "runs 768", "half"), (4, 2, 16, 16, 0, "runs 64", "interleaved"),
    (8, 2, 32, 8, 24, "runs 100", "interleaved"), (40, 2, 96, 8, 0, "runs 30", "interleaved"),
    (6, 3, 48, 8, 100, "runs 1000", "interleaved"), (4, 2, 192, 16, 0, "runs 16", "half"), (2, 1, 256, 8, 0, "runs 5", "half")])
def test_attention_decode_fused(nq, nkv, d, ps, window, splits, pairing, with_norm, with_rope):
    """Decode steps from the raw projection output: q/k norm, rotation, the token's key and value
    into its page and attention in one kernel, against each part's formula; the slot of the new
    token holds large numbers beforehand, which must not reach the result; nothing else in the
    cache changes.  One entry has a negative slot (a padding row of a captured step, a call that
    reads another call's cache): nothing of it is written and its key and value come from its
    page.  Without a slot mapping the cache is read only."""
    ops = _ops()
    from tffinfer_amd.parts.position import RotaryEmbedding
    eps, theta = 1e-5, 5000.0
    entries = [(0, 1), (1, 1), (31, 1), (32, 1), (700, 1), (255, 1), (64, 1), (7, 1), (8, 1)]
    unwritten = 2
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=d + ps)
    R = batch.num_tokens
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(R, (nq + 2 * nkv) * d, generator=g).to(torch.bfloat16)
    qw = (1 + 0.1 * torch.randn(d, generator=g)) if with_norm else None
    kw = (1 + 0.1 * torch.randn(d, generator=g)) if with_norm else None
    table = RotaryEmbedding(d, theta, pairing).table(1024, DEV) if with_rope else None
    pr = 1 if pairing == "interleaved" else 0
    x = qkv.double()

    def norm(a, w):
        return a if w is None else a * torch.rsqrt((a * a).mean(-1, keepdim=True) + eps) * w.double()

    def rotate(a):
        if not with_rope:
            return a
        ang = positions.double()[:, None] * torch.exp(-(2.0 * torch.arange(d // 2).double() / d) * math.log(theta))
        c, sn = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        out = a.clone()
        if pairing == "half":
            lo, hi = a[..., :d // 2], a[..., d // 2:]
            out[..., :d // 2] = lo * c - hi * sn
            out[..., d // 2:] = lo * sn + hi * c
        else:
            ev, od = a[..., 0::2], a[..., 1::2]
            out[..., 0::2] = ev * c - od * sn
            out[..., 1::2] = ev * sn + od * c
        return out

    q = rotate(norm(x[:, :nq * d].reshape(R, nq, d), qw)).to(torch.bfloat16)
    k_new = rotate(norm(x[:, nq * d:(nq + nkv) * d].reshape(R, nkv, d), kw)).to(torch.bfloat16)
    v_new = qkv[:, (nq + nkv) * d:].reshape(R, nkv, d)
    scale = 1 / math.sqrt(d)
    refs = []
    for r, (P, _) in enumerate(entries):
        if r == unwritten:          # its key and value are the page's
            k, v = ks[r][:P + 1], vs[r][:P + 1]
        else:
            k = torch.cat([ks[r][:P], k_new[r:r + 1]])
            v = torch.cat([vs[r][:P], v_new[r:r + 1]])
        refs.append(_attn_ref(q[r:r + 1], k, v, positions[r:r + 1], window, scale)[0])
    ref = torch.stack(refs)
    # the slots of the new tokens hold numbers that would wreck the result if they were read
    bt = kv.block_tables.cpu()
    kc0, vc0 = kv.k_cache.cpu().clone(), kv.v_cache.cpu().clone()
    slots = []
    for r, (P, _) in enumerate(entries):
        if r == unwritten:
            slots.append(-1)
            continue
        kc0[bt[r, P // ps], :, P % ps] = 300.0
        vc0[bt[r, P // ps], :, :, P % ps] = -300.0
        slots.append(int(bt[r, P // ps]) * ps + P % ps)
    slots = torch.tensor(slots, dtype=torch.int32, device=DEV)
    kv.k_cache, kv.v_cache = kc0.to(DEV), vc0.to(DEV)
    w = (None if qw is None else qw.to(DEV), None if kw is None else kw.to(DEV))
    assert ops.decode_fused_supported(qkv.to(DEV), d, ps, table, pr, batch)
    how = dict(splits=splits)
    if isinstance(splits, str):
        from tffinfer_amd.kernels.key_runs import deal_key_runs
        runs, run_start, _, merge = deal_key_runs([P for P, _ in entries], window, nkv, target=int(splits.split()[1]), min_steps=1,
                                                  blocks=False)
        assert merge and run_start[-1] > R, "no entry has several runs"
        how = dict(key_runs=torch.from_numpy(runs.copy()).to(DEV), run_start=torch.from_numpy(run_start.copy()).to(DEV))
        splits = None
    out = ops.attention_decode_fused(qkv.to(DEV), nq, nkv, d, w[0], w[1], eps, table, pr, kv, batch, window, scale,
                                     slot_mapping=slots, **how)
    _close(out.reshape(R, nq, d), ref, ATTN_TOL, "fused decode attention")
    kc1, vc1 = kv.k_cache.cpu(), kv.v_cache.cpu()
    expect_k, expect_v = kc0.clone(), vc0.clone()
    for r, (P, _) in enumerate(entries):
        if r == unwritten:
            continue
        _close(kc1[bt[r, P // ps], :, P % ps], k_new[r].double(), 8e-3, f"key of entry {r} in its page")
        assert torch.equal(vc1[bt[r, P // ps], :, :, P % ps], v_new[r]), f"value of entry {r} in its page"
        expect_k[bt[r, P // ps], :, P % ps] = kc1[bt[r, P // ps], :, P % ps]
        expect_v[bt[r, P // ps], :, :, P % ps] = vc1[bt[r, P // ps], :, :, P % ps]
    assert torch.equal(kc1, expect_k) and torch.equal(vc1, expect_v), "a slot of another token was written"
    # a call that only reads: the pages hold the tokens already
    out2 = ops.attention_decode_fused(qkv.to(DEV), nq, nkv, d, w[0], w[1], eps, table, pr, kv, batch, window, scale,
                                      slot_mapping=None, **how)
    assert torch.equal(kv.k_cache.cpu(), kc1) and torch.equal(kv.v_cache.cpu(), vc1)
    _close(out2.reshape(R, nq, d), ref, ATTN_TOL, "fused decode attention, cache read only")
    # the two-kernel path gives the same to rounding
    kv.k_cache, kv.v_cache = kc0.to(DEV), vc0.to(DEV)
    dq = qkv.to(DEV).clone()
    ops.qk_norm_rope_kv(dq, nq, nkv, d, w[0], w[1], eps, table, pr, batch.positions, slots, kv.k_cache, kv.v_cache)
    out3 = ops.attention_mfma(dq, nq, nkv, d, kv, batch, window, scale, splits=splits or None)
    _close(out.reshape(R, nq, d), out3.reshape(R, nq, d).double().cpu(), ATTN_TOL, "fused against two kernels")


@pytest.mark.parametrize("d,ps,window", [(32, 8, 0), (128, 16, 0), (64, 8, 5000)])
def test_attention_decode_fused_blocks_of_eight_waves_over_long_contexts(d, ps, window):
    """A block of eight waves per entry and kv head: runs of keys of very different lengths in one
    launch (a wave with more pages than it keeps at hand works through them in segments; short
    entries leave most waves of their block without keys), one key far back made to dominate, the
    token's own key and value from registers.  What the block picks by itself from the step's sizes
    is the same kernel."""
    ops = _ops()
    nq, nkv = 8, 2
    far = 77
    entries = [(20000, 1), (40, 1), (0, 1), (95, 1), (96, 1), (3000, 1), (255, 1), (256, 1)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=3 + d)
    R = len(entries)
    g = torch.Generator().manual_seed(7)
    qkv = torch.randn(R, (nq + 2 * nkv) * d, generator=g).to(torch.bfloat16)
    q = qkv[:, :nq * d].reshape(R, nq, d)
    k_new = qkv[:, nq * d:(nq + nkv) * d].reshape(R, nkv, d)
    v_new = qkv[:, (nq + nkv) * d:].reshape(R, nkv, d)
    if window == 0:
        kfar = (30 * q[0, 0].float() / q[0, 0].float().norm()).to(torch.bfloat16)
        kv.k_cache[int(kv.block_tables[0, far // ps]), 0, far % ps] = kfar.to(DEV)
        ks[0][far, 0] = kfar
    scale = 1 / math.sqrt(d)
    bt = kv.block_tables.cpu()
    slots = torch.tensor([int(bt[r, P // ps]) * ps + P % ps for r, (P, _) in enumerate(entries)], dtype=torch.int32, device=DEV)
    refs = []
    for r, (P, _) in enumerate(entries):
        k = torch.cat([ks[r][:P], k_new[r:r + 1]])
        v = torch.cat([vs[r][:P], v_new[r:r + 1]])
        refs.append(_attn_ref(q[r:r + 1], k, v, positions[r:r + 1], window, scale)[0])
    ref = torch.stack(refs)
    out = ops.attention_decode_fused(qkv.to(DEV), nq, nkv, d, None, None, 1e-6, None, 0, kv, batch, window, scale,
                                     slot_mapping=slots, splits=0)
    _close(out.reshape(R, nq, d), ref, ATTN_TOL, "blocks of eight waves")
    if window == 0:
        assert torch.allclose(out.reshape(R, nq, d)[0, 0].float().cpu(), vs[0][far, 0].float(), atol=5e-2)
    # with so many pairs of entry and kv head, that is what a step gets unasked
    assert 128 * nkv >= ops.BLOCK_DECODE_MIN_PAIRS
    big = [(100 + 7 * i, 1) for i in range(128)]
    batch2, kv2, ks2, vs2, pos2, _ = _fake_step(big, ps, nkv, d, torch.bfloat16, seed=11)
    qkv2 = torch.randn(128, (nq + 2 * nkv) * d, generator=g).to(torch.bfloat16)
    bt2 = kv2.block_tables.cpu()
    slots2 = torch.tensor([int(bt2[r, P // ps]) * ps + P % ps for r, (P, _) in enumerate(big)], dtype=torch.int32, device=DEV)
    a = ops.attention_decode_fused(qkv2.to(DEV), nq, nkv, d, None, None, 1e-6, None, 0, kv2, batch2, window, scale,
                                   slot_mapping=slots2)
    b = ops.attention_decode_fused(qkv2.to(DEV), nq, nkv, d, None, None, 1e-6, None, 0, kv2, batch2, window, scale,
                                   slot_mapping=None, splits=0)
    assert torch.equal(a, b)


@pytest.mark.parametrize("nq,nkv,d,ps,window,waves,blocks", [
    (8, 2, 32, 8, 0, 768, False), (8, 2, 128, 16, 0, 64, False), (16, 2, 64, 8, 5000, 200, False), (34, 2, 64, 16, 0, 96, False),
    (4, 4, 256, 32, 0, 768, False), (8, 8, 128, 128, 700, 768, False),
    # a block of eight waves per run and kv head
    (8, 2, 32, 8, 0, 64, True), (8, 2, 128, 16, 0, 40, True), (16, 2, 64, 8, 5000, 96, True), (8, 8, 112, 128, 700, 256, True)])
def test_attention_decode_fused_keys_dealt_into_runs(nq, nkv, d, ps, window, waves, blocks):
    """Entries of very different lengths with their keys dealt into runs by the host, as the engine
    deals them (the long entry is many runs, most others one, which write their result themselves;
    a wave with more pages than it keeps at hand works through them in segments; a kv head with
    more than sixteen query heads has several column tiles; a wave per run, or a block of eight
    that split the run among them), one key far back made to dominate,
    the token's own key and value from registers and into their page.  Tables with runs that are
    not in use, and with a padding row's run, as a captured step has them."""
    ops = _ops()
    from tffinfer_amd.kernels.key_runs import deal_key_runs
    far = 77
    entries = [(20000, 1), (40, 1), (0, 1), (95, 1), (96, 1), (3000, 1), (255, 1), (256, 1), (31, 1), (32, 1), (1023, 1)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=3 + d)
    R = len(entries)
    g = torch.Generator().manual_seed(7)
    qkv = torch.randn(R, (nq + 2 * nkv) * d, generator=g).to(torch.bfloat16)
    q = qkv[:, :nq * d].reshape(R, nq, d)
    k_new = qkv[:, nq * d:(nq + nkv) * d].reshape(R, nkv, d)
    v_new = qkv[:, (nq + nkv) * d:].reshape(R, nkv, d)
    if window == 0:
        kfar = (30 * q[0, 0].float() / q[0, 0].float().norm()).to(torch.bfloat16)
        kv.k_cache[int(kv.block_tables[0, far // ps]), 0, far % ps] = kfar.to(DEV)
        ks[0][far, 0] = kfar
    scale = 1 / math.sqrt(d)
    bt = kv.block_tables.cpu()
    slots = torch.tensor([int(bt[r, P // ps]) * ps + P % ps for r, (P, _) in enumerate(entries)], dtype=torch.int32, device=DEV)
    refs = []
    for r, (P, _) in enumerate(entries):
        k = torch.cat([ks[r][:P], k_new[r:r + 1]])
        v = torch.cat([vs[r][:P], v_new[r:r + 1]])
        refs.append(_attn_ref(q[r:r + 1], k, v, positions[r:r + 1], window, scale)[0])
    ref = torch.stack(refs)
    runs, run_start, _, merge = deal_key_runs([P for P, _ in entries], window, nkv, target=waves, blocks=blocks)
    assert merge
    counts = run_start[1:] - run_start[:-1]
    assert counts[0] > 4 and (counts == 1).sum() >= 6 and (runs[:, 0] == -1).any()
    out = ops.attention_decode_fused(qkv.to(DEV), nq, nkv, d, None, None, 1e-6, None, 0, kv, batch, window, scale,
                                     slot_mapping=slots, key_runs=torch.from_numpy(runs.copy()).to(DEV),
                                     run_start=torch.from_numpy(run_start.copy()).to(DEV), runs_for_blocks=blocks)
    _close(out.reshape(R, nq, d), ref, ATTN_TOL, "keys dealt into runs")
    if window == 0:
        assert torch.allclose(out.reshape(R, nq, d)[0, 0].float().cpu(), vs[0][far, 0].float(), atol=5e-2)
    for r, (P, _) in enumerate(entries):
        assert torch.equal(kv.v_cache[int(bt[r, P // ps]), :, :, P % ps].cpu(), v_new[r]), f"value of entry {r} in its page"
    # what the kernel picks by itself (every entry's keys split alike) agrees to rounding
    same = ops.attention_decode_fused(qkv.to(DEV), nq, nkv, d, None, None, 1e-6, None, 0, kv, batch, window, scale)
    _close(out.reshape(R, nq, d), same.reshape(R, nq, d).double().cpu(), ATTN_TOL, "runs against equal splits")


@pytest.mark.parametrize("nq,nkv,d,ps,window", [(32, 8, 128, 16, 0), (8, 2, 32, 8, 300), (40, 2, 96, 8, 0)])
def test_attention_mfma_portions_beside_decoding_requests(nq, nkv, d, ps, window):
    """A step of long portions and of requests that bring one token with a long context: the
    latter have their keys dealt into runs for single waves (the longest one into several, whose
    partial results are merged), the former go to the block kernel, into the same output."""
    ops = _ops()
    entries = [(900, 1), (0, 300), (40, 1), (333, 150), (1500, 1), (7, 1)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=nq + d)
    T = batch.num_tokens
    g = torch.Generator().manual_seed(8)
    q = torch.randn(T, nq, d, generator=g).to(torch.bfloat16)
    scale = 1 / math.sqrt(d)
    out = ops.attention_mfma(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kv, batch, window, scale)
    runs, run_start, tokens, merge = batch._attn_work[("single_runs", nkv, window)]
    assert merge and run_start.tolist()[-1] > 4 and tokens.tolist() == [0, 301, 452, 453]
    gen = ops.attention_generic(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kv.k_cache, kv.v_cache, kv.block_tables,
                                batch.token_req, batch.positions, window, scale)
    _close(out, gen.double(), ATTN_TOL, "mixed step against the general kernel")
    # every entry's keys split alike, as before the runs: the same to rounding
    batch._attn_work.clear()
    same = ops.attention_mfma(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kv, batch, window, scale, splits=3)
    assert "single_rows" in batch._attn_work
    _close(same, gen.double(), ATTN_TOL, "mixed step with equal splits against the general kernel")
    cu = batch.host_cu_tokens
    for r, (P, n) in enumerate(entries):
        mine = torch.tensor([cu[r], cu[r + 1] - 1])
        ref = _attn_ref(q[mine], ks[r], vs[r], positions[mine], window, scale)
        _close(out.reshape(T, nq, d)[mine], ref, ATTN_TOL, f"request {r}")


@pytest.mark.parametrize("nq,nkv,d,ps,window", [(32, 8, 128, 16, 0), (8, 2, 32, 8, 300), (40, 2, 96, 8, 0)])
def test_attention_mfma_short_portions_beside_decoding_requests(nq, nkv, d, ps, window):
    """Portions of a few tokens (a wave of their own per 16 columns) beside requests that bring
    one token with a long context: those have their keys dealt into runs here too, and do not go
    to a single wave that walks all their keys."""
    ops = _ops()
    entries = [(900, 1), (0, 3), (1500, 1), (44, 2), (300, 1), (9, 1)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=nq + d + 1)
    assert batch.max_new_tokens * (nq // nkv) <= 64
    T = batch.num_tokens
    g = torch.Generator().manual_seed(9)
    q = torch.randn(T, nq, d, generator=g).to(torch.bfloat16)
    scale = 1 / math.sqrt(d)
    out = ops.attention_mfma(q.reshape(T, nq * d).to(DEV), nq, nkv, d, kv, batch, window, scale)
    assert ("single_runs", nkv, window) in batch._attn_work, "the decoding requests' keys were not dealt into runs"
    for r in range(len(entries)):
        sel = (token_req == r).nonzero().flatten()
        ref = _attn_ref(q[sel], ks[r], vs[r], positions[sel], window, scale)
        _close(out.reshape(T, nq, d)[sel], ref, ATTN_TOL, f"request {r}")


@pytest.mark.parametrize("splits", [1, 2, 5])
def test_attention_mfma_decode_more_pages_than_the_wave_keeps(splits):
    """A wave keeps 1024 page numbers at hand; with more pages in its run of keys it works
    through them in segments.  One key far back is made to dominate."""
    ops = _ops()
    nq, nkv, d, ps = 4, 2, 32, 8
    P, far = 8300, 77
    entries = [(P, 1), (40, 1)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=21)
    g = torch.Generator().manual_seed(5)
    q = torch.randn(2, nq, d, generator=g).to(torch.bfloat16)
    kfar = (30 * q[0, 0].float() / q[0, 0].float().norm()).to(torch.bfloat16)
    kv.k_cache[int(kv.block_tables[0, far // ps]), 0, far % ps] = kfar.to(DEV)
    ks[0][far, 0] = kfar
    scale = 1 / math.sqrt(d)
    ref = torch.stack([_attn_ref(q[r:r + 1], ks[r], vs[r], positions[r:r + 1], 0, scale)[0] for r in range(2)])
    out = ops.attention_mfma(q.reshape(2, nq * d).to(DEV), nq, nkv, d, kv, batch, 0, scale, splits=splits)
    _close(out.reshape(2, nq, d), ref, ATTN_TOL, "decode attention over 1038 pages")
    assert torch.allclose(out.reshape(2, nq, d)[0, 0].float().cpu(), vs[0][far, 0].float(), atol=5e-2)


@pytest.mark.parametrize("window", [0, 9000])
def test_attention_mfma_portion_over_more_pages_than_a_block_keeps(window):
    """A block keeps 2048 page numbers at hand; a portion late in a long prompt goes through
    its keys in segments, each with page numbers and a pipeline of copies of its own.  One
    key in the first segment and one in the last are made to stand out for two of the heads."""
    ops = _ops()
    nq, nkv, d, ps = 4, 2, 32, 8
    P, n, far1, far2 = 17300, 40, 131, 16900
    batch, kv, ks, vs, positions, token_req = _fake_step([(P, n)], ps, nkv, d, torch.bfloat16, seed=33)
    assert (P + n) // ps > 2048
    g = torch.Generator().manual_seed(6)
    q = torch.randn(n, nq, d, generator=g).to(torch.bfloat16)
    for far, (t, h) in ((far1, (3, 0)), (far2, (20, 3))):
        kfar = (30 * q[t, h].float() / q[t, h].float().norm()).to(torch.bfloat16)
        kv.k_cache[int(kv.block_tables[0, far // ps]), h // 2, far % ps] = kfar.to(DEV)
        ks[0][far, h // 2] = kfar
    scale = 1 / math.sqrt(d)
    ref = _attn_ref(q, ks[0], vs[0], positions, window, scale)
    out = ops.attention_mfma(q.reshape(n, nq * d).to(DEV), nq, nkv, d, kv, batch, window, scale)
    _close(out.reshape(n, nq, d), ref, ATTN_TOL, "portion over 2,167 pages")
    got = out.reshape(n, nq, d).float().cpu()
    if window == 0:      # (with the window the first of the two keys is out of sight)
        assert torch.allclose(got[3, 0], vs[0][far1, 0].float(), atol=5e-2)
    assert torch.allclose(got[20, 3], vs[0][far2, 1].float(), atol=5e-2)


def test_attention_mfma_far_key_and_window_edge():
    """A key far back is made to dominate; with a window that just excludes it
    the output must not see it, with a window that just includes it, it must."""
    ops = _ops()
    nq, nkv, d, ps = 8, 2, 64, 16
    P = 900
    far = 517
    for n in (1, 5):
        entries = [(P, n)]
        batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=9)
        q = torch.randn(n, nq, d).to(torch.bfloat16)
        for gidx in range(nkv):
            q[:, gidx * 4:(gidx + 1) * 4] = q[:, gidx * 4:gidx * 4 + 1]
            kfar = (40 * q[0, gidx * 4].float() / q[0, gidx * 4].float().norm()).to(torch.bfloat16)
            page = int(kv.block_tables[0, far // ps])
            kv.k_cache[page, gidx, far % ps] = kfar.to(DEV)
            ks[0][far, gidx] = kfar
        q[1:] = q[:1]
        for window, sees in ((0, True), (P - far + 1, True), (P - far, False)):
            ref = _attn_ref(q, ks[0], vs[0], positions, window, 1 / math.sqrt(d))
            out = ops.attention_mfma(q.reshape(n, nq * d).to(DEV), nq, nkv, d, kv, batch, window, 1 / math.sqrt(d))
            _close(out.reshape(n, nq, d), ref, ATTN_TOL, f"n={n} window={window}")
            hit = torch.allclose(out.reshape(n, nq, d)[0, 0].float().cpu(), vs[0][far, 0].float(), atol=5e-2)
            assert hit == sees, f"n={n} window={window}: far key {'missed' if sees else 'seen'}"


@pytest.mark.parametrize("cols", [128, 256])
def test_attention_mfma_blocks_far_key_and_window_edge(cols):
    """The same for the kernels whose blocks share keys through LDS (a portion of 40 tokens,
    blocks of 128 and of 256 columns): every token's query points at one key far back, whose
    score towers over all others (the softmax's reference has to jump to it and stay), and each
    token's window either just holds that key or has just passed it."""
    ops = _ops()
    nq, nkv, d, ps = 8, 2, 64, 16
    P, n, far = 900, 40, 517
    entries = [(P, n)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, nkv, d, torch.bfloat16, seed=19)
    q = torch.randn(1, nq, d).to(torch.bfloat16).repeat(n, 1, 1)
    for gidx in range(nkv):
        q[:, gidx * 4:(gidx + 1) * 4] = q[:, gidx * 4:gidx * 4 + 1]
        kfar = (40 * q[0, gidx * 4].float() / q[0, gidx * 4].float().norm()).to(torch.bfloat16)
        page = int(kv.block_tables[0, far // ps])
        kv.k_cache[page, gidx, far % ps] = kfar.to(DEV)
        ks[0][far, gidx] = kfar
    # token t is at position P + t: a window of P - far + 1 + t0 holds the far key for t <= t0 only
    for window, last_seeing in ((0, n - 1), (P - far + 1 + 17, 17), (P - far + 1, 0), (P - far, -1)):
        ref = _attn_ref(q, ks[0], vs[0], positions, window, 1 / math.sqrt(d))
        out = ops.attention_mfma(q.reshape(n, nq * d).to(DEV), nq, nkv, d, kv, batch, window, 1 / math.sqrt(d),
                                 block_cols=cols)
        _close(out.reshape(n, nq, d), ref, ATTN_TOL, f"window={window}")
        for t in range(n):
            hit = torch.allclose(out.reshape(n, nq, d)[t, 0].float().cpu(), vs[0][far, 0].float(), atol=5e-2)
            assert hit == (t <= last_seeing), f"window={window}, token {t}: far key {'missed' if t <= last_seeing else 'seen'}"


def test_attention_mfma_blocks_scores_that_creep_up():
    """Keys whose scores rise a little with every slice, by less than the slack the softmax's
    reference is given, for hundreds of keys, then by a lot: what the kernel sums against a
    reference that lags behind must equal the float64 softmax."""
    ops = _ops()
    nq, nkv, d, ps = 4, 1, 64, 16
    P, n = 0, 600
    batch, kv, ks, vs, positions, token_req = _fake_step([(P, n)], ps, nkv, d, torch.bfloat16, seed=29)
    u = torch.zeros(d)
    u[0] = 1.0
    q = (8.0 * u).to(torch.bfloat16).repeat(n, nq, 1)            # every query: 8 along the first axis
    for j in range(n):
        rise = 0.02 * j if j < 500 else 10.0 + 0.5 * (j - 500)    # scaled score = rise (d = 64: 8 * k0 / 8)
        k = torch.zeros(d)
        k[0] = rise
        ks[0][j, 0] = k.to(torch.bfloat16)
        kv.k_cache[int(kv.block_tables[0, j // ps]), 0, j % ps] = k.to(torch.bfloat16).to(DEV)
    ref = _attn_ref(q, ks[0], vs[0], positions, 0, 1 / math.sqrt(d))
    for cols in (128, 256):
        out = ops.attention_mfma(q.reshape(n, nq * d).to(DEV), nq, nkv, d, kv, batch, 0, 1 / math.sqrt(d), block_cols=cols)
        _close(out.reshape(n, nq, d), ref, ATTN_TOL, f"creeping scores, blocks of {cols}")


@pytest.mark.parametrize("M", [1, 8, 20, 50, 200])
@pytest.mark.parametrize("I,K", [(200, 96), (64, 64), (1000, 256), (12288, 512), (8200, 104), (4100, 1000), (3000, 2080)])
def test_linear_with_gated_epilogue(M, I, K):
    """Gate and up interleaved in one weight: the product yields silu(x Wg^T) * (x Wu^T)."""
    ops = _ops()
    g = torch.Generator().manual_seed(I + M)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    wg = (torch.randn(I, K, generator=g) * 0.2).to(torch.bfloat16)
    wu = (torch.randn(I, K, generator=g) * 0.2).to(torch.bfloat16)
    pw = ops.pack_gate_up(wg.to(DEV), wu.to(DEV))
    assert pw.glu_out == I and pw.N == 2 * (-(-I // 16) * 16)
    out = ops.linear(x.to(DEV), pw)
    assert out.shape == (M, I) and out.dtype == torch.bfloat16
    gt, up = x.double() @ wg.double().T, x.double() @ wu.double().T
    _close(out, gt / (1 + torch.exp(-gt)) * up, 8e-3, "gated product")
    out32 = ops.linear(x.to(DEV), pw, out_dtype=torch.float32)
    _close(out32, gt / (1 + torch.exp(-gt)) * up, 3e-5, "gated product, float32 out")


def test_measured_ceilings_are_plausible():
    """The measuring kernels run and land where an MI355X can: well above a fraction of the
    published peaks, never above them."""
    c = _ops().measure_ceilings(DEV, gib=1.0)
    assert 1000 < c["stream_read_GBps"] <= 8000
    assert 300 < c["mfma_bf16_TFLOPs_1_waves_per_simd"] <= c["mfma_bf16_TFLOPs_4_waves_per_simd"] * 1.1 <= 2500 * 1.1

    # operands that change cost power, never gain speed (a tenth of slack for the clock's wander)
    assert 300 < c["mfma_bf16_TFLOPs_varied_operands"] <= c["mfma_bf16_TFLOPs_4_waves_per_simd"] * 1.1
