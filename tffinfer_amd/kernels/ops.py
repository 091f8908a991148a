"""The op table: every operation of the engine bound to exactly one HIP kernel.

Each function checks on the host that its operands have the device, element
type, contiguity and shape the kernel assumes (a kernel is never launched on
operands it cannot address), allocates the result with torch's allocator and
launches on torch's current stream.  There is no CPU path and no library
fallback: without the compiled library every call raises.

The reference binds ops to kernels by name in its FunctionFactory
(include/FunctionFactory.h:18-116, kernel/include/TFFOPCreatorBase.h:73-97)
with a device dispatch; here the table has one entry per op and no dispatch.
"""
from __future__ import annotations

import ctypes
import math

import numpy as np
import torch

from . import lib as _lib
from .key_runs import deal_key_runs
from . import staging as _staging

_DT = {torch.float32: 0, torch.bfloat16: 1}


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DT[dt]
    except KeyError:
        raise _lib.KernelError(f"element type {dt} is not supported (float32 or bfloat16)") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current stream's handle.  Asked for at every launch (hundreds a step when a step is
    launched kernel by kernel): through torch's C binding where there is one, which costs a
    tenth of building a Stream object."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _req(t: torch.Tensor, name: str, dtype=None, ndim=None):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise _lib.KernelError(f"{name}: expected a tensor on the GPU")
    if not t.is_contiguous():
        raise _lib.KernelError(f"{name}: tensor is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise _lib.KernelError(f"{name}: expected {dtype}, got {t.dtype}")
    if ndim is not None and t.dim() != ndim:
        raise _lib.KernelError(f"{name}: expected {ndim} dimensions, got shape {tuple(t.shape)}")
    return t


def _check_cache(k_cache, v_cache, nkv, d, what):
    """Keys [pages, nkv, page_size, d]; values transposed [pages, nkv, d, page_size]."""
    pages, h, ps, dd = k_cache.shape
    if h != nkv or dd != d or tuple(v_cache.shape) != (pages, nkv, d, ps) or v_cache.dtype != k_cache.dtype:
        raise _lib.KernelError(
            f"{what}: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} are not keys "
            f"[pages, {nkv}, page_size, {d}] and values [pages, {nkv}, {d}, page_size]")


def _ptr(t):
    return None if t is None else t.data_ptr()


class PackedWeight:
    """A bfloat16 matrix [N, K] in the fragment order of the matrix-core
    products: tiles of 16 rows by 32 k stored as the 1 KB operand a wave loads,
    rows and k padded with zeros to multiples of 16 and 32."""
    __slots__ = ("data", "N", "K", "glu_out")

    def __init__(self, data: torch.Tensor, N: int, K: int, glu_out: int = 0):
        self.data, self.N, self.K = data, int(N), int(K)
        #: > 0: the 16-row groups alternate between a gate and an up projection and the
        #: product yields silu(gate) * up with this many columns
        self.glu_out = int(glu_out)

    @property
    def shape(self):
        return (self.N, self.K)

    @property
    def out_features(self) -> int:
        return self.glu_out or self.N

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def device(self):
        return self.data.device

    def data_ptr(self) -> int:
        return self.data.data_ptr()

    def unpack(self) -> torch.Tensor:
        """Back to row-major [N, K] (for tests and inspection)."""
        NB, KB = -(-self.N // 16), -(-self.K // 32)
        t = self.data.view(NB, KB, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(NB * 16, KB * 32)
        return t[:self.N, :self.K].contiguous()


def pack_weight(w: torch.Tensor) -> PackedWeight:
    """Row-major bfloat16 [N, K] on the GPU -> fragment order."""
    _req(w, "pack_weight", torch.bfloat16, 2)
    N, K = w.shape
    if K % 8:
        raise _lib.KernelError(f"pack_weight: inner size {K} must be a multiple of 8")
    NB, KB = -(-N // 16), -(-K // 32)
    out = torch.empty(NB * KB * 512, dtype=torch.bfloat16, device=w.device)
    L = _lib.load()
    _lib.check(L.tff_pack_weight(w.data_ptr(), out.data_ptr(), N, K, _stream()))
    return PackedWeight(out, N, K)


def pack_gate_up(gate: torch.Tensor, up: torch.Tensor) -> PackedWeight:
    """Gate and up projections [I, K] (bfloat16, on the GPU) as one weight whose
    16-row groups alternate gate, up, gate, up, ..., in fragment order.  A
    product with it yields silu(x gate^T) * (x up^T) directly: the activation
    runs in the product's epilogue, on the float32 accumulators."""
    _req(gate, "gate", torch.bfloat16, 2)
    _req(up, "up", torch.bfloat16, 2)
    if gate.shape != up.shape:
        raise _lib.KernelError(f"pack_gate_up: gate {tuple(gate.shape)} and up {tuple(up.shape)} differ")
    I, K = gate.shape
    groups = -(-I // 16)
    padded = torch.zeros(2, groups * 16, K, dtype=torch.bfloat16, device=gate.device)
    padded[0, :I] = gate
    padded[1, :I] = up
    both = padded.view(2, groups, 16, K).permute(1, 0, 2, 3).reshape(groups * 32, K).contiguous()
    pw = pack_weight(both)
    pw.glu_out = I
    return pw


def embed(table, ids: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """Rows of ``table`` [V, H] (a row-major tensor or a PackedWeight) for
    int32 ``ids`` [T] as float32 [T, H]."""
    packed = isinstance(table, PackedWeight)
    if packed:
        _req(table.data, "embed table", torch.bfloat16, 1)
    else:
        _req(table, "embed table", ndim=2)
    _req(ids, "embed ids", torch.int32, 1)
    V, H = table.shape
    T = ids.numel()
    if out is None:
        out = torch.empty(T, H, dtype=torch.float32, device=table.device)
    else:
        _req(out, "embed out", torch.float32, 2)
        if tuple(out.shape) != (T, H):
            raise _lib.KernelError(f"embed out: shape {tuple(out.shape)} is not {(T, H)}")
    L = _lib.load()
    if packed:
        _lib.check(L.tff_embed_packed(table.data_ptr(), ids.data_ptr(), out.data_ptr(), T, H, V, _stream()))
    else:
        _lib.check(L.tff_embed(table.data_ptr(), ids.data_ptr(), out.data_ptr(), T, H, V,
                               dtype_code(table.dtype), _stream()))
    return out


class PendingProduct:
    """A product ``x . weight^T`` of up to 16 bfloat16 rows that ``linear`` was
    asked for with ``partials=True`` and has not run: ``add_rmsnorm`` runs it
    with the residual sum and the norm's weight in its epilogue when the norm's
    result goes to another such product, and plainly (:meth:`run`) otherwise."""

    def __init__(self, x: torch.Tensor, weight: "PackedWeight"):
        self.x, self.weight = x, weight
        self.shape = (x.shape[0], weight.shape[0])
        self.device = x.device

    def run(self) -> torch.Tensor:
        return linear(self.x, self.weight, out_dtype=torch.float32)


class ScaledRows:
    """The result of an RMS norm whose per-row factor has not been applied:
    ``x`` [M, H] bfloat16 = (residual stream) * (norm weight), and the sums of
    squares of every row's groups of 16 columns, ``ss`` [16, stride] float32
    (``count`` of them a row).  ``linear`` applies rsqrt(sum / H + eps) to its
    accumulators; :meth:`materialize` writes the normalised rows out, from the
    float32 residual stream ``resid`` (which must still hold the sum the norm
    was taken of) and the norm's ``weight``, so that they are rounded to
    bfloat16 once, as the norm's own kernel rounds them."""

    def __init__(self, x: torch.Tensor, ss: torch.Tensor, count: int, eps: float,
                 resid: torch.Tensor, weight: torch.Tensor):
        self.x, self.ss, self.count, self.eps = x, ss, int(count), float(eps)
        self.resid, self.weight = resid, weight
        self.shape, self.dtype, self.device = x.shape, x.dtype, x.device

    def materialize(self) -> torch.Tensor:
        return add_rmsnorm(self.resid, None, self.weight, self.eps, self.x.dtype)


def as_tensor(t) -> torch.Tensor:
    """Whatever ``linear`` or ``add_rmsnorm`` returned, as a plain tensor: a
    product that has not run is run, partial sums [S, T, H] are added up in
    order, rows that lack their norm's factor get it."""
    if isinstance(t, PendingProduct):
        return t.run()
    if isinstance(t, ScaledRows):
        return t.materialize()
    if isinstance(t, torch.Tensor) and t.dim() == 3:
        acc = t[0].clone()
        for part in t[1:]:
            acc += part
        return acc
    return t


def _fused_prenorm(p: PendingProduct, resid: torch.Tensor, weight: torch.Tensor, eps: float) -> ScaledRows:
    x = p.x
    M, K = x.shape
    N = p.weight.shape[0]
    lda = x.stride(0) if M > 1 else K
    groups = -(-N // 16)
    stride = -(-groups // 4) * 4
    xs = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    ss = torch.empty(16, stride, dtype=torch.float32, device=x.device)
    L = _lib.load()
    _lib.check(L.tff_gemm_residual_prenorm(x.data_ptr(), p.weight.data_ptr(), M, N, K, lda, resid.data_ptr(),
                                           weight.data_ptr(), xs.data_ptr(), ss.data_ptr(), stride, _stream()))
    return ScaledRows(xs, ss, groups, eps, resid, weight)


def add_rmsnorm(resid: torch.Tensor, delta, weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: torch.Tensor | None = None,
                out: torch.Tensor | None = None, for_linear: bool = False):
    """``resid += delta`` (when given and ``rows`` is None) and the RMS norm of
    the sum; with ``rows`` the norm of those rows only, ``resid`` untouched.
    ``delta`` may be what ``linear`` returns with ``partials=True``: a stack
    [S, T, H] of partial sums, which are added up first, in order, or a
    product that has not run.  ``for_linear``: the result goes to ``linear``
    and nowhere else, so it may be a :class:`ScaledRows`."""
    _req(resid, "add_rmsnorm resid", torch.float32, 2)
    H = resid.shape[1]
    _req(weight, "add_rmsnorm weight", torch.float32, 1)
    if weight.numel() != H:
        raise _lib.KernelError(f"add_rmsnorm: weight has {weight.numel()} elements, rows have {H}")
    if isinstance(delta, PendingProduct):
        if tuple(delta.shape) != tuple(resid.shape):
            raise _lib.KernelError(
                f"add_rmsnorm: delta {tuple(delta.shape)} does not match resid {tuple(resid.shape)}")
        if for_linear and rows is None and out is None and out_dtype == torch.bfloat16:
            return _fused_prenorm(delta, resid, weight, eps)
        delta = delta.run()
    planes, plane = 1, 0
    if delta is not None:
        _req(delta, "add_rmsnorm delta", torch.float32, 3 if delta.dim() == 3 else 2)
        if tuple(delta.shape[-2:]) != tuple(resid.shape):
            raise _lib.KernelError(
                f"add_rmsnorm: delta {tuple(delta.shape)} does not match resid {tuple(resid.shape)}")
        if delta.dim() == 3:
            planes, plane = delta.shape[0], delta.stride(0)
    if rows is not None:
        _req(rows, "add_rmsnorm rows", torch.int32, 1)
        n = rows.numel()
    else:
        n = resid.shape[0]
    if out is None:
        out = torch.empty(n, H, dtype=out_dtype, device=resid.device)
    else:
        _req(out, "add_rmsnorm out", out_dtype, 2)
        if tuple(out.shape) != (n, H):
            raise _lib.KernelError(f"add_rmsnorm out: shape {tuple(out.shape)} is not {(n, H)}")
    L = _lib.load()
    _lib.check(L.tff_add_rmsnorm(resid.data_ptr(), _ptr(delta), planes, plane, weight.data_ptr(), float(eps),
                                 out.data_ptr(), _ptr(rows), n, H, dtype_code(out_dtype), _stream()))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm over the last dimension of a dense tensor, float32 weight."""
    _req(x, "rmsnorm x")
    H = x.shape[-1]
    _req(weight, "rmsnorm weight", torch.float32, 1)
    if weight.numel() != H:
        raise _lib.KernelError(f"rmsnorm: weight has {weight.numel()} elements, rows have {H}")
    out = torch.empty_like(x)
    L = _lib.load()
    _lib.check(L.tff_rmsnorm(x.data_ptr(), weight.data_ptr(), float(eps), out.data_ptr(),
                             x.numel() // H, H, dtype_code(x.dtype), _stream()))
    return out


_plan_cache: dict = {}


def _plan_tile(L, M: int, N: int, K: int) -> int:
    """Rows of the tile the product's plan takes when partial sums are kept (0: the streaming kernel)."""
    key = (M, N, K)
    if key not in _plan_cache:
        r, c, s = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        _lib.check(L.tff_gemm_plan(M, N, K, 0, 1, ctypes.byref(r), ctypes.byref(c), ctypes.byref(s)))
        _plan_cache[key] = r.value
    return _plan_cache[key]


def linear(x: torch.Tensor, weight, out_dtype: torch.dtype | None = None,
           out: torch.Tensor | None = None, partials: bool = False) -> torch.Tensor:
    """``x . weight^T`` for x [M, K] (rows may be strided) and weight [N, K]:
    a row-major float32 tensor, or a PackedWeight for bfloat16.

    ``partials=True`` (float32 result): where the product splits K over
    blocks, the partial sums are returned as they are, [S, M, N], for a
    consumer that adds them up anyway (``add_rmsnorm``); else the result is
    [M, N] as always."""
    packed = isinstance(weight, PackedWeight)
    if isinstance(x, ScaledRows):
        if packed and out is None and not partials and x.shape[1] == weight.shape[1]:
            return _linear_row_scaled(x, weight, out_dtype or x.dtype)
        x = x.materialize()
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dim() != 2 or x.stride(1) != 1:
        raise _lib.KernelError("linear x: expected a GPU matrix with unit inner stride")
    if packed:
        _req(weight.data, "linear weight", x.dtype, 1)
    else:
        _req(weight, "linear weight", x.dtype, 2)
        if weight.dtype == torch.bfloat16:
            raise _lib.KernelError("linear: a bfloat16 weight must be a PackedWeight (pack_weight)")
    M, K = x.shape
    N, K2 = weight.shape
    if K != K2:
        raise _lib.KernelError(f"linear: x has inner size {K}, weight [out, in] = {tuple(weight.shape)}")
    lda = x.stride(0) if M > 1 else K
    if lda < K:
        raise _lib.KernelError("linear x: rows overlap")
    out_dtype = out_dtype or x.dtype
    glu_out = weight.glu_out if packed else 0
    n_out = glu_out or N
    L = _lib.load()
    # some shapes (few columns for the rows) split K over blocks and need room for partial sums
    want = bool(partials and packed and out is None and out_dtype == torch.float32 and not glu_out)
    if want and M <= 16 and N % 8 == 0 and x.dtype == torch.bfloat16 and x.data_ptr() % 16 == 0 and lda % 8 == 0:
        if _plan_tile(L, M, N, K) == 0:
            return PendingProduct(x, weight)   # a few rows: the consumer runs it with its own work in the epilogue
        # (else the streaming kernel's blocks would go badly round the CUs: tiles that split K, partial sums kept)
    ws_bytes = (L.tff_gemm_workspace_bytes(M, N, K, dtype_code(x.dtype), 1 if glu_out else 0, 1 if want else 0)
                if packed else 0)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=x.device) if ws_bytes else None
    keep = want and ws is not None
    if keep:
        out = ws.view(-1, M, N)
    elif out is None:
        out = torch.empty(M, n_out, dtype=out_dtype, device=x.device)
    else:
        _req(out, "linear out", out_dtype, 2)
        if tuple(out.shape) != (M, n_out):
            raise _lib.KernelError(f"linear out: shape {tuple(out.shape)} is not {(M, n_out)}")
    _lib.check(L.tff_gemm(x.data_ptr(), weight.data_ptr(), out.data_ptr(), M, N, K, lda,
                          dtype_code(x.dtype), dtype_code(out_dtype), 1 if packed else 0, glu_out,
                          _ptr(ws), ws_bytes, 1 if keep else 0, _stream()))
    return out


def _linear_row_scaled(x: ScaledRows, weight: "PackedWeight", out_dtype: torch.dtype) -> torch.Tensor:
    M, K = x.shape
    N = weight.shape[0]
    glu_out = weight.glu_out
    out = torch.empty(M, glu_out or N, dtype=out_dtype, device=x.device)
    L = _lib.load()
    _lib.check(L.tff_gemm_row_scaled(x.x.data_ptr(), weight.data_ptr(), out.data_ptr(), M, N, K, K,
                                     dtype_code(out_dtype), glu_out, x.ss.data_ptr(), x.ss.stride(0), x.count, K,
                                     x.eps, _stream()))
    return out


def qk_norm_rope_kv(qkv: torch.Tensor, nq: int, nkv: int, d: int,
                    q_weight: torch.Tensor | None, k_weight: torch.Tensor | None, eps: float,
                    cos_sin: torch.Tensor | None, pairing: int,
                    positions: torch.Tensor, slot_mapping: torch.Tensor,
                    k_cache: torch.Tensor, v_cache: torch.Tensor) -> None:
    """In place on the fused projection output ``qkv`` [T, (nq + 2 nkv) d]; see
    the entry point's comment.  ``cos_sin`` is [max_pos, rot/2, 2] float32."""
    _req(qkv, "qk_norm_rope_kv qkv", ndim=2)
    T = qkv.shape[0]
    if qkv.shape[1] != (nq + 2 * nkv) * d:
        raise _lib.KernelError(
            f"qk_norm_rope_kv: rows of {qkv.shape[1]} are not (nq + 2 nkv) d = {(nq + 2 * nkv) * d}")
    for w, nm in ((q_weight, "q norm weight"), (k_weight, "k norm weight")):
        if w is not None:
            _req(w, nm, torch.float32, 1)
            if w.numel() != d:
                raise _lib.KernelError(f"{nm}: {w.numel()} elements, head size {d}")
    rot, max_pos = 0, 0
    if cos_sin is not None:
        _req(cos_sin, "rotation table", torch.float32, 3)
        max_pos, half, two = cos_sin.shape
        if two != 2:
            raise _lib.KernelError("rotation table: last dimension must hold (cos, sin)")
        rot = 2 * half
    _req(positions, "positions", torch.int32, 1)
    _req(slot_mapping, "slot_mapping", torch.int32, 1)
    if positions.numel() != T or slot_mapping.numel() != T:
        raise _lib.KernelError("qk_norm_rope_kv: positions and slot_mapping need one entry per token")
    _req(k_cache, "k cache", ndim=4)
    _req(v_cache, "v cache", ndim=4)
    _check_cache(k_cache, v_cache, nkv, d, "qk_norm_rope_kv")
    L = _lib.load()
    _lib.check(L.tff_qk_norm_rope_kv(
        qkv.data_ptr(), T, nq, nkv, d, _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(cos_sin),
        rot, int(pairing), max_pos, positions.data_ptr(), slot_mapping.data_ptr(),
        k_cache.data_ptr(), v_cache.data_ptr(), k_cache.shape[2], k_cache.shape[0],
        dtype_code(qkv.dtype), dtype_code(k_cache.dtype), _stream()))


def attention_generic(q: torch.Tensor, nq: int, nkv: int, d: int, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, block_tables: torch.Tensor, token_req: torch.Tensor,
                      positions: torch.Tensor, window: int = 0, scale: float | None = None,
                      out: torch.Tensor | None = None) -> torch.Tensor:
    """Attention of each token over its request's pages; q is [T, >= nq*d]
    with the query heads at the start of each row.  Returns [T, nq*d]."""
    _req(q, "attention q", ndim=2)
    T = q.shape[0]
    if q.shape[1] < nq * d:
        raise _lib.KernelError(f"attention q: rows of {q.shape[1]} hold fewer than nq*d = {nq * d}")
    _req(k_cache, "k cache", q.dtype, 4)
    _req(v_cache, "v cache", q.dtype, 4)
    _check_cache(k_cache, v_cache, nkv, d, "attention")
    _req(block_tables, "block tables", torch.int32, 2)
    _req(token_req, "token_req", torch.int32, 1)
    _req(positions, "positions", torch.int32, 1)
    if token_req.numel() != T or positions.numel() != T:
        raise _lib.KernelError("attention: token_req and positions need one entry per token")
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    if out is None:
        out = torch.empty(T, nq * d, dtype=q.dtype, device=q.device)
    L = _lib.load()
    _lib.check(L.tff_attention_generic(
        q.data_ptr(), q.stride(0), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
        block_tables.data_ptr(), block_tables.stride(0), token_req.data_ptr(), positions.data_ptr(),
        T, nq, nkv, d, k_cache.shape[2], k_cache.shape[0], int(window), float(scale),
        dtype_code(q.dtype), dtype_code(k_cache.dtype), _stream()))
    return out


def mfma_attention_supported(dtype: torch.dtype, d: int, page_size: int) -> bool:
    return dtype == torch.bfloat16 and bool(_lib.load().tff_attention_mfma_supported(int(d), int(page_size)))


def _entries(batch, which: str) -> list[int]:
    """Rows of the step's entries: all, those that bring one token, or the others."""
    cu = batch.host_cu_tokens
    rows = range(len(cu) - 1)
    if which == "all":
        return list(rows)
    one = which == "single"
    return [r for r in rows if (cu[r + 1] - cu[r] == 1) == one]


def _attention_work(batch, G: int, cols: int, device, which: str = "all") -> torch.Tensor:
    """(entry, first column) of every wave's tile for the step's entries; a
    column is a (token, q head of the group) pair numbered token * G + head."""
    cache = getattr(batch, "_attn_work", None)
    if cache is None:
        cache = batch._attn_work = {}
    key = (G, cols, which)
    if key not in cache:
        cu = batch.host_cu_tokens
        flat = []
        for r in _entries(batch, which):
            for c0 in range(0, (cu[r + 1] - cu[r]) * G, cols):
                flat.extend((r, c0))
        cache[key] = _staging.send(device, [np.asarray(flat, dtype=np.int32).reshape(-1, 2)])[0]
    return cache[key]


_cu_count = {}


def _num_cus(device) -> int:
    idx = torch.device(device).index or 0
    if idx not in _cu_count:
        _cu_count[idx] = torch.cuda.get_device_properties(idx).multi_processor_count
    return _cu_count[idx]


def _attention_block_work(batch, G: int, nkv: int, window: int, device, cols: int = 128,
                          bins: int | None = None, which: str = "all", key_groups: int | None = None,
                          head_dim: int = 128, num_cus: int | None = None):
    """Work table of the block kernel: items (entry, first column) of ``cols``
    columns, dealt to blocks so that every block goes through about the same
    number of 32-key slices (an item late in a long prompt sees many times the
    keys of an early one).  There are at most as many blocks as the device
    can hold at once, so none waits for another to end: with little work one
    block a CU whose two groups of waves share an item's slices, with plenty
    (some 96 slices a block and more) two blocks of one group a CU.  Returns
    (items [n, 2], block_items [blocks + 1], blocks, key groups)."""
    cache = getattr(batch, "_attn_work", None)
    if cache is None:
        cache = batch._attn_work = {}
    key = ("blocks", G, nkv, cols, window, bins, which, key_groups, head_dim, num_cus)
    if key not in cache:
        cu, P = batch.host_cu_tokens, batch.host_start_pos
        items = []                       # (slices, entry, first column)
        for r in _entries(batch, which):
            ncols = (cu[r + 1] - cu[r]) * G
            for c0 in range(0, ncols, cols):
                first = P[r] + c0 // G
                last = P[r] + (min(c0 + cols, ncols) - 1) // G
                lo = max(0, first - window + 1) if window > 0 else 0
                items.append((last // 32 - lo // 32 + 1, r, c0))
        if num_cus is None:
            num_cus = _num_cus(device) if torch.device(device).type == "cuda" else 256
        per_cu = max(1, num_cus // max(1, nkv))
        groups = key_groups
        if groups is None:
            groups = 2
            if head_dim <= 128 and sum(it[0] for it in items) >= 96 * 2 * per_cu:
                groups = 1
        if head_dim > 128:
            groups = 1                   # LDS holds one group's stages there
        nbins = bins if bins is not None else (per_cu if groups == 2 or head_dim > 128 else 2 * per_cu)
        if len(items) <= nbins:
            order = sorted(items, reverse=True)        # the longest start first
            starts = list(range(len(order) + 1))
        else:
            # longest first, each to the block with the least to do so far
            import heapq
            loads = [(0, b) for b in range(nbins)]
            heapq.heapify(loads)
            per_bin = [[] for _ in range(nbins)]
            for it in sorted(items, reverse=True):
                load, b = heapq.heappop(loads)
                per_bin[b].append(it)
                heapq.heappush(loads, (load + it[0], b))
            order, starts = [], [0]
            for lst in per_bin:
                order.extend(lst)
                starts.append(len(order))
        flat = [x for it in order for x in it[1:]]
        items_d, starts_d = _staging.send(device, [np.asarray(flat, dtype=np.int32).reshape(-1, 2),
                                                   np.asarray(starts, dtype=np.int32)])
        cache[key] = (items_d, starts_d, len(starts) - 1, groups)
    return cache[key]


def _pick_block_cols(batch, G: int, nkv: int, window: int, device, which: str, head_dim: int) -> int:
    """128 or 256 columns to a block of the prompt attention.  Blocks of 256 columns (two
    column tiles a wave) read half as much from LDS and fetch half as many keys per flop.
    Measured alone they are ahead from some 3,500 tokens on (a tenth at 32,768 tokens, a
    quarter on the slower boxes of the pool); inside a whole prefill, between products that
    hold the chip at its power limit, the two are within a percent or two of each other up to
    16,384 tokens.  They are taken for the longest prompts only, where they were never behind:
    4,096 slices of 32 keys a block and more (some 24,000 tokens at four query heads to a key
    head)."""
    if head_dim > 128:
        return 128
    cache = getattr(batch, "_attn_work", None)
    if cache is None:
        cache = batch._attn_work = {}
    key = ("block_cols", G, nkv, window, which, head_dim)
    if key not in cache:
        cu, P = batch.host_cu_tokens, batch.host_start_pos
        slices = 0
        for r in _entries(batch, which):
            ncols = (cu[r + 1] - cu[r]) * G
            for c0 in range(0, ncols, 256):
                first = P[r] + c0 // G
                last = P[r] + (min(c0 + 256, ncols) - 1) // G
                lo = max(0, first - window + 1) if window > 0 else 0
                slices += last // 32 - lo // 32 + 1
        num_cus = _num_cus(device) if torch.device(device).type == "cuda" else 256
        per_cu = max(1, num_cus // max(1, nkv))
        cache[key] = 256 if slices >= 4096 * per_cu else 128
    return cache[key]


#: (for a caller that brings no runs of keys, see ``kernels.key_runs``, which is how the engine's steps come)
#: entries x kv heads from which a decode step gives every pair a block of eight waves that
#: split its keys and merge in LDS, instead of splitting the keys over blocks of one wave and
#: merging in a second kernel.  A block a pair keeps only as many CUs busy as there are pairs, and
#: eight waves do not pull a CU's share of HBM alone: measured at the 8B shape (eight kv heads),
#: 128 pairs are 1 % (2,048 cached tokens) to 11 % (32,768) slower as blocks, 160 pairs and more
#: 3 to 7 % faster at every length.
BLOCK_DECODE_MIN_PAIRS = 160


def pick_splits(waves: int, max_context: int) -> int:
    """Into how many runs the keys of a decoding request are split so that
    the launch has enough waves to pull on all of HBM: about 512 waves (a wave
    alone on its SIMD streams some 30 GB/s), at least 128 keys per run."""
    return max(1, min(-(-512 // max(1, waves)), -(-max_context // 128), 256))


def attention_mfma(q: torch.Tensor, nq: int, nkv: int, d: int, kv, batch, window: int = 0,
                   scale: float | None = None, splits: int | None = None,
                   block_bins: int | None = None, key_groups: int | None = None,
                   block_cols: int | None = None) -> torch.Tensor:
    """bfloat16 attention of the step's tokens on the matrix cores; decode-only
    steps split each request's keys over several waves and merge them.
    ``splits``, ``block_bins`` (blocks per kv head that share the work of
    long portions) and ``key_groups`` (groups of waves in such a block)
    override the choices made from the step's sizes."""
    _req(q, "attention q", torch.bfloat16, 2)
    T = q.shape[0]
    if q.shape[1] < nq * d:
        raise _lib.KernelError(f"attention q: rows of {q.shape[1]} hold fewer than nq*d = {nq * d}")
    k_cache, v_cache = kv.k_cache, kv.v_cache
    _req(k_cache, "k cache", q.dtype, 4)
    _req(v_cache, "v cache", q.dtype, 4)
    _check_cache(k_cache, v_cache, nkv, d, "attention")
    bt = _req(kv.block_tables, "block tables", torch.int32, 2)
    _req(batch.cu_tokens, "cu_tokens", torch.int32, 1)
    _req(batch.start_pos, "start_pos", torch.int32, 1)
    R = batch.num_reqs
    if batch.cu_tokens.numel() != R + 1 or batch.start_pos.numel() != R or bt.shape[0] != R:
        raise _lib.KernelError("attention: the step's tables do not describe the same number of requests")
    if batch.num_tokens != T:
        raise _lib.KernelError(f"attention: {T} query rows for a step of {batch.num_tokens} tokens")
    G = nq // nkv
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    out = torch.empty(T, nq * d, dtype=q.dtype, device=q.device)
    L = _lib.load()
    stream = _stream()

    def launch(work, num_work, block_items, num_blocks, tiles, cols, splits, rows=None, groups=2):
        # partial results of split keys are kept by entry (split entries bring one token each)
        part_o = part_ml = None
        if splits > 1:
            part_o = torch.empty(splits, R, nq, d, dtype=torch.float32, device=q.device)
            part_ml = torch.empty(splits, R, nq, 2, dtype=torch.float32, device=q.device)
        _lib.check(L.tff_attention_mfma(
            q.data_ptr(), q.stride(0), out.data_ptr(), _ptr(part_o), _ptr(part_ml), k_cache.data_ptr(),
            v_cache.data_ptr(), bt.data_ptr(), bt.stride(0), batch.cu_tokens.data_ptr(),
            batch.start_pos.data_ptr(), _ptr(work), num_work, _ptr(block_items), num_blocks, tiles, cols,
            groups, splits, R if splits > 1 else T, nq, nkv, d, k_cache.shape[2], k_cache.shape[0], int(window),
            float(scale), stream))
        if splits > 1:
            _lib.check(L.tff_attention_split_reduce(
                part_o.data_ptr(), part_ml.data_ptr(), out.data_ptr(), splits, R, nq, d, _ptr(rows),
                0 if rows is None else rows.shape[0], stream))

    if batch.max_new_tokens == 1:
        # decoding only: a wave per request, kv head and run of keys; sizes come from the tables
        tiles = -(-G // 16)
        runs = getattr(kv, "key_runs", None)
        if splits is None and runs is not None and kv.runs_window == int(window) and T == R:
            # (the keys dealt into runs by the step's tables; entry i's token is row i)
            part_o = torch.empty(runs.shape[0], nq, d, dtype=torch.float32, device=q.device)
            part_ml = torch.empty(runs.shape[0], nq, 2, dtype=torch.float32, device=q.device)
            _lib.check(L.tff_attention_mfma_runs(
                q.data_ptr(), q.stride(0), out.data_ptr(), part_o.data_ptr(), part_ml.data_ptr(), k_cache.data_ptr(),
                v_cache.data_ptr(), bt.data_ptr(), bt.stride(0), batch.cu_tokens.data_ptr(), batch.start_pos.data_ptr(),
                runs.data_ptr(), kv.run_start.data_ptr(), batch.cu_tokens.data_ptr(), runs.shape[0], R,
                1 if kv.runs_merge else 0, T, nq, nkv, d, k_cache.shape[2], k_cache.shape[0], int(window), float(scale),
                stream))
            return out
        if splits is None:
            splits = pick_splits(R * tiles * nkv, batch.max_context)
        launch(None, R * tiles, None, 0, tiles, 16, splits)
        return out
    # long portions: blocks that share their keys through LDS (128 columns); short ones: a wave
    # of its own per 16 columns
    cols = 128 if batch.max_new_tokens * G > 64 else 16
    which = "all"
    single = _entries(batch, "single")
    if single and batch.max_context >= 256:
        # Requests that decode beside the portions have one token each and possibly long
        # contexts: they get the split-key kernel of their own rather than one block, or one
        # wave, each for all their keys.
        which = "multi"
        cache = getattr(batch, "_attn_work", None)
        if cache is None:
            cache = batch._attn_work = {}
        if splits is None and getattr(batch, "host_start_pos", None) is not None:
            # their keys dealt into runs of similar length, whatever the requests' lengths
            key = ("single_runs", nkv, int(window))
            if key not in cache:
                cu = batch.host_cu_tokens
                dealt = deal_key_runs([batch.host_start_pos[r] for r in single], int(window), nkv, blocks=False)
                runs = dealt.runs.copy()
                used = int(dealt.run_start[-1])
                runs[:used, 0] = np.asarray(single, dtype=np.int32)[runs[:used, 0]]     # rows of the step's tables
                cache[key] = tuple(_staging.send(q.device, [runs, dealt.run_start.copy(),
                                                            np.asarray([cu[r] for r in single], dtype=np.int32)])) \
                    + (dealt.merge,)
            runs, run_start, tokens, merge = cache[key]
            part_o = torch.empty(runs.shape[0], nq, d, dtype=torch.float32, device=q.device)
            part_ml = torch.empty(runs.shape[0], nq, 2, dtype=torch.float32, device=q.device)
            _lib.check(L.tff_attention_mfma_runs(
                q.data_ptr(), q.stride(0), out.data_ptr(), part_o.data_ptr(), part_ml.data_ptr(), k_cache.data_ptr(),
                v_cache.data_ptr(), bt.data_ptr(), bt.stride(0), batch.cu_tokens.data_ptr(), batch.start_pos.data_ptr(),
                runs.data_ptr(), run_start.data_ptr(), tokens.data_ptr(), runs.shape[0], len(single), 1 if merge else 0,
                T, nq, nkv, d, k_cache.shape[2], k_cache.shape[0], int(window), float(scale), stream))
        else:
            work = _attention_work(batch, G, 16, q.device, "single")
            if "single_rows" not in cache:
                cu = batch.host_cu_tokens
                cache["single_rows"] = _staging.send(q.device, [np.asarray([(r, cu[r]) for r in single], dtype=np.int32)])[0]
            sp = splits if splits is not None else pick_splits(work.shape[0] * nkv, batch.max_context)
            launch(work, work.shape[0], None, 0, 1, 16, sp, cache["single_rows"])
    if cols == 128:
        bcols = block_cols or _pick_block_cols(batch, G, nkv, int(window), q.device, which, d)
        if bcols == 256:
            # long prompts: items of 256 columns for blocks whose waves take two column tiles
            # each (one block a CU, so one bin a CU and kv head)
            per_cu = max(1, _num_cus(q.device) // max(1, nkv))
            work, block_items, num_blocks, _ = _attention_block_work(
                batch, G, nkv, int(window), q.device, cols=256, bins=block_bins or per_cu, which=which,
                key_groups=1, head_dim=d)
            launch(work, work.shape[0], block_items, num_blocks, 1, 256, 1, groups=1)
            return out
        work, block_items, num_blocks, groups = _attention_block_work(
            batch, G, nkv, int(window), q.device, bins=block_bins, which=which, key_groups=key_groups, head_dim=d)
        launch(work, work.shape[0], block_items, num_blocks, 1, 128, 1, groups=groups)
    else:
        work = _attention_work(batch, G, cols, q.device, which)
        launch(work, work.shape[0], None, 0, 1, cols, 1)
    return out


def decode_fused_supported(qkv: torch.Tensor, d: int, page_size: int, cos_sin, pairing: int, batch) -> bool:
    """Whether :func:`attention_decode_fused` takes this step: bfloat16, a head
    size of the matrix-core kernel, every entry one token, the whole head
    rotated (or none of it) with a pairing the kernel has in one lane."""
    if batch.max_new_tokens != 1 or not mfma_attention_supported(qkv.dtype, d, page_size):
        return False
    if cos_sin is None:
        return True
    return 2 * cos_sin.shape[1] == d and (pairing == 1 or d % 64 == 0)


def attention_decode_fused(qkv: torch.Tensor, nq: int, nkv: int, d: int, q_weight, k_weight, eps: float,
                           cos_sin, pairing: int, kv, batch, window: int = 0, scale: float | None = None,
                           slot_mapping: torch.Tensor | None = None, splits: int | None = None,
                           key_runs: torch.Tensor | None = None, run_start: torch.Tensor | None = None,
                           runs_for_blocks: bool = False, runs_merge: bool = True) -> torch.Tensor:
    """A decode-only step from the fused projection's output ``qkv`` [R, (nq +
    2 nkv) d]: q/k norm, rotation, the new keys and values into their pages and
    the attention over the pages, in one kernel (plus the merge of split keys).
    ``slot_mapping`` (int32 [R]) says which tokens' keys and values are written
    (entries >= 0; the place is the one the block table gives for the token's
    position); None: no token's, the pages hold them already.  ``key_runs``
    (int32 [runs, 4]: row, first key, end of keys, the row's position) and ``run_start`` (int32
    [R + 1]): the rows' keys dealt into runs by the host, a wave per run and
    kv head (``kernels.key_runs``), or a block of eight waves if they were
    dealt for that (``runs_for_blocks``) and the head size allows it;
    ``runs_merge`` False: the caller knows that every row is one run, and the
    kernel that merges partial results is left out.  Without runs every
    row's keys are split alike (``splits``)."""
    _req(qkv, "attention_decode_fused qkv", torch.bfloat16, 2)
    R = batch.num_reqs
    if qkv.shape[0] != R or batch.num_tokens != R or batch.max_new_tokens != 1:
        raise _lib.KernelError("attention_decode_fused: every entry of the step must bring one token")
    if qkv.shape[1] != (nq + 2 * nkv) * d:
        raise _lib.KernelError(
            f"attention_decode_fused: rows of {qkv.shape[1]} are not (nq + 2 nkv) d = {(nq + 2 * nkv) * d}")
    k_cache, v_cache = kv.k_cache, kv.v_cache
    _req(k_cache, "k cache", qkv.dtype, 4)
    _req(v_cache, "v cache", qkv.dtype, 4)
    _check_cache(k_cache, v_cache, nkv, d, "attention_decode_fused")
    bt = _req(kv.block_tables, "block tables", torch.int32, 2)
    _req(batch.cu_tokens, "cu_tokens", torch.int32, 1)
    _req(batch.start_pos, "start_pos", torch.int32, 1)
    if batch.cu_tokens.numel() != R + 1 or batch.start_pos.numel() != R or bt.shape[0] != R:
        raise _lib.KernelError("attention_decode_fused: the step's tables do not describe the same number of requests")
    for w, nm in ((q_weight, "q norm weight"), (k_weight, "k norm weight")):
        if w is not None:
            _req(w, nm, torch.float32, 1)
            if w.numel() != d:
                raise _lib.KernelError(f"{nm}: {w.numel()} elements, head size {d}")
    max_pos = 0
    if cos_sin is not None:
        _req(cos_sin, "rotation table", torch.float32, 3)
        max_pos = cos_sin.shape[0]
        if 2 * cos_sin.shape[1] != d or cos_sin.shape[2] != 2:
            raise _lib.KernelError(f"attention_decode_fused: a rotation table of shape {tuple(cos_sin.shape)} "
                                   f"does not rotate whole heads of {d}")
    if slot_mapping is not None:
        _req(slot_mapping, "slot_mapping", torch.int32, 1)
        if slot_mapping.numel() != R:
            raise _lib.KernelError("attention_decode_fused: slot_mapping needs one entry per token")
    G = nq // nkv
    tiles = -(-G // 16)
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    if key_runs is not None and splits is None:
        _req(key_runs, "key_runs", torch.int32, 2)
        _req(run_start, "run_start", torch.int32, 1)
        if key_runs.shape[1] != 4 or run_start.numel() != R + 1:
            raise _lib.KernelError(f"attention_decode_fused: runs of shape {tuple(key_runs.shape)} and "
                                   f"{run_start.numel()} run starts for {R} rows")
        P = key_runs.shape[0]
        out = torch.empty(R, nq * d, dtype=qkv.dtype, device=qkv.device)
        part_o = torch.empty(P, nq, d, dtype=torch.float32, device=qkv.device)
        part_ml = torch.empty(P, nq, 2, dtype=torch.float32, device=qkv.device)
        _lib.check(_lib.load().tff_attention_decode_runs(
            qkv.data_ptr(), qkv.stride(0), out.data_ptr(), part_o.data_ptr(), part_ml.data_ptr(), k_cache.data_ptr(),
            v_cache.data_ptr(), bt.data_ptr(), bt.stride(0), batch.cu_tokens.data_ptr(), batch.start_pos.data_ptr(),
            _ptr(slot_mapping), _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(cos_sin), max_pos, int(pairing),
            key_runs.data_ptr(), run_start.data_ptr(), P, 8 if (runs_for_blocks and d <= 128 and tiles == 1) else 1,
            1 if runs_merge else 0, R, nq, nkv, d, k_cache.shape[2], k_cache.shape[0],
            int(window), float(scale), _stream()))
        return out
    if splits is None:
        # entries x kv heads enough for a block each to saturate HBM between them: the keys of
        # an entry are split among the eight waves of its block and merged in LDS (splits 0)
        splits = 0 if (R * nkv >= BLOCK_DECODE_MIN_PAIRS and tiles == 1 and d <= 128) else \
            pick_splits(R * tiles * nkv, batch.max_context)
    out = torch.empty(R, nq * d, dtype=qkv.dtype, device=qkv.device)
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty(splits, R, nq, d, dtype=torch.float32, device=qkv.device)
        part_ml = torch.empty(splits, R, nq, 2, dtype=torch.float32, device=qkv.device)
    L = _lib.load()
    stream = _stream()
    _lib.check(L.tff_attention_decode_fused(
        qkv.data_ptr(), qkv.stride(0), out.data_ptr(), _ptr(part_o), _ptr(part_ml), k_cache.data_ptr(),
        v_cache.data_ptr(), bt.data_ptr(), bt.stride(0), batch.cu_tokens.data_ptr(), batch.start_pos.data_ptr(),
        _ptr(slot_mapping), _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(cos_sin), max_pos, int(pairing),
        splits, R, nq, nkv, d, k_cache.shape[2], k_cache.shape[0], int(window), float(scale), stream))
    if splits > 1:
        _lib.check(L.tff_attention_split_reduce(part_o.data_ptr(), part_ml.data_ptr(), out.data_ptr(), splits, R,
                                                nq, d, None, 0, stream))
    return out


def qkv_attention(qkv: torch.Tensor, nq: int, nkv: int, d: int, q_weight, k_weight, eps: float, cos_sin,
                  pairing: int, kv, batch, window: int = 0, scale: float | None = None) -> torch.Tensor:
    """From the fused projection's output to the attention's output [T, nq d]:
    q/k norm and rotation, the step's keys and values into the cache at
    ``kv.slot_mapping`` (negative entries: not written; the call reads a cache
    that another call fills, or the row is padding), attention over the cache.  Decode-only steps in bfloat16 are one kernel."""
    if decode_fused_supported(qkv, d, kv.k_cache.shape[2], cos_sin, pairing, batch):
        # (a call that only reads its cache, or a padding row, has negative slots)
        runs = getattr(kv, "key_runs", None)
        if runs is not None and kv.runs_window != int(window):
            runs = None       # dealt for another window than this call's
        return attention_decode_fused(qkv, nq, nkv, d, q_weight, k_weight, eps, cos_sin, pairing, kv, batch,
                                      window, scale, slot_mapping=kv.slot_mapping, key_runs=runs,
                                      run_start=kv.run_start if runs is not None else None,
                                      runs_for_blocks=runs is not None and kv.runs_for_blocks,
                                      runs_merge=runs is None or kv.runs_merge)
    qk_norm_rope_kv(qkv, nq, nkv, d, q_weight, k_weight, eps, cos_sin, pairing, batch.positions,
                    kv.slot_mapping, kv.k_cache, kv.v_cache)
    return paged_attention(qkv, nq, nkv, d, kv, batch, window, scale)


def paged_attention(q: torch.Tensor, nq: int, nkv: int, d: int, kv, batch, window: int = 0,
                    scale: float | None = None) -> torch.Tensor:
    """Attention of a step's tokens over the cache view ``kv`` (k_cache,
    v_cache, block_tables) with the step's ``batch``.  bfloat16 with a head
    size the matrix-core kernel takes runs there; everything else (float32,
    other head sizes) on the general kernel."""
    if mfma_attention_supported(q.dtype, d, kv.k_cache.shape[2]):
        return attention_mfma(q, nq, nkv, d, kv, batch, window, scale)
    return attention_generic(q, nq, nkv, d, kv.k_cache, kv.v_cache, kv.block_tables,
                             batch.token_req, batch.positions, window, scale)


def swiglu(gate_up: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """``silu(gate) * up`` for gate_up [T, 2I] = [gate | up]."""
    _req(gate_up, "swiglu input", ndim=2)
    T, two_i = gate_up.shape
    if two_i % 2:
        raise _lib.KernelError("swiglu: odd row width")
    I = two_i // 2
    if out is None:
        out = torch.empty(T, I, dtype=gate_up.dtype, device=gate_up.device)
    L = _lib.load()
    _lib.check(L.tff_swiglu(gate_up.data_ptr(), out.data_ptr(), T, I, dtype_code(gate_up.dtype), _stream()))
    return out


def cast(src: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    _req(src, "cast src")
    out = torch.empty(src.shape, dtype=dtype, device=src.device)
    L = _lib.load()
    _lib.check(L.tff_cast(src.data_ptr(), dtype_code(src.dtype), out.data_ptr(), dtype_code(dtype),
                          src.numel(), _stream()))
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """Lowest index among the maxima of each row of float32 logits [R, V]."""
    _req(logits, "argmax logits", torch.float32, 2)
    R, V = logits.shape
    out = torch.empty(R, dtype=torch.int32, device=logits.device)
    L = _lib.load()
    ws_bytes = L.tff_argmax_workspace_bytes(R, V)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=logits.device) if ws_bytes else None
    _lib.check(L.tff_argmax(logits.data_ptr(), out.data_ptr(), R, V, _ptr(ws), _stream()))
    return out


def repetition_penalty(logits: torch.Tensor, seen: torch.Tensor, cu_seen: torch.Tensor,
                       penalty: torch.Tensor) -> None:
    _req(logits, "repetition_penalty logits", torch.float32, 2)
    R, V = logits.shape
    _req(seen, "seen", torch.int32, 1)
    _req(cu_seen, "cu_seen", torch.int32, 1)
    _req(penalty, "penalty", torch.float32, 1)
    if cu_seen.numel() != R + 1 or penalty.numel() != R:
        raise _lib.KernelError("repetition_penalty: cu_seen needs rows + 1 entries, penalty one per row")
    L = _lib.load()
    _lib.check(L.tff_repetition_penalty(logits.data_ptr(), R, V, seen.data_ptr(), cu_seen.data_ptr(),
                                        penalty.data_ptr(), _stream()))


def sample(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
           top_k: torch.Tensor | None = None, top_p: torch.Tensor | None = None,
           min_p: torch.Tensor | None = None, return_probs: bool = False):
    """One token per row of float32 logits [R, V]; see the entry point."""
    _req(logits, "sample logits", torch.float32, 2)
    R, V = logits.shape
    _req(temperature, "temperature", torch.float32, 1)
    _req(uniform, "uniform", torch.float32, 1)
    for t, nm, dt in ((top_k, "top_k", torch.int32), (top_p, "top_p", torch.float32),
                      (min_p, "min_p", torch.float32)):
        if t is not None:
            _req(t, nm, dt, 1)
            if t.numel() != R:
                raise _lib.KernelError(f"sample: {nm} needs one entry per row")
    if temperature.numel() != R or uniform.numel() != R:
        raise _lib.KernelError("sample: temperature and uniform need one entry per row")
    out = torch.empty(R, dtype=torch.int32, device=logits.device)
    probs = torch.empty(R, V, dtype=torch.float32, device=logits.device) if return_probs else None
    L = _lib.load()
    _lib.check(L.tff_sample(logits.data_ptr(), out.data_ptr(), R, V, temperature.data_ptr(),
                            _ptr(top_k), _ptr(top_p), _ptr(min_p), uniform.data_ptr(), _ptr(probs),
                            _stream()))
    return (out, probs) if return_probs else out


def measure_ceilings(device="cuda:0", gib: float = 4.0, quick: bool = False) -> dict:
    """What this machine gives to kernels that do nothing else: streaming reads
    from HBM into registers (a buffer of ``gib`` GiB, far larger than the
    caches) and back-to-back bfloat16 MFMAs at 1, 2 and 4 waves per SIMD, with
    operands that never change and (``..._varied_operands``) with operands that
    change from one instruction to the next as a real product's do: the matrix
    cores then draw more power and the clock settles lower.  ``quick``: the
    streaming read and the four-wave MFMA figure only (some 50 ms)."""
    L = _lib.load()
    dev = torch.device(device)
    cus = _num_cus(dev)
    sink = torch.zeros(4, dtype=torch.float32, device=dev)
    buf = torch.empty(int(gib * (1 << 30)) // 4, dtype=torch.int32, device=dev).fill_(1)
    nbytes = buf.numel() * 4

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize(dev)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize(dev)
        return e0.elapsed_time(e1) / 1e3 / reps

    out = {"compute_units": cus}
    with torch.cuda.device(dev):
        st = _stream()
        t = min(timed(lambda: _lib.check(L.tff_probe_stream_read(buf.data_ptr(), nbytes, sink.data_ptr(), cus * b, st)), 3)
                for b in (8, 16, 32))
        out["stream_read_GBps"] = round(nbytes / t / 1e9, 1)
        iters = 20000
        for waves in ((4,) if quick else (1, 2, 4)):
            t = timed(lambda: _lib.check(L.tff_probe_mfma(sink.data_ptr(), cus * waves, iters, 0, st)), 2)
            out[f"mfma_bf16_TFLOPs_{waves}_waves_per_simd"] = round(cus * waves * 4 * iters * 16 * 16384 / t / 1e12, 1)
        if quick:
            return out
        iters = 100000   # long enough for the clock to settle
        t = timed(lambda: _lib.check(L.tff_probe_mfma(sink.data_ptr(), cus * 4, iters, 1, st)), 2)
        out["mfma_bf16_TFLOPs_varied_operands"] = round(cus * 4 * 4 * iters * 16 * 16384 / t / 1e12, 1)
    return out


OP_TABLE = {
    "embed": embed,
    "add_rmsnorm": add_rmsnorm,
    "rmsnorm": rmsnorm,
    "linear": linear,
    "as_tensor": as_tensor,
    "pack_weight": pack_weight,
    "qk_norm_rope_kv": qk_norm_rope_kv,
    "attention": paged_attention,
    "attention_generic": attention_generic,
    "attention_mfma": attention_mfma,
    "attention_decode_fused": attention_decode_fused,
    "qkv_attention": qkv_attention,
    "swiglu": swiglu,
    "cast": cast,
    "argmax": argmax,
    "repetition_penalty": repetition_penalty,
    "sample": sample,
}
