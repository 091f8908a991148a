"""Each part of a layer alone against the plain functions, at sizes of its own."""
import math

import pytest
import torch

import plain_qwen3 as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ctx(cache, entries, act_dtype, max_positions=512, cache_id=0, writes=True):
    from tffinfer_amd.engine.batch import KVView, build_step_batch
    from tffinfer_amd.engine.runner import LayerContext
    from tffinfer_amd.kernels import ops
    for e in entries:
        if not cache.has_request(e.req):
            cache.add_request(e.req)
        cache.reserve(e.req, len(e.tokens))
    batch = build_step_batch(entries, cache, DEV)
    ctx = LayerContext(ops, act_dtype, batch, max_positions)
    gi = cache.group_index(cache_id)
    if gi is not None:
        k, v = cache.kv_tensors(cache_id)
        gt = batch.groups[gi]
        ctx.kv = KVView(k, v, gt.block_tables, gt.slot_mapping if writes else gt.no_slot_mapping,
                        cache.page_size, gi)
    return ctx


def _err(got, ref):
    from tffinfer_amd.kernels import ops
    # a part may return what only the norm after it understands: partial sums, a product not yet run
    got, ref = ops.as_tensor(got).double().cpu(), ref.double().cpu()
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 8e-3)])
def test_rmsnorm_part(dtype, tol):
    from tffinfer_amd.engine.runner import LayerContext
    from tffinfer_amd.kernels import ops
    from tffinfer_amd.parts import RMSNorm
    n = RMSNorm(size=72, eps=1e-4)
    assert n.weight_specs()["weight"].shape == (72,)
    w = 1 + 0.1 * torch.randn(72)
    n.load_weights({"weight": w.to(torch.bfloat16 if dtype == torch.bfloat16 else torch.float32)}, dtype, DEV)
    assert n.weight.dtype == torch.float32
    ctx = LayerContext(ops, dtype, None, 0)
    resid = torch.randn(5, 72)
    delta = torch.randn(5, 72)
    r = resid.to(DEV).clone()
    y = n.forward(ctx, r, delta.to(DEV))
    assert y.dtype == dtype
    ref = P.plain_rmsnorm((resid + delta).double(), n.weight.double().cpu(), 1e-4)
    assert _err(y, ref) < tol
    assert _err(r, resid + delta) < 1e-6


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 2e-2)])
def test_swiglu_part(dtype, tol):
    from tffinfer_amd.engine.runner import LayerContext
    from tffinfer_amd.kernels import ops
    from tffinfer_amd.parts import SwiGLU
    H, I = 48, 104
    ff = SwiGLU(hidden_size=H, intermediate_size=I)
    assert {k: v.shape for k, v in ff.weight_specs().items()} == {
        "gate_proj.weight": (I, H), "up_proj.weight": (I, H), "down_proj.weight": (H, I)}
    w = {k: (torch.randn(s.shape) * 0.2).to(torch.bfloat16) for k, s in ff.weight_specs().items()}
    ff.load_weights(w, dtype, DEV)
    x = torch.randn(6, H).to(dtype)
    out = ops.as_tensor(ff.forward(LayerContext(ops, dtype, None, 0), x.to(DEV)))
    assert out.dtype == torch.float32
    ref = P.plain_swiglu_mlp(x.double(), w["gate_proj.weight"].double(), w["up_proj.weight"].double(),
                             w["down_proj.weight"].double())
    assert _err(out, ref) < tol


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("window", [0, 10])
def test_attention_part_whole_and_in_two_steps(dtype, tol, window):
    """The mixer alone: a whole sequence in one step, then the same sequence as
    a portion of 11 and a portion of the rest; both equal the plain block."""
    from tffinfer_amd.cache import CacheManager
    from tffinfer_amd.config.base import PartSpec
    from tffinfer_amd.engine.batch import StepEntry
    from tffinfer_amd.parts import GQAttention
    H, nq, nkv, d, theta, eps = 40, 6, 3, 16, 3000.0, 1e-4
    att = GQAttention(hidden_size=H, num_heads=nq, num_kv_heads=nkv, head_dim=d, qk_norm_eps=eps, window=window,
                      position=PartSpec("rope", {"head_dim": d, "theta": theta}))
    g = torch.Generator().manual_seed(3)
    w = {}
    for k, s in att.weight_specs().items():
        t = torch.randn(s.shape, generator=g)
        w[k] = (1 + 0.1 * t) if s.init == "norm" else (t * 0.3).to(torch.bfloat16)
    att.load_weights(w, dtype, DEV)
    T = 29
    x = torch.randn(T, H, generator=g).to(dtype)
    lw = {k.split(".")[0]: v.double() for k, v in w.items()}
    cfg = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": d, "hidden_size": H,
           "rms_norm_eps": eps, "rope_theta": theta}
    ref = P.plain_attention_block(x.double(), list(range(T)), lw, cfg, window)
    reqs = [(0, True, att.cache_spec(), None)]
    toks = [0] * T
    cache = CacheManager(reqs, 8, 8, 2, dtype=dtype, device=DEV)
    ctx = _ctx(cache, [StepEntry("w", toks, [])], dtype)
    out = att.forward(ctx, x.to(DEV))
    assert _err(out, ref) < tol
    cache.commit("w", T)
    ctx = _ctx(cache, [StepEntry("p", toks[:11], [])], dtype)
    o1 = att.forward(ctx, x[:11].to(DEV))
    cache.commit("p", 11)
    ctx = _ctx(cache, [StepEntry("p", toks[11:], [])], dtype)
    o2 = att.forward(ctx, x[11:].to(DEV))
    from tffinfer_amd.kernels import ops
    assert _err(torch.cat([ops.as_tensor(o1), ops.as_tensor(o2)]), ref) < tol


def test_attention_part_without_norm_or_position_is_plain_attention():
    from tffinfer_amd.cache import CacheManager
    from tffinfer_amd.engine.batch import StepEntry
    from tffinfer_amd.parts import GQAttention
    H, nq, d = 32, 2, 16
    att = GQAttention(hidden_size=H, num_heads=nq, num_kv_heads=nq, head_dim=d, qk_norm_eps=None, position=None)
    assert set(att.weight_specs()) == {"q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight"}
    eye = torch.eye(H)
    att.load_weights({"q_proj.weight": eye, "k_proj.weight": eye, "v_proj.weight": eye, "o_proj.weight": eye},
                     torch.float32, DEV)
    T = 7
    x = torch.randn(T, H)
    cache = CacheManager([(0, True, att.cache_spec(), None)], 8, 4, 1, dtype=torch.float32, device=DEV)
    out = att.forward(_ctx(cache, [StepEntry("r", [0] * T, [])], torch.float32), x.to(DEV))
    q = x.reshape(T, nq, d).transpose(0, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(q, q, q, is_causal=True).transpose(0, 1).reshape(T, H)
    assert _err(out, ref) < 3e-6


@pytest.mark.parametrize("T", [13, 29])   # up to 16 bfloat16 rows the norms are taken into the products
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 2e-2)])
def test_prenorm_block(dtype, tol, T):
    from tffinfer_amd.cache import CacheManager
    from tffinfer_amd.config.base import PartSpec
    from tffinfer_amd.engine.batch import StepEntry
    from tffinfer_amd.kernels import ops
    from tffinfer_amd.parts import GQAttention, PreNormBlock, RMSNorm, SwiGLU
    H, nq, nkv, d, I, eps, theta = 48, 4, 1, 16, 72, 1e-5, 1e4
    att = GQAttention(hidden_size=H, num_heads=nq, num_kv_heads=nkv, head_dim=d, qk_norm_eps=eps,
                      position=PartSpec("rope", {"head_dim": d, "theta": theta}))
    blk = PreNormBlock(att, SwiGLU(H, I), lambda: RMSNorm(H, eps))
    assert list(blk.children()) == ["norm1", "mixer", "norm2", "feed_forward"]
    g = torch.Generator().manual_seed(8)
    lw = {}
    for cname, part in blk.children().items():
        ws = {}
        for k, s in part.weight_specs().items():
            t = torch.randn(s.shape, generator=g)
            ws[k] = (1 + 0.1 * t) if s.init == "norm" else (t * 0.2).to(torch.bfloat16)
            lw[(cname, k)] = ws[k].double()
        part.load_weights(ws, dtype, DEV)
    x = torch.randn(T, H, generator=g)
    pending = torch.randn(T, H, generator=g) * 0.1
    plain_lw = {
        "input_layernorm": lw[("norm1", "weight")], "post_attention_layernorm": lw[("norm2", "weight")],
        "q_proj": lw[("mixer", "q_proj.weight")], "k_proj": lw[("mixer", "k_proj.weight")],
        "v_proj": lw[("mixer", "v_proj.weight")], "o_proj": lw[("mixer", "o_proj.weight")],
        "q_norm": lw[("mixer", "q_norm.weight")], "k_norm": lw[("mixer", "k_norm.weight")],
        "gate_proj": lw[("feed_forward", "gate_proj.weight")], "up_proj": lw[("feed_forward", "up_proj.weight")],
        "down_proj": lw[("feed_forward", "down_proj.weight")],
    }
    cfg = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": d, "hidden_size": H,
           "rms_norm_eps": eps, "rope_theta": theta}
    ref = P.plain_decoder_layer((x + pending).double(), list(range(T)), plain_lw, cfg, 0)
    cache = CacheManager([(0, True, att.cache_spec(), None)], 8, 4, 1, dtype=dtype, device=DEV)
    ctx = _ctx(cache, [StepEntry("r", [0] * T, [])], dtype)
    resid = x.to(DEV).clone()
    out_pending = ops.as_tensor(blk.forward(ctx, resid, pending.to(DEV)))
    assert _err(resid + out_pending, ref) < tol


def test_embedding_and_tied_head():
    from tffinfer_amd.engine.runner import LayerContext
    from tffinfer_amd.kernels import ops
    from tffinfer_amd.parts import Embedding, OutputHead
    emb = Embedding(50, 24)
    head = OutputHead(50, 24, tied_to=emb)
    assert head.weight_specs() == {}
    table = torch.randn(50, 24).to(torch.bfloat16)
    emb.load_weights({"weight": table}, torch.bfloat16, DEV)
    assert head.weight.data_ptr() == emb.weight.data_ptr()     # one allocation
    ctx = LayerContext(ops, torch.bfloat16, None, 0)
    ids = torch.tensor([3, 49, 0], dtype=torch.int32, device=DEV)
    x = emb.forward(ctx, ids)
    assert torch.equal(x.cpu(), table.float()[[3, 49, 0]])
    logits = head.forward(ctx, x.to(torch.bfloat16))
    assert logits.dtype == torch.float32 and logits.shape == (3, 50)
    assert _err(logits, table.double()[[3, 49, 0]] @ table.double().T) < 1e-5
    free = OutputHead(50, 24, tied_to=None)
    assert free.weight_specs()["weight"].shape == (50, 24)


def test_rotary_table_closed_form():
    from tffinfer_amd.parts import RotaryEmbedding
    r = RotaryEmbedding(head_dim=32, theta=1e6)
    t = r.table(100, DEV).cpu()
    assert t.shape == (100, 16, 2)
    for pos, i in ((0, 0), (1, 0), (7, 3), (99, 15)):
        ang = pos * 1e6 ** (-2 * i / 32)
        assert abs(float(t[pos, i, 0]) - math.cos(ang)) < 1e-6 and abs(float(t[pos, i, 1]) - math.sin(ang)) < 1e-6
