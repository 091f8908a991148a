"""Pins the plain implementation by what fixes it beside the reference's text:
special cases that reduce to a library routine, and invariants, each chosen so
that a plausible mistake fails it.  The reference holds no test vectors of its
own (its only test is an end-to-end program whose output is read by eye,
test/main.cu:17-66), so parity with it beyond these is unpinned."""
import math

import pytest
import torch

import plain_qwen3 as P
from helpers import TINY_A, TINY_B, make_model_dir, random_tokens

torch.manual_seed(0)


# ---- rmsnorm ---------------------------------------------------------------
def test_rmsnorm_closed_form_and_eps_inside_root_on_mean():
    x = torch.randn(5, 24, dtype=torch.float64)
    w = torch.ones(24, dtype=torch.float64)
    eps = 0.37
    y = P.plain_rmsnorm(x, w, eps)
    n = 24
    ss = (x * x).sum(-1)
    # ||y||^2 = n ||x||^2 / (||x||^2 + n eps): wrong if eps is added to the sum or outside the root
    assert torch.allclose((y * y).sum(-1), n * ss / (ss + n * eps), rtol=1e-12)


def test_rmsnorm_weight_multiplies_directly():
    x = torch.randn(3, 8, dtype=torch.float64)
    w = torch.zeros(8, dtype=torch.float64)
    assert torch.equal(P.plain_rmsnorm(x, w, 1e-6), torch.zeros_like(x))  # (1 + w) would give x / rms
    w2 = torch.full((8,), 2.0, dtype=torch.float64)
    assert torch.allclose(P.plain_rmsnorm(x, w2, 1e-6), 2 * P.plain_rmsnorm(x, torch.ones(8, dtype=torch.float64), 1e-6))


def test_rmsnorm_scale_invariance():
    x = torch.randn(4, 16, dtype=torch.float64)
    w = torch.rand(16, dtype=torch.float64)
    assert torch.allclose(P.plain_rmsnorm(7.0 * x, w, 1e-30), P.plain_rmsnorm(x, w, 1e-30), rtol=1e-10)


# ---- linear ----------------------------------------------------------------
def test_linear_is_x_wt():
    x = torch.randn(5, 7, dtype=torch.float64)
    w = torch.randn(3, 7, dtype=torch.float64)     # [out, in], non-square
    assert torch.allclose(P.plain_linear(x, w), x @ w.T, rtol=1e-12)
    assert torch.allclose(P.plain_linear(x, torch.eye(7, dtype=torch.float64)), x)


# ---- rope ------------------------------------------------------------------
def test_rope_position_zero_is_identity_and_norm_preserved():
    x = torch.randn(3, 2, 16, dtype=torch.float64)
    assert torch.allclose(P.plain_rope_neox(x, [0, 0, 0], 1e4), x)
    y = P.plain_rope_neox(x, [5, 77, 1000], 1e4)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), rtol=1e-12)


def test_rope_pairing_and_sign_by_one_hot():
    d = 8
    x = torch.zeros(1, 1, d, dtype=torch.float64)
    x[0, 0, 1] = 1.0                      # element 1 pairs with 1 + d/2 = 5 (not with 0 or 2)
    y = P.plain_rope_neox(x, [3], 100.0)
    ang = 3 * 100.0 ** (-2 * 1 / d)
    want = torch.zeros(d, dtype=torch.float64)
    want[1], want[5] = math.cos(ang), math.sin(ang)   # +sin in the upper half: a wrong sign flips it
    assert torch.allclose(y[0, 0], want, atol=1e-12)
    yi = P.plain_rope_interleaved(x, [3], 100.0)      # element 1 is the odd half of pair 0
    wi = torch.zeros(d, dtype=torch.float64)
    wi[0], wi[1] = -math.sin(3.0), math.cos(3.0)
    assert torch.allclose(yi[0, 0], wi, atol=1e-12)


def test_rope_scores_depend_on_distance_only():
    q = torch.randn(1, 1, 32, dtype=torch.float64)
    k = torch.randn(1, 1, 32, dtype=torch.float64)

    def score(m, n):
        return (P.plain_rope_neox(q, [m], 1e6) * P.plain_rope_neox(k, [n], 1e6)).sum()

    assert abs(score(10, 3) - score(110, 103)) < 1e-10
    assert abs(score(10, 3) - score(10, 4)) > 1e-6


def test_rope_angles_closed_form():
    a = P.plain_rope_angles([7], 16, 1e4)
    for i in range(8):
        assert abs(float(a[0, i]) - 7 * 1e4 ** (-2 * i / 16)) < 1e-12


# ---- attention ---------------------------------------------------------------
def test_attention_reduces_to_library_softmax():
    T, nq, d = 6, 3, 8
    q = torch.randn(T, nq, d, dtype=torch.float64)
    k = torch.randn(T, nq, d, dtype=torch.float64)
    v = torch.randn(T, nq, d, dtype=torch.float64)
    out = P.plain_attention(q, k, v, list(range(T)))
    s = torch.einsum("thd,jhd->htj", q, k) / math.sqrt(d)
    s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1)[None], float("-inf"))
    ref = torch.einsum("htj,jhd->thd", torch.softmax(s, -1), v)
    assert torch.allclose(out, ref, rtol=1e-10)


def test_attention_against_the_library_routine_with_groups_and_a_causal_mask():
    """torch's own attention routine (no model code: one function of the tensor library), with
    its causal mask and its grouping of query heads over key heads: scale 1/sqrt(d), which way
    the mask faces, and q head h reading kv head h // (nq / nkv) in one comparison."""
    F = torch.nn.functional
    if "enable_gqa" not in (F.scaled_dot_product_attention.__doc__ or ""):
        pytest.skip("this torch's attention routine has no grouped heads")
    T, nq, nkv, d = 7, 6, 2, 8
    q = torch.randn(T, nq, d, dtype=torch.float64)
    k = torch.randn(T, nkv, d, dtype=torch.float64)
    v = torch.randn(T, nkv, d, dtype=torch.float64)
    out = P.plain_attention(q, k, v, list(range(T)))
    ref = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                         is_causal=True, enable_gqa=True)[0].transpose(0, 1)
    assert torch.allclose(out, ref, rtol=1e-10, atol=1e-12)


def test_rmsnorm_against_the_library_routine():
    x = torch.randn(5, 24, dtype=torch.float64) * 3.0
    w = torch.rand(24, dtype=torch.float64) + 0.5
    if not hasattr(torch.nn.functional, "rms_norm"):
        pytest.skip("this torch has no rms_norm routine")
    for eps in (1e-6, 0.3):     # an eps large enough that its place (inside the root, on the mean) shows
        ref = torch.nn.functional.rms_norm(x, (24,), w, eps)
        assert torch.allclose(P.plain_rmsnorm(x, w, eps), ref, rtol=1e-12)


def test_attention_single_key_and_uniform_scores():
    d = 4
    q = torch.randn(1, 2, d, dtype=torch.float64)
    k = torch.randn(1, 1, d, dtype=torch.float64)
    v = torch.randn(1, 1, d, dtype=torch.float64)
    out = P.plain_attention(q, k, v, [0])
    assert torch.allclose(out[0, 0], v[0, 0]) and torch.allclose(out[0, 1], v[0, 0])
    k0 = torch.zeros(5, 1, d, dtype=torch.float64)
    v5 = torch.randn(5, 1, d, dtype=torch.float64)
    out = P.plain_attention(q, k0, v5, [4])
    assert torch.allclose(out[0, 0], v5[:, 0].mean(0))


def test_attention_group_mapping_and_causality_and_window():
    nq, nkv, d, N = 4, 2, 4, 6
    q = torch.randn(N, nq, d, dtype=torch.float64)
    k = torch.randn(N, nkv, d, dtype=torch.float64)
    v = torch.zeros(N, nkv, d, dtype=torch.float64)
    v[:, 0] = 1.0
    v[:, 1] = 2.0
    out = P.plain_attention(q, k, v, list(range(N)))
    assert torch.allclose(out[:, :2], torch.ones(N, 2, d, dtype=torch.float64))   # heads 0,1 -> kv 0
    assert torch.allclose(out[:, 2:], torch.full((N, 2, d), 2.0, dtype=torch.float64))
    v = torch.randn(N, nkv, d, dtype=torch.float64)
    a = P.plain_attention(q, k, v, list(range(N)))
    k2, v2 = k.clone(), v.clone()
    k2[4:] += 5.0
    v2[4:] -= 3.0
    b = P.plain_attention(q, k2, v2, list(range(N)))
    assert torch.allclose(a[:4], b[:4]) and not torch.allclose(a[4:], b[4:])
    # window 2: the query at 5 sees keys 4 and 5 only
    w = P.plain_attention(q[5:], k, v, [5], window=2)
    w_ref = P.plain_attention(q[5:], k[4:], v[4:], [1])
    assert torch.allclose(w, w_ref)


# ---- swiglu ------------------------------------------------------------------
def test_silu_and_roles():
    assert float(P.plain_silu(torch.tensor(0.0, dtype=torch.float64))) == 0.0
    assert abs(float(P.plain_silu(torch.tensor(40.0, dtype=torch.float64))) - 40.0) < 1e-9
    x = torch.tensor(1.7, dtype=torch.float64)
    assert abs(float(P.plain_silu(-x)) + float(x) / (1 + math.exp(float(x)))) < 1e-12
    z = torch.randn(2, 6, dtype=torch.float64)
    wg = torch.randn(5, 6, dtype=torch.float64)
    wu = torch.randn(5, 6, dtype=torch.float64)
    wd = torch.randn(6, 5, dtype=torch.float64)
    ref = (torch.nn.functional.silu(z @ wg.T) * (z @ wu.T)) @ wd.T
    assert torch.allclose(P.plain_swiglu_mlp(z, wg, wu, wd), ref, rtol=1e-10)
    # the gate goes through silu, not the up projection: silu(g) * u != g * silu(u)
    swapped = P.plain_swiglu_mlp(z, wu, wg, wd)
    assert not torch.allclose(swapped, ref)


# ---- whole model -------------------------------------------------------------
@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("plain")
    return {"A": make_model_dir(str(base / "A"), TINY_A, 3), "B": make_model_dir(str(base / "B"), TINY_B, 4)}


@pytest.mark.parametrize("name", ["A", "B"])
def test_fast_forward_equals_plain_forward(dirs, name):
    cfg, raw = P.load_plain_model(dirs[name])
    toks = random_tokens(30 if name == "B" else 12, cfg["vocab_size"], 9)   # B: longer than its window of 24
    a = P.plain_forward(cfg, raw, toks)
    b = P.fast_forward(cfg, raw, toks)
    assert float((a - b).abs().max()) < 1e-10 * float(a.abs().max()) + 1e-12


def test_identity_layers_give_norm_of_embedding_times_head(dirs):
    cfg, raw = P.load_plain_model(dirs["B"])
    raw = dict(raw)
    for i in range(cfg["num_hidden_layers"]):
        raw[f"model.layers.{i}.self_attn.o_proj.weight"] = torch.zeros_like(raw[f"model.layers.{i}.self_attn.o_proj.weight"])
        raw[f"model.layers.{i}.mlp.down_proj.weight"] = torch.zeros_like(raw[f"model.layers.{i}.mlp.down_proj.weight"])
    toks = [5, 9, 200]
    out = P.plain_forward(cfg, raw, toks)
    x = raw["model.embed_tokens.weight"][toks]
    y = P.plain_rmsnorm(x, raw["model.norm.weight"], cfg["rms_norm_eps"])
    assert torch.allclose(out, y @ raw["lm_head.weight"].T, rtol=1e-10)


def test_qk_norm_stands_before_rotation(dirs):
    """With a non-constant norm weight, norm-then-rotate differs from
    rotate-then-norm; the plain block must be the former."""
    cfg, raw = P.load_plain_model(dirs["A"])
    lw = P._layer_weights(raw, 0)
    x = torch.randn(4, cfg["hidden_size"], dtype=torch.float64)
    pos = [0, 1, 2, 3]
    got = P.plain_attention_block(x, pos, lw, cfg, 0)
    nq, nkv, d = 4, 2, 16
    q = P.plain_linear(x, lw["q_proj"]).reshape(4, nq, d)
    k = P.plain_linear(x, lw["k_proj"]).reshape(4, nkv, d)
    v = P.plain_linear(x, lw["v_proj"]).reshape(4, nkv, d)
    q_wrong = P.plain_rmsnorm(P.plain_rope_neox(q, pos, cfg["rope_theta"]), lw["q_norm"], cfg["rms_norm_eps"])
    k_wrong = P.plain_rmsnorm(P.plain_rope_neox(k, pos, cfg["rope_theta"]), lw["k_norm"], cfg["rms_norm_eps"])
    wrong = P.plain_linear(P.plain_attention(q_wrong, k_wrong, v, pos).reshape(4, nq * d), lw["o_proj"])
    assert not torch.allclose(got, wrong, rtol=1e-6)


def test_shift_of_all_positions_leaves_attention_unchanged():
    """Only distances count: q and k rotated at p + s give the same scores."""
    q = torch.randn(5, 2, 16, dtype=torch.float64)
    k = torch.randn(5, 2, 16, dtype=torch.float64)
    v = torch.randn(5, 2, 16, dtype=torch.float64)
    pos = list(range(5))

    def run(shift):
        p = [x + shift for x in pos]
        return P.plain_attention(P.plain_rope_neox(q, p, 1e4), P.plain_rope_neox(k, p, 1e4), v, pos)

    assert torch.allclose(run(0), run(37), rtol=1e-9)


def test_tied_head_uses_embedding(dirs):
    cfg, raw = P.load_plain_model(dirs["A"])
    assert cfg["tie_word_embeddings"] and "lm_head.weight" not in raw
    out = P.plain_forward(cfg, raw, [1, 2])
    assert out.shape == (2, cfg["vocab_size"])


def test_layer_windows_rule():
    assert P.layer_windows(TINY_A) == [0, 0]
    assert P.layer_windows(TINY_B) == [0, 24, 24]
    c = dict(TINY_B, layer_types=["sliding_attention", "full_attention", "sliding_attention"])
    assert P.layer_windows(c) == [24, 0, 24]


# ---- sampling ----------------------------------------------------------------
def test_greedy_first_maximum():
    assert P.plain_greedy(torch.tensor([0.0, 3.0, 3.0, 1.0])) == 1


def test_probs_filters():
    logits = torch.log(torch.tensor([0.5, 0.25, 0.15, 0.1]))
    assert torch.allclose(P.plain_probs(logits, 1.0), torch.tensor([0.5, 0.25, 0.15, 0.1], dtype=torch.float64))
    assert torch.allclose(P.plain_probs(logits, 1.0, top_k=2), torch.tensor([2 / 3, 1 / 3, 0, 0], dtype=torch.float64))
    assert torch.allclose(P.plain_probs(logits, 1.0, top_p=0.7), torch.tensor([2 / 3, 1 / 3, 0, 0], dtype=torch.float64))
    assert torch.allclose(P.plain_probs(logits, 1.0, min_p=0.4), torch.tensor([2 / 3, 1 / 3, 0, 0], dtype=torch.float64))
    cold = P.plain_probs(logits, 0.01)
    assert cold[0] > 0.999
    assert P.plain_inverse_cdf(torch.tensor([0.5, 0.25, 0.25]), 0.49) == 0
    assert P.plain_inverse_cdf(torch.tensor([0.5, 0.25, 0.25]), 0.5) == 1
    assert P.plain_inverse_cdf(torch.tensor([0.5, 0.0, 0.5]), 0.999) == 2
