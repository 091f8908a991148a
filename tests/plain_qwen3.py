"""Plain, slow implementation of the Qwen3 dense decoder, used only by tests.

Whole sequences, no cache, no batching, one function per part.  It shares no
code with the package: it reads ``config.json`` with ``json`` and the weights
with the ``safetensors`` library, and computes with element-level torch
arithmetic in float64 by default.  Every function cites the place in the
reference (paths relative to the reference's root) whose formula it follows.
The reference was read, not run.
"""
from __future__ import annotations

import json
import math
import os

import torch


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------

def plain_embedding(table: torch.Tensor, token_ids) -> torch.Tensor:
    """x[t, :] = E[token[t], :]; no scaling.

    src/kernel/cpu/embedding.cpp:34-49 (row lookup),
    src/core/model/qwen3/QWen3Creator.cpp:283-321 (wired as the first node).
    """
    rows = [table[int(t)].clone() for t in token_ids]
    return torch.stack(rows, 0)


def plain_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y_j = x_j * rsqrt(mean_j(x_j^2) + eps) * w_j over the last dimension.

    src/kernel/cuda/norm.cu:31-48: sum of squares, ``mean = sum / dim0``,
    ``rms = rsqrtf(mean + eps)``, ``dst = src * rms * weight[d]`` (weight
    multiplies directly, no ``1 + w``).
    """
    n = x.shape[-1]
    ss = (x * x).sum(-1, keepdim=True)
    mean = ss / n
    r = 1.0 / torch.sqrt(mean + eps)
    return x * r * weight


def plain_linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """y = x . W^T with W stored [out, in]; no bias.

    src/core/graph/op/TFFOPNode.h:95-101 (out = weight.shape[1], fp32 result),
    src/core/model/qwen3/QWen3Creator.cpp:66-75,332-337 (q/k/v as three
    separate products), src/core/model/base/ModelCreatorBase.cpp:121-176.
    """
    out_features, in_features = weight.shape
    assert x.shape[-1] == in_features
    y = torch.zeros(*x.shape[:-1], out_features, dtype=x.dtype)
    for o in range(out_features):
        y[..., o] = (x * weight[o]).sum(-1)
    return y


def plain_rope_angles(positions, head_dim: int, theta: float) -> torch.Tensor:
    """angle[pos, i] = pos * exp(-(2 i / d) * ln(theta)), i in [0, d/2).

    src/kernel/cuda/rope_table.cu:32-36.
    """
    half = head_dim // 2
    out = torch.zeros(len(positions), half, dtype=torch.float64)
    log_base = math.log(theta)
    for r, pos in enumerate(positions):
        for i in range(half):
            out[r, i] = float(pos) * math.exp(-(2.0 * i) / head_dim * log_base)
    return out


def plain_rope_neox(x: torch.Tensor, positions, theta: float) -> torch.Tensor:
    """Rotate-half pairing (i, i + d/2) over the full head dimension.

    x: [T, heads, d].  x'_i = x_i cos - x_{i+d/2} sin;
    x'_{i+d/2} = x_i sin + x_{i+d/2} cos.
    src/kernel/cuda/paged_flash_attention.cu:343-355 (K), :386-451 (Q);
    the table entry is (cos, sin), src/kernel/cuda/rope_table.cu:35-36.
    """
    T, _, d = x.shape
    half = d // 2
    ang = plain_rope_angles(positions, d, theta).to(x.dtype)
    cos = torch.cos(ang)[:, None, :]
    sin = torch.sin(ang)[:, None, :]
    lo = x[..., :half]
    hi = x[..., half:]
    out = torch.empty_like(x)
    out[..., :half] = lo * cos - hi * sin
    out[..., half:] = lo * sin + hi * cos
    return out


def plain_rope_interleaved(x: torch.Tensor, positions, theta: float) -> torch.Tensor:
    """Pairs (2i, 2i+1) rotated as a complex product with (cos, sin).

    The reference's rope type 0, src/kernel/cuda/paged_flash_attention.cu:175-195.
    """
    T, _, d = x.shape
    ang = plain_rope_angles(positions, d, theta).to(x.dtype)
    cos = torch.cos(ang)[:, None, :]
    sin = torch.sin(ang)[:, None, :]
    ev = x[..., 0::2]
    od = x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = ev * cos - od * sin
    out[..., 1::2] = ev * sin + od * cos
    return out


def plain_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                    q_positions, window: int = 0, scale: float | None = None) -> torch.Tensor:
    """Causal grouped-query attention of T queries over N >= T keys.

    q: [T, nq, d]; k, v: [N, nkv, d]; query t stands at absolute position
    q_positions[t] and key j at position j.  q head h reads kv head h // G
    (src/kernel/cuda/paged_flash_attention.cu:891-892).  The score is the dot
    product times ``1/sqrt(d)`` applied after the product (:723, :1158); key j
    is visible to a query at position p iff j <= p
    (src/kernel/cuda/mask_op.cu:37-43), and with ``window`` > 0 also
    p - j < window; softmax over visible keys, then the weighted sum of V
    (:746-790 in tiles; here in one piece).
    """
    T, nq, d = q.shape
    N, nkv, _ = k.shape
    G = nq // nkv
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    out = torch.zeros(T, nq, d, dtype=q.dtype)
    for t in range(T):
        p = int(q_positions[t])
        lo = 0 if window <= 0 else max(0, p - window + 1)
        keys = list(range(lo, p + 1))
        for h in range(nq):
            g = h // G
            s = torch.stack([(q[t, h] * k[j, g]).sum() for j in keys]) * scale
            m = s.max()
            e = torch.exp(s - m)
            w = e / e.sum()
            acc = torch.zeros(d, dtype=q.dtype)
            for idx, j in enumerate(keys):
                acc = acc + w[idx] * v[j, g]
            out[t, h] = acc
    return out


def plain_silu(x: torch.Tensor) -> torch.Tensor:
    """silu(x) = x / (1 + exp(-x)).  src/kernel/cuda/unary.cu:10-12."""
    return x / (1.0 + torch.exp(-x))


def plain_swiglu_mlp(z, w_gate, w_up, w_down):
    """f = (silu(z Wgate^T) * (z Wup^T)) Wdown^T.

    src/core/model/base/ModelCreatorBase.cpp:51-70 (up, gate, unary, down),
    :73-94 (x1 = gate goes through silu, x2 = up multiplies),
    src/kernel/cuda/unary.cu:26.
    """
    g = plain_linear(z, w_gate)
    u = plain_linear(z, w_up)
    return plain_linear(plain_silu(g) * u, w_down)


# --------------------------------------------------------------------------
# model
# --------------------------------------------------------------------------

def layer_windows(cfg: dict) -> list[int]:
    """Window (0 = all keys) of each layer from the configuration's own keys:
    ``use_sliding_window``, ``sliding_window``, ``max_window_layers`` and, when
    present, ``layer_types``.  The reference keeps ``_n_swa`` and per-layer
    ``_swa_layers`` (src/core/model/BaseDefine.h:143-146) without using them;
    the rule here is the configuration's: layers from ``max_window_layers`` on
    slide, and a query at p sees keys j with p - j < sliding_window.
    """
    L = cfg["num_hidden_layers"]
    sw = cfg.get("sliding_window") if cfg.get("use_sliding_window", False) else None
    if not sw:
        return [0] * L
    types = cfg.get("layer_types")
    if types is None:
        mwl = cfg.get("max_window_layers", L)
        types = ["sliding_attention" if i >= mwl else "full_attention" for i in range(L)]
    return [int(sw) if t == "sliding_attention" else 0 for t in types]


def plain_attention_block(x, positions, lw, cfg, window):
    """q/k/v projections, per-head q/k RMS norm before the rotation, rotation,
    attention, output projection.  src/core/model/qwen3/QWen3Creator.cpp:62-131.
    V is neither normed nor rotated (:110-111).
    """
    nq = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nq)
    d = cfg.get("head_dim", cfg["hidden_size"] // nq)
    eps = cfg.get("rms_norm_eps", 1e-6)
    theta = cfg.get("rope_theta", 10000.0)
    T = x.shape[0]
    q = plain_linear(x, lw["q_proj"]).reshape(T, nq, d)
    k = plain_linear(x, lw["k_proj"]).reshape(T, nkv, d)
    v = plain_linear(x, lw["v_proj"]).reshape(T, nkv, d)
    q = plain_rmsnorm(q, lw["q_norm"], eps)      # one [d] weight for all heads
    k = plain_rmsnorm(k, lw["k_norm"], eps)
    q = plain_rope_neox(q, positions, theta)
    k = plain_rope_neox(k, positions, theta)
    o = plain_attention(q, k, v, positions, window=window)
    return plain_linear(o.reshape(T, nq * d), lw["o_proj"])


def plain_decoder_layer(x, positions, lw, cfg, window):
    """Pre-norm block: r = x + attn(norm(x)); out = r + mlp(norm(r)).
    src/core/model/qwen3/QWen3Creator.cpp:62-65 (attn norm), :140 (residual 1),
    :142-148 (ffn norm, ffn), :150-151 (residual 2).
    """
    eps = cfg.get("rms_norm_eps", 1e-6)
    h = plain_rmsnorm(x, lw["input_layernorm"], eps)
    r = x + plain_attention_block(h, positions, lw, cfg, window)
    z = plain_rmsnorm(r, lw["post_attention_layernorm"], eps)
    return r + plain_swiglu_mlp(z, lw["gate_proj"], lw["up_proj"], lw["down_proj"])


def load_plain_model(model_dir: str, dtype=torch.float64):
    """Reads config.json and model.safetensors of a model folder."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    raw = load_file(os.path.join(model_dir, "model.safetensors"))
    raw = {k: v.to(dtype) for k, v in raw.items()}
    return cfg, raw


def _layer_weights(raw: dict, i: int) -> dict:
    p = f"model.layers.{i}."
    return {
        "input_layernorm": raw[p + "input_layernorm.weight"],
        "post_attention_layernorm": raw[p + "post_attention_layernorm.weight"],
        "q_proj": raw[p + "self_attn.q_proj.weight"],
        "k_proj": raw[p + "self_attn.k_proj.weight"],
        "v_proj": raw[p + "self_attn.v_proj.weight"],
        "o_proj": raw[p + "self_attn.o_proj.weight"],
        "q_norm": raw[p + "self_attn.q_norm.weight"],
        "k_norm": raw[p + "self_attn.k_norm.weight"],
        "gate_proj": raw[p + "mlp.gate_proj.weight"],
        "up_proj": raw[p + "mlp.up_proj.weight"],
        "down_proj": raw[p + "mlp.down_proj.weight"],
    }


def plain_forward(cfg: dict, raw: dict, token_ids) -> torch.Tensor:
    """Logits [T, V] of one whole sequence at positions 0..T-1.

    Embedding, L blocks, final norm, output head
    (src/core/model/qwen3/QWen3Creator.cpp:43-165); with tied embeddings the
    head is the embedding table (the reference has no such case,
    QWen3Creator.cpp:161-162, the rule is the configuration's
    ``tie_word_embeddings``).
    """
    eps = cfg.get("rms_norm_eps", 1e-6)
    T = len(token_ids)
    positions = list(range(T))
    x = plain_embedding(raw["model.embed_tokens.weight"], token_ids)
    wins = layer_windows(cfg)
    for i in range(cfg["num_hidden_layers"]):
        x = plain_decoder_layer(x, positions, _layer_weights(raw, i), cfg, wins[i])
    y = plain_rmsnorm(x, raw["model.norm.weight"], eps)
    if cfg.get("tie_word_embeddings", False):
        head = raw["model.embed_tokens.weight"]
    else:
        head = raw["lm_head.weight"]
    return plain_linear(y, head)


# --------------------------------------------------------------------------
# faster but still independent whole-sequence forward (matrix form), pinned to
# the element-wise one above by tests; used where sequences are long.
# --------------------------------------------------------------------------

def fast_forward(cfg: dict, raw: dict, token_ids) -> torch.Tensor:
    """Same mathematics as :func:`plain_forward` written with matrix products
    so that sequences of a few hundred tokens take seconds.  Tests check it
    against plain_forward on short sequences.
    """
    nq = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nq)
    H = cfg["hidden_size"]
    d = cfg.get("head_dim", H // nq)
    eps = cfg.get("rms_norm_eps", 1e-6)
    theta = cfg.get("rope_theta", 10000.0)
    G = nq // nkv
    E = raw["model.embed_tokens.weight"]
    where = E.device      # the weights may sit on a GPU, for the widths of the large models
    ids = torch.as_tensor(list(token_ids), dtype=torch.long, device=where)
    T = ids.numel()
    x = E[ids]
    dt = x.dtype
    pos = torch.arange(T, dtype=torch.float64)
    inv = torch.exp(-(2.0 * torch.arange(d // 2, dtype=torch.float64)) / d * math.log(theta))
    ang = pos[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).to(dt)[:, None, :].to(where), torch.sin(ang).to(dt)[:, None, :].to(where)

    def norm(a, w):
        return a * torch.rsqrt((a * a).mean(-1, keepdim=True) + eps) * w

    def rope(a):
        lo, hi = a[..., : d // 2], a[..., d // 2:]
        return torch.cat([lo * cos - hi * sin, lo * sin + hi * cos], -1)

    wins = layer_windows(cfg)
    ii = torch.arange(T, device=where)
    for i in range(cfg["num_hidden_layers"]):
        lw = _layer_weights(raw, i)
        h = norm(x, lw["input_layernorm"])
        q = (h @ lw["q_proj"].T).reshape(T, nq, d)
        k = (h @ lw["k_proj"].T).reshape(T, nkv, d)
        v = (h @ lw["v_proj"].T).reshape(T, nkv, d)
        q = rope(norm(q, lw["q_norm"]))
        k = rope(norm(k, lw["k_norm"]))
        kk = k.repeat_interleave(G, dim=1)
        vv = v.repeat_interleave(G, dim=1)
        s = torch.einsum("thd,jhd->htj", q, kk) / math.sqrt(d)
        vis = ii[None, :] <= ii[:, None]
        if wins[i] > 0:
            vis = vis & ((ii[:, None] - ii[None, :]) < wins[i])
        s = s.masked_fill(~vis[None], float("-inf"))
        p = torch.softmax(s, -1)
        o = torch.einsum("htj,jhd->thd", p, vv).reshape(T, nq * d)
        r = x + o @ lw["o_proj"].T
        z = norm(r, lw["post_attention_layernorm"])
        g = z @ lw["gate_proj"].T
        u = z @ lw["up_proj"].T
        x = r + ((g / (1.0 + torch.exp(-g))) * u) @ lw["down_proj"].T
    y = norm(x, raw["model.norm.weight"])
    head = E if cfg.get("tie_word_embeddings", False) else raw["lm_head.weight"]
    return y @ head.T


# --------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------

def plain_greedy(logits: torch.Tensor) -> int:
    """First maximum wins (std::max_element),
    src/core/sampler/LLMSampler.cpp:43-45."""
    best, arg = None, 0
    for i, v in enumerate(logits.tolist()):
        if best is None or v > best:
            best, arg = v, i
    return arg


def plain_repetition_penalty(logits: torch.Tensor, seen, penalty: float) -> torch.Tensor:
    """Each seen token once: positive logits divided, others multiplied.
    src/core/sampler/LLMSampler.cpp:21-34."""
    out = logits.clone()
    for t in set(int(s) for s in seen):
        if 0 <= t < out.numel():
            out[t] = out[t] / penalty if out[t] > 0 else out[t] * penalty
    return out


def plain_probs(logits: torch.Tensor, temperature: float, top_k: int = 0,
                top_p: float = 1.0, min_p: float = 0.0) -> torch.Tensor:
    """Distribution a random draw is taken from.

    Temperature multiplies the logits by 1/temp
    (src/core/sampler/LLMSampler.cpp:36-41); the reference then normalises the
    values it is given (:47-54), which is a distribution only after a softmax,
    so the softmax is taken here.  top_k / top_p / min_p are the fields of
    SamplingConfig (src/core/sampler/LLMSampler.h:55-63) in their usual
    meaning: keep the k most likely; keep the smallest set of most likely
    tokens whose mass reaches top_p; keep tokens with p >= min_p * p_max.
    Ties at a threshold are all kept.
    """
    z = logits.double() / temperature
    p = torch.softmax(z, -1)
    keep = torch.ones_like(p, dtype=torch.bool)
    if top_k and top_k > 0 and top_k < p.numel():
        kth = torch.sort(p, descending=True).values[top_k - 1]
        keep &= p >= kth
    if top_p < 1.0:
        pk = torch.where(keep, p, torch.zeros_like(p))
        pk = pk / pk.sum()
        sp, _ = torch.sort(pk, descending=True)
        c = torch.cumsum(sp, 0)
        n = int((c < top_p).sum().item()) + 1
        thr = sp[min(n, sp.numel()) - 1]
        keep &= pk >= thr
    if min_p > 0.0:
        keep &= p >= min_p * p.max()
    p = torch.where(keep, p, torch.zeros_like(p))
    return p / p.sum()


def plain_inverse_cdf(probs: torch.Tensor, u: float) -> int:
    """Smallest index whose cumulative probability exceeds u."""
    c = 0.0
    last = 0
    for i, pv in enumerate(probs.tolist()):
        if pv > 0.0:
            last = i
            c += pv
            if u < c:
                return i
    return last
