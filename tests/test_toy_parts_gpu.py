"""Parts defined here, outside the package, can be registered, built into a
model of an architecture of their own and stepped, without a change to the
package's files: a mixer with state of its own, a feed-forward with routing,
another position encoding; a run order that names a layer twice and lets a
call read another call's cache.  The toy parts compute with torch (they are
no product code); the package's step function, cache manager, state slots and
attention kernels carry them."""
import math
from dataclasses import dataclass

import pytest
import torch

import plain_qwen3 as P
import replay_lib as rl
from helpers import random_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

H, V, NQ, NKV, D, I = 32, 96, 4, 2, 16, 48
EPS = 1e-5


def _register():
    from tffinfer_amd.config.base import LayerCall, LayerSpec, ModelConfig, PartSpec
    from tffinfer_amd.models import TensorNames, register_architecture
    from tffinfer_amd.parts import (FeedForward, Mixer, PositionEncoding, StateSpec, WeightSpec,
                                    register_feed_forward, register_mixer, register_position_encoding)

    @register_mixer("toy_running_mean")
    class RunningMean(Mixer):
        """out_t = W . mean(x_0..x_t): the state is the running sum and the count."""

        def __init__(self, hidden_size):
            self.h = hidden_size
            self.w = None

        def state_spec(self):
            return StateSpec((self.h + 1,), torch.float32)

        def weight_specs(self):
            return {"proj.weight": WeightSpec((self.h, self.h))}

        def load_weights(self, weights, dtype, device):
            self.w = weights["proj.weight"].float().to(device)

        def forward(self, ctx, x):
            b = ctx.batch
            out = torch.empty(x.shape[0], self.h, dtype=torch.float32, device=x.device)
            for r in range(b.num_reqs):
                lo, hi = b.host_cu_tokens[r], b.host_cu_tokens[r + 1]
                st = ctx.state[b.host_state_slots[r]]
                if b.host_start_pos[r] == 0:
                    st.zero_()
                sums = st[:self.h] + torch.cumsum(x[lo:hi].float(), 0)
                counts = st[self.h] + torch.arange(1, hi - lo + 1, device=x.device, dtype=torch.float32)
                out[lo:hi] = (sums / counts[:, None]) @ self.w.T
                st[:self.h] = sums[-1]
                st[self.h] = counts[-1]
            return out

    @register_feed_forward("toy_top1_of_2")
    class Top1(FeedForward):
        """Two linear experts, the router's larger logit picks one per token."""

        def __init__(self, hidden_size):
            self.h = hidden_size

        def weight_specs(self):
            return {"router.weight": WeightSpec((2, self.h)), "experts.0.weight": WeightSpec((self.h, self.h)),
                    "experts.1.weight": WeightSpec((self.h, self.h))}

        def load_weights(self, weights, dtype, device):
            self.router = weights["router.weight"].float().to(device)
            self.experts = [weights[f"experts.{e}.weight"].float().to(device) for e in range(2)]

        def forward(self, ctx, x):
            xf = x.float()
            pick = (xf @ self.router.T).argmax(-1)
            both = torch.stack([xf @ w.T for w in self.experts], 0)
            return both[pick, torch.arange(x.shape[0], device=x.device)]

    @register_position_encoding("toy_harmonic")
    class Harmonic(PositionEncoding):
        """angle(pos, i) = pos / (i + 1), neighbouring pairs."""
        pairing = "interleaved"

        def __init__(self, head_dim):
            self.rotary_dim = head_dim

        def table(self, max_positions, device):
            a = torch.arange(max_positions, dtype=torch.float64)[:, None] / torch.arange(
                1, self.rotary_dim // 2 + 1, dtype=torch.float64)[None, :]
            return torch.stack([torch.cos(a), torch.sin(a)], -1).float().contiguous().to(device)

    @dataclass
    class ToyConfig(ModelConfig):
        hidden_size: int = H
        vocab_size: int = V
        max_position_embeddings: int = 256
        tie_word_embeddings: bool = False
        architecture = "ToyForCausalLM"

        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return {"architectures": ["ToyForCausalLM"]}

        def layer_specs(self):
            norm = PartSpec("rmsnorm", {"size": H, "eps": EPS})

            def attn(pos):
                return PartSpec("gqa_attention", {"hidden_size": H, "num_heads": NQ, "num_kv_heads": NKV,
                                                  "head_dim": D, "qk_norm_eps": EPS, "position": pos})
            return [
                LayerSpec(PartSpec("prenorm"), attn(PartSpec("rope", {"head_dim": D, "theta": 100.0})),
                          PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I}), norm),
                LayerSpec(PartSpec("prenorm"), PartSpec("toy_running_mean", {"hidden_size": H}),
                          PartSpec("toy_top1_of_2", {"hidden_size": H}), norm),
                LayerSpec(PartSpec("prenorm"), attn(PartSpec("toy_harmonic", {"head_dim": D})),
                          PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I}), norm),
            ]

        def layer_schedule(self):
            # layer 0 runs twice (a cache per call); the last call runs layer 2 again on the
            # cache its first call filled, writing nothing
            return [LayerCall(0, 0), LayerCall(1, 1), LayerCall(2, 2), LayerCall(0, 3),
                    LayerCall(2, 2, writes_cache=False)]

        def final_norm_spec(self):
            return PartSpec("rmsnorm", {"size": H, "eps": EPS})

    register_architecture("ToyForCausalLM", ToyConfig, TensorNames(
        children={"norm1": "ln1", "mixer": "mix", "norm2": "ln2", "feed_forward": "ff"}))
    return ToyConfig


def toy_reference(raw, tokens):
    """Whole-sequence float64 forward of the toy model, written out by hand."""
    T = len(tokens)
    pos = list(range(T))
    w = {k: v.double() for k, v in raw.items()}

    def attn_layer(x, i, kind, kv_from=None):
        p = f"model.layers.{i}."
        h = P.plain_rmsnorm(x, w[p + "ln1.weight"], EPS)
        q = P.plain_linear(h, w[p + "mix.q_proj.weight"]).reshape(T, NQ, D)
        k = P.plain_linear(h, w[p + "mix.k_proj.weight"]).reshape(T, NKV, D)
        v = P.plain_linear(h, w[p + "mix.v_proj.weight"]).reshape(T, NKV, D)
        q = P.plain_rmsnorm(q, w[p + "mix.q_norm.weight"], EPS)
        k = P.plain_rmsnorm(k, w[p + "mix.k_norm.weight"], EPS)
        if kind == "rope":
            q, k = P.plain_rope_neox(q, pos, 100.0), P.plain_rope_neox(k, pos, 100.0)
        else:
            ang = torch.arange(T, dtype=torch.float64)[:, None] / torch.arange(1, D // 2 + 1, dtype=torch.float64)
            c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]

            def rot(a):
                o = a.clone()
                o[..., 0::2] = a[..., 0::2] * c - a[..., 1::2] * s
                o[..., 1::2] = a[..., 0::2] * s + a[..., 1::2] * c
                return o
            q, k = rot(q), rot(k)
        if kv_from is not None:
            k, v = kv_from
        o = P.plain_attention(q, k, v, pos).reshape(T, NQ * D)
        r = x + P.plain_linear(o, w[p + "mix.o_proj.weight"])
        z = P.plain_rmsnorm(r, w[p + "ln2.weight"], EPS)
        f = P.plain_swiglu_mlp(z, w[p + "ff.gate_proj.weight"], w[p + "ff.up_proj.weight"],
                               w[p + "ff.down_proj.weight"])
        return r + f, (k, v)

    def mean_layer(x):
        p = "model.layers.1."
        h = P.plain_rmsnorm(x, w[p + "ln1.weight"], EPS)
        mean = torch.cumsum(h, 0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None]
        r = x + mean @ w[p + "mix.proj.weight"].T
        z = P.plain_rmsnorm(r, w[p + "ln2.weight"], EPS)
        pick = (z @ w[p + "ff.router.weight"].T).argmax(-1)
        f = torch.stack([z[t] @ w[p + f"ff.experts.{int(pick[t])}.weight"].T for t in range(T)])
        return r + f

    x = w["model.embed_tokens.weight"][tokens]
    x, _ = attn_layer(x, 0, "rope")
    x = mean_layer(x)
    x, kv2 = attn_layer(x, 2, "harmonic")
    x, _ = attn_layer(x, 0, "rope")
    x, _ = attn_layer(x, 2, "harmonic", kv_from=kv2)
    y = P.plain_rmsnorm(x, w["model.norm.weight"], EPS)
    return y @ w["lm_head.weight"].T


def test_toy_architecture_is_registered_built_and_stepped(tmp_path):
    from safetensors.torch import load_file
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.models import load_model
    from tffinfer_amd.weights import write_random_model
    ToyConfig = _register()
    d = write_random_model(str(tmp_path / "toy"), ToyConfig(), seed=77, dtype="float32")
    raw = load_file(d + "/model.safetensors")
    assert "model.layers.1.mix.proj.weight" in raw and "model.layers.1.ff.router.weight" in raw
    model = load_model(d, torch.float32, DEV)
    reqs = model.call_requirements()
    assert [r[0] for r in reqs] == [0, 1, 2, 3, 2] and reqs[4][1] is False
    assert reqs[1][2] is None and reqs[1][3] is not None      # the toy mixer: state, no keys
    requests = {f"t{i}": random_tokens(n, V, 5 + i) for i, n in enumerate([9, 37, 20, 51])}
    refs = {rid: toy_reference(raw, toks) for rid, toks in requests.items()}
    for mode in (rl.trace_whole, rl.trace_chunks, rl.trace_mixed):
        steps = mode(requests)
        pages = rl.max_live_tokens(steps, 8) // 8
        runner = ModelRunner(model, page_size=8, num_pages=pages, max_seqs=4)
        assert len(runner.cache.groups) == 1 and runner.cache.groups[0].cache_ids == [0, 2, 3]
        assert list(runner.cache.state_tensors) == [1]
        results = rl.run_steps_in_process(runner, steps)
        _check(requests, refs, steps, results, mode.__name__)


def _check(requests, refs, steps, results, what):
    done = {rid: 0 for rid in requests}
    for s in steps:
        row = 0
        for e in s["entries"]:
            for wnt in e["want"]:
                got = results[s["step"]][row]
                ref = refs[e["id"]][done[e["id"]] + wnt]
                err = float((got.double() - ref).abs().max() / ref.abs().max())
                assert err < 2e-5, f"{what} step {s['step']} request {e['id']} pos {done[e['id']] + wnt}: {err:.2e}"
                row += 1
            done[e["id"]] += len(e["tokens"])


def test_a_part_that_cannot_be_captured_splits_the_graph(tmp_path):
    """The toy mixer and feed-forward loop on the host, so their layer call cannot go into a HIP
    graph.  The decode step is then three pieces: a graph (embedding, first call), the toy layer
    run eagerly on the live rows (it keeps state per request: a padding row must never reach
    it), a graph (the other calls, final norm, head)."""
    from safetensors.torch import load_file
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.models import load_model
    from tffinfer_amd.weights import write_random_model
    ToyConfig = _register()
    d = write_random_model(str(tmp_path / "toy"), ToyConfig(), seed=78, dtype="float32")
    raw = load_file(d + "/model.safetensors")
    model = load_model(d, torch.float32, DEV)
    assert not model.graph_safe()
    assert [(safe, items) for safe, items in model.graph_pieces()] == [
        (True, ["embed", 0]), (False, [1]), (True, [2, 3, 4, "finish"])]
    requests = {f"t{i}": random_tokens(n, V, 15 + i) for i, n in enumerate([9, 37, 20])}    # three live rows of four
    refs = {rid: toy_reference(raw, toks) for rid, toks in requests.items()}
    for mode in (rl.trace_tail, rl.trace_mixed):
        steps = mode(requests)
        pages = rl.max_live_tokens(steps, 8) // 8
        runner = ModelRunner(model, page_size=8, num_pages=pages, max_seqs=4, use_graphs=True)
        results = rl.run_steps_in_process(runner, steps)
        assert runner._graphs, "no decode step went through the graphs"
        for g in runner._graphs.values():
            assert [pc.graph is not None for pc in g.pieces] == [True, False, True]
        _check(requests, refs, steps, results, mode.__name__ + " with graphs")


@pytest.mark.parametrize("use_graphs", [False, True])
def test_toy_architecture_through_the_engine_with_a_preemption(tmp_path, use_graphs):
    """The scheduler, the cache manager and the state slots carry a model with per-request state
    of fixed size: three requests on a pool so small that the newest is preempted while it
    decodes, when its running mean is long past zero, and is computed again from its first
    token (its slot is cleared when it comes back).  Every kept row of logits is compared with
    the hand-written reference on the request's own sequence, and every request's tokens with
    what the engine gives it alone."""
    from safetensors.torch import load_file
    from tffinfer_amd import EngineOptions, LLMEngine
    from tffinfer_amd.models import load_model
    from tffinfer_amd.weights import write_random_model
    ToyConfig = _register()
    d = write_random_model(str(tmp_path / "toy"), ToyConfig(), seed=79, dtype="float32")
    raw = load_file(d + "/model.safetensors")
    model = load_model(d, torch.float32, DEV)
    prompts = [random_tokens(n, V, 25 + i) for i, n in enumerate([11, 30, 19])]
    new = [40, 34, 45]
    opt = EngineOptions(dtype="float32", page_size=8, num_pages=16, max_num_seqs=3, max_num_batched_tokens=32,
                        prefill_chunk=16, max_model_len=128, use_graphs=use_graphs, run_ahead=True)
    eng = LLMEngine(model, opt)
    eng.keep_logits = True
    preempted_with_state = []
    inner = eng.scheduler._preempt_last

    def preempt():
        victim = eng.scheduler.running[-1]
        slot = eng.runner.cache.slot(victim.id)
        state = eng.runner.cache.state_tensors[1][slot]
        preempted_with_state.append((victim.id, victim.num_computed, float(state[-1]), float(state[:-1].abs().max())))
        return inner()

    eng.scheduler._preempt_last = preempt
    ids = [eng.add_request(p, max_new_tokens=n, ignore_eos=True) for p, n in zip(prompts, new)]
    while eng.has_work:
        eng.step()
        eng.runner.cache.check()
    assert eng.scheduler.stats.preemptions > 0, "the pool was meant to run out"
    # a victim had tokens behind it: a count and a sum that the cleared slot must not keep
    assert any(count > 0 and biggest > 0 for _, _, count, biggest in preempted_with_state), preempted_with_state
    results = [eng.pop_result(i) for i in ids]
    for r, n in zip(results, new):
        assert len(r.output) == n and r.finish_reason == "length"
        ref = toy_reference(raw, r.prompt + r.output)
        for i, (row, tok) in enumerate(zip(r.logits[:n], r.output)):
            want = ref[len(r.prompt) + i - 1]
            err = float((row.double() - want).abs().max() / want.abs().max())
            assert err < 2e-5, f"request {r.id} output {i}: {err:.2e}"
            assert tok == int(torch.argmax(row))
    assert any(r.num_preemptions > 0 for r in results)
    for p, n, r in zip(prompts, new, results):
        alone = LLMEngine(model, EngineOptions(dtype="float32", page_size=8, num_pages=24, max_num_seqs=1,
                                               max_model_len=128, use_graphs=use_graphs))
        assert alone.generate([p], max_new_tokens=n, ignore_eos=True)[0].output == r.output
    assert all(g.pool.num_used == 0 for g in eng.runner.cache.groups)
