"""A toy mixer with state of its own that *can* be captured: it addresses its state through the
step's device tables only (no loop on the host over the step's entries), so the whole decode
step is one HIP graph.  The graph's padding rows then run through the mixer too, in every replay
and in the two runs on nothing but padding rows before the capture, and update a state: the row
of the state tensor that no request holds.  Defined here, outside the package; computed with
torch (it is no product code)."""
from dataclasses import dataclass

import pytest
import torch

import plain_qwen3 as P
import replay_lib as rl
from helpers import random_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
H, V, NQ, NKV, D, I = 48, 120, 4, 2, 16, 64
EPS = 1e-5


def _register():
    from tffinfer_amd.config.base import LayerCall, LayerSpec, ModelConfig, PartSpec
    from tffinfer_amd.models import TensorNames, register_architecture
    from tffinfer_amd.parts import Mixer, StateSpec, WeightSpec, register_mixer

    @register_mixer("toy_captured_mean")
    class CapturedMean(Mixer):
        """out_t = W . mean(x_0 .. x_t).  The state is the running sum; the count is the token's
        position + 1.  Everything is indexed by tensors on the device."""
        graph_safe = True

        def __init__(self, hidden_size):
            self.h = hidden_size
            self.w = None

        def state_spec(self):
            return StateSpec((self.h,), torch.float32)

        def weight_specs(self):
            return {"proj.weight": WeightSpec((self.h, self.h))}

        def load_weights(self, weights, dtype, device):
            self.w = weights["proj.weight"].float().to(device)

        def forward(self, ctx, x):
            b = ctx.batch
            xf = x.float()
            req = b.token_req.long()                              # request (row of the step) of every token
            cu = b.cu_tokens.long()
            slots = b.state_slots.long()
            c = torch.cumsum(xf, 0)
            first = cu[:-1]                                       # a request's first token of this step
            before = torch.where((first > 0)[:, None], c[(first - 1).clamp_min(0)], torch.zeros_like(c[:1]))
            old = torch.where((b.start_pos > 0)[:, None], ctx.state[slots], torch.zeros_like(c[:1]))
            sums = c - before[req] + old[req]                     # running sums per token
            ctx.state[slots] = sums[cu[1:] - 1]                   # a request's last token of this step
            mean = sums / (b.positions.float() + 1.0)[:, None]
            return mean @ self.w.T

    @dataclass
    class ToyConfig(ModelConfig):
        hidden_size: int = H
        vocab_size: int = V
        max_position_embeddings: int = 128
        tie_word_embeddings: bool = True
        architecture = "ToyCapturedForCausalLM"

        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return {"architectures": ["ToyCapturedForCausalLM"]}

        def layer_specs(self):
            norm = PartSpec("rmsnorm", {"size": H, "eps": EPS})
            ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I})
            attn = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": NQ, "num_kv_heads": NKV, "head_dim": D,
                                              "qk_norm_eps": EPS,
                                              "position": PartSpec("rope", {"head_dim": D, "theta": 1000.0})})
            return [LayerSpec(PartSpec("prenorm"), attn, ffn, norm),
                    LayerSpec(PartSpec("prenorm"), PartSpec("toy_captured_mean", {"hidden_size": H}), ffn, norm)]

        def layer_schedule(self):
            return [LayerCall(0, 0), LayerCall(1, 1)]

        def final_norm_spec(self):
            return PartSpec("rmsnorm", {"size": H, "eps": EPS})

    register_architecture("ToyCapturedForCausalLM", ToyConfig, TensorNames(
        children={"norm1": "ln1", "mixer": "mix", "norm2": "ln2", "feed_forward": "ff"}))
    return ToyConfig


def reference(raw, tokens):
    """Whole-sequence float64 forward, written out by hand."""
    T = len(tokens)
    pos = list(range(T))
    w = {k: v.double() for k, v in raw.items()}

    def ffn(r, p):
        z = P.plain_rmsnorm(r, w[p + "ln2.weight"], EPS)
        return r + P.plain_swiglu_mlp(z, w[p + "ff.gate_proj.weight"], w[p + "ff.up_proj.weight"],
                                      w[p + "ff.down_proj.weight"])

    x = w["model.embed_tokens.weight"][tokens]
    p = "model.layers.0."
    h = P.plain_rmsnorm(x, w[p + "ln1.weight"], EPS)
    q = P.plain_linear(h, w[p + "mix.q_proj.weight"]).reshape(T, NQ, D)
    k = P.plain_linear(h, w[p + "mix.k_proj.weight"]).reshape(T, NKV, D)
    v = P.plain_linear(h, w[p + "mix.v_proj.weight"]).reshape(T, NKV, D)
    q = P.plain_rope_neox(P.plain_rmsnorm(q, w[p + "mix.q_norm.weight"], EPS), pos, 1000.0)
    k = P.plain_rope_neox(P.plain_rmsnorm(k, w[p + "mix.k_norm.weight"], EPS), pos, 1000.0)
    o = P.plain_attention(q, k, v, pos).reshape(T, NQ * D)
    x = ffn(x + P.plain_linear(o, w[p + "mix.o_proj.weight"]), p)
    p = "model.layers.1."
    h = P.plain_rmsnorm(x, w[p + "ln1.weight"], EPS)
    mean = torch.cumsum(h, 0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None]
    x = ffn(x + mean @ w[p + "mix.proj.weight"].T, p)
    y = P.plain_rmsnorm(x, w["model.norm.weight"], EPS)
    return y @ w["model.embed_tokens.weight"].T


def test_a_captured_mixer_with_state_runs_its_padding_rows_on_a_slot_of_their_own(tmp_path):
    from safetensors.torch import load_file
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.models import load_model
    from tffinfer_amd.weights import write_random_model
    ToyConfig = _register()
    d = write_random_model(str(tmp_path / "toy"), ToyConfig(), seed=91, dtype="float32")
    raw = load_file(d + "/model.safetensors")
    model = load_model(d, torch.float32, DEV)
    assert model.graph_safe()                  # one graph for the whole decode step
    requests = {f"t{i}": random_tokens(n, V, 35 + i) for i, n in enumerate([12, 41, 23])}    # three live rows of four
    refs = {rid: reference(raw, toks) for rid, toks in requests.items()}
    for mode in (rl.trace_whole, rl.trace_chunks, rl.trace_tail, rl.trace_mixed):
        steps = mode(requests)
        pages = rl.max_live_tokens(steps, 8) // 8
        graphs = mode in (rl.trace_tail, rl.trace_mixed)
        runner = ModelRunner(model, page_size=8, num_pages=pages, max_seqs=4, use_graphs=graphs)
        state = runner.cache.state_tensors[1]
        assert state.shape == (5, H)
        results = rl.run_steps_in_process(runner, steps)
        done = {rid: 0 for rid in requests}
        for s in steps:
            row = 0
            for e in s["entries"]:
                for wnt in e["want"]:
                    got, ref = results[s["step"]][row], refs[e["id"]][done[e["id"]] + wnt]
                    err = float((got.double() - ref).abs().max() / ref.abs().max())
                    assert err < 2e-5, f"{mode.__name__} step {s['step']} request {e['id']} pos {done[e['id']] + wnt}: {err:.2e}"
                    row += 1
                done[e["id"]] += len(e["tokens"])
        if graphs:
            assert runner._graphs and all(len(g.pieces) == 1 for g in runner._graphs.values())
            # the padding rows went through the mixer, on the slot that no request holds
            assert float(state[runner.cache.padding_slot].abs().max()) > 0
