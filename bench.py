"""Decode and prefill throughput of the engine at the Qwen3-8B shape with random
weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole engine (scheduler, batch tables, model,
sampling, tokens back on the host) for a batch of 8 requests that each hold a
2,048-token context.  Prints one JSON line: decoded tokens a second, a prefill
of 2,048 tokens with its share of the bf16 MFMA peak, the decode step's share
of the HBM peak, and decode throughput at batch 1 and 64.
"""
import argparse
import json
import statistics
import sys
import time

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_PEAK = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}   # dense, published

# layer sizes of the benchmark configuration (Qwen3-8B shape) and of the two larger shapes
QWEN3_8B = dict(
    architectures=["Qwen3ForCausalLM"], hidden_size=4096, num_hidden_layers=36,
    num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288,
    vocab_size=151936, max_position_embeddings=8192, rms_norm_eps=1e-6, rope_theta=1000000.0,
    tie_word_embeddings=False,
)
SHAPES = {
    "8b": ("Qwen3-8B shape", QWEN3_8B),
    "14b": ("Qwen3-14B shape", dict(QWEN3_8B, hidden_size=5120, num_hidden_layers=40, num_attention_heads=40,
                                    intermediate_size=17408)),
    "32b": ("Qwen3-32B shape", dict(QWEN3_8B, hidden_size=5120, num_hidden_layers=64, num_attention_heads=64,
                                    intermediate_size=25600, max_position_embeddings=16384)),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--shape", choices=sorted(SHAPES), default="8b",
                    help="layer sizes: the benchmark configuration (8b) or one of the larger shapes")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--only", choices=["prefill", "decode"], default=None,
                    help="measure one phase only (for profiling); the JSON line then lacks the other")
    ap.add_argument("--mixed", type=int, default=0, metavar="R",
                    help="instead of the decode steps: R requests with prompt lengths uniform in [128, 4096], "
                         "prompt portions of --chunk tokens beside decoding requests, 256 tokens generated each")
    ap.add_argument("--chunk", type=int, default=512, help="prompt portion of the --mixed workload")
    ap.add_argument("--budget", type=int, default=0,
                    help="tokens of a step of the --mixed workload (default: a portion beside every decoding request, at least 1,024)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--ceilings", action="store_true",
                    help="measure streaming-read bandwidth and back-to-back MFMA rate on this machine and stop")
    return ap.parse_args()


def random_prompt(gen, n, vocab):
    import torch
    return torch.randint(0, vocab, (n,), generator=gen).tolist()


def matmul_params_per_layer(c):
    H, nq, nkv, d, I = (c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"],
                        c["head_dim"], c["intermediate_size"])
    return (nq + 2 * nkv) * d * H + nq * d * H + 3 * I * H


def prefill_flops(c, L, T):
    gemm = 2.0 * T * matmul_params_per_layer(c) * L
    attn = 4.0 * c["num_attention_heads"] * c["head_dim"] * (T * (T + 1) / 2) * L
    head = 2.0 * c["hidden_size"] * c["vocab_size"]
    return gemm + attn + head


def decode_bytes(c, L, batch, context, esz=2):
    weights = (matmul_params_per_layer(c) * L + c["hidden_size"] * c["vocab_size"]) * esz
    kv = 2 * L * c["num_key_value_heads"] * c["head_dim"] * esz * batch * context
    return weights + kv


def sync():
    import torch
    torch.cuda.synchronize()


def measure_prefill(engine, gen, T, vocab, reps=5, warm=2):
    from tffinfer_amd.engine.batch import StepEntry
    times = []
    for i in range(reps + warm):
        rid = f"prefill{i}"
        toks = random_prompt(gen, T, vocab)
        engine.runner.add_request(rid)
        sync()
        t0 = time.perf_counter()
        logits = engine.runner.step([StepEntry(rid, toks, [T - 1])])
        sync()
        dt = time.perf_counter() - t0
        assert logits.shape[0] == 1
        engine.runner.free_request(rid)
        if i >= warm:   # the first runs warm up (allocator, work tables, clocks)
            times.append(dt)
    return statistics.median(times)


def decode_slack(batch, context, chunk=2048):
    """Steps the first request may decode while the last one still reads its prompt."""
    return batch * (-(-context // chunk) + 1)


def measure_decode(engine, gen, batch, context, steps, warmup, vocab):
    """Fills ``batch`` requests with ``context`` tokens each (untimed prefill),
    then times ``steps`` decode steps of the engine."""
    for _ in range(batch):
        # requests that finish their prompt early decode while the others still prefill
        engine.add_request(random_prompt(gen, context, vocab),
                           max_new_tokens=warmup + steps + decode_slack(batch, context) + 8, ignore_eos=True)
    # untimed: prompts, up to the first decode-only step
    while any(r.num_pending > 1 for r in engine.scheduler.running) or engine.scheduler.waiting:
        engine.step()
    for _ in range(warmup):
        out = engine.step()
        assert len(out) == batch
    sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        out = engine.step()
    sync()
    dt = time.perf_counter() - t0
    assert len(out) == batch
    for r in list(engine.scheduler.running):
        engine.abort(r.id)
    return dt


def measure_mixed(engine, gen, requests, vocab, new_tokens=256, lo=128, hi=4096):
    """Continuous batching: all requests arrive at once, the scheduler admits them as
    slots and pages allow, cuts prompts into portions and decodes the others beside them."""
    import torch
    lens = torch.randint(lo, hi + 1, (requests,), generator=gen).tolist()
    for n in lens:
        engine.add_request(random_prompt(gen, n, vocab), max_new_tokens=new_tokens, ignore_eos=True)
    sync()
    t0 = time.perf_counter()
    steps = 0
    while engine.has_work:
        engine.step()
        steps += 1
    sync()
    dt = time.perf_counter() - t0
    st = engine.scheduler.stats
    return {"requests": requests, "prompt_tokens": sum(lens), "generated_tokens": requests * new_tokens,
            "seconds": round(dt, 3), "engine_steps": steps, "preemptions": st.preemptions,
            "total_tokens_per_s": round((sum(lens) + requests * new_tokens) / dt, 1),
            "generated_tokens_per_s": round(requests * new_tokens / dt, 1)}


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on a single GPU)")
        sys.exit(2)
    import torch
    from tffinfer_amd import EngineOptions, LLMEngine
    from tffinfer_amd.kernels import lib as kernel_lib
    from tffinfer_amd.models import build_model_skeleton, config_from_dict

    kernel_lib.load()
    if args.ceilings:
        from tffinfer_amd.kernels import ops
        print(json.dumps({"ceilings": ops.measure_ceilings("cuda:0"),
                          "published": {"hbm_GBps": HBM_PEAK_GBS, "bf16_TFLOPs": MFMA_PEAK["bf16"] / 1e12}}))
        return
    shape_name, shape = SHAPES[args.shape]
    cfg = dict(shape)
    L_full = cfg["num_hidden_layers"]
    L = args.layers or L_full
    cfg["num_hidden_layers"] = L
    # a context beyond the shape's own limit: the limit grows with it (it sizes the rotation table only)
    longest = max(args.prefill_tokens, args.context + args.steps + args.warmup + decode_slack(max(args.batch, 64), args.context) + 16)
    if not args.mixed and longest > cfg["max_position_embeddings"]:
        cfg["max_position_embeddings"] = 1 << (longest - 1).bit_length()
    vocab = cfg["vocab_size"]
    gen = torch.Generator().manual_seed(args.seed)
    model = build_model_skeleton(config_from_dict(cfg))
    model.init_random(args.seed, torch.bfloat16, "cuda:0", on_device=True)
    sync()
    if args.mixed:
        kv_tokens = args.mixed * (4096 + 256 + args.page_size)
        opt = EngineOptions(dtype="bfloat16", page_size=args.page_size, kv_tokens=kv_tokens,
                            max_num_seqs=args.mixed, max_num_batched_tokens=args.budget or max(args.chunk + args.mixed, 1024),
                            prefill_chunk=args.chunk, max_model_len=cfg["max_position_embeddings"],
                            use_graphs=not args.no_graphs)
        engine = LLMEngine(model, opt)
        res = measure_mixed(engine, gen, args.mixed, vocab)
        print(json.dumps({"workload": "mixed", "model": shape_name, "layers_run": L, "chunk": args.chunk, **res}))
        return
    max_batch = args.batch if (args.no_points or args.only) else max(args.batch, 64)
    total_steps = args.steps + args.warmup + decode_slack(max_batch, args.context) + 16
    kv_tokens = max_batch * (args.context + total_steps + args.page_size) + args.prefill_tokens
    opt = EngineOptions(dtype="bfloat16", page_size=args.page_size, kv_tokens=kv_tokens, max_num_seqs=max_batch,
                        max_num_batched_tokens=max(4096, max_batch), prefill_chunk=2048,
                        max_model_len=cfg["max_position_embeddings"], use_graphs=not args.no_graphs)
    engine = LLMEngine(model, opt)

    t_prefill = t_decode = None
    if args.only != "decode":
        t_prefill = measure_prefill(engine, gen, args.prefill_tokens, vocab)
    if args.only != "prefill":
        t_decode = measure_decode(engine, gen, args.batch, args.context, args.steps, args.warmup, vocab)
    if args.only:
        part = ({"prefill_ms": round(1000 * t_prefill, 3)} if t_prefill else
                {"decode_ms_per_step": round(1000 * t_decode / args.steps, 4)})
        print(json.dumps({"only": args.only, **part, "batch": args.batch, "context": args.context}))
        return
    points = {}
    if not args.no_points:
        for b, key in ((1, "decode_b1"), (64, "decode_b64")):
            k = min(args.steps, 32)
            dt = measure_decode(engine, gen, b, args.context, k, min(args.warmup, 4), vocab)
            points[key] = round(b * k / dt, 1)

    ms_step = 1000.0 * t_decode / args.steps
    value = args.batch * args.steps / t_decode
    mean_context = args.context + args.warmup + args.steps / 2.0
    nbytes = decode_bytes(cfg, L, args.batch, mean_context)
    achieved = nbytes / (t_decode / args.steps) / 1e9
    pf = prefill_flops(cfg, L, args.prefill_tokens)
    out = {
        "metric": "decode_tokens_per_s", "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (seeded random weights and token ids)",
        "config": {
            "model": shape_name, "layers": L_full, "layers_run": L, "hidden": cfg["hidden_size"],
            "q_heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["head_dim"], "intermediate": cfg["intermediate_size"], "vocab": vocab,
            "rope_theta": cfg["rope_theta"], "rms_norm_eps": cfg["rms_norm_eps"],
            "max_context": cfg["max_position_embeddings"], "global_batch": args.batch,
            "seq_len": args.context, "prefill_tokens": args.prefill_tokens, "page_size": args.page_size,
            "hip_graphs": not args.no_graphs, "parallelism": "single GPU",
        },
        "prefill": {"value": round(args.prefill_tokens / t_prefill, 1), "tokens": args.prefill_tokens,
                    "ms": round(1000.0 * t_prefill, 3), "frac": round(pf / t_prefill / MFMA_PEAK["bf16"], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
