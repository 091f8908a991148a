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
import sys

# layer sizes of the benchmark configuration (Qwen3-8B shape), of three smaller shapes and of two larger ones
QWEN3_8B = dict(
    architectures=["Qwen3ForCausalLM"], hidden_size=4096, num_hidden_layers=36,
    num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288,
    vocab_size=151936, max_position_embeddings=8192, rms_norm_eps=1e-6, rope_theta=1000000.0,
    tie_word_embeddings=False,
)
SHAPES = {
    "0.6b": ("Qwen3-0.6B shape", dict(QWEN3_8B, hidden_size=1024, num_hidden_layers=28, num_attention_heads=16,
                                      intermediate_size=3072, tie_word_embeddings=True)),
    "1.7b": ("Qwen3-1.7B shape", dict(QWEN3_8B, hidden_size=2048, num_hidden_layers=28, num_attention_heads=16,
                                      intermediate_size=6144, tie_word_embeddings=True)),
    "4b": ("Qwen3-4B shape", dict(QWEN3_8B, hidden_size=2560, intermediate_size=9728, tie_word_embeddings=True)),
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
    ap.add_argument("--contexts", default=None,
                    help="with --only decode: requests of these context lengths instead of --batch requests of --context, "
                         "comma-separated, NxC for N requests of C tokens (32768,63x1024)")
    ap.add_argument("--shape", choices=sorted(SHAPES), default="8b",
                    help="layer sizes: the benchmark configuration (8b) or one of the smaller and larger shapes")
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
                    help="tokens of a step of the --mixed workload (default: the engine's own default, 2,048: four portions, "
                         "or fewer beside the requests that decode)")
    ap.add_argument("--token-quantum", type=int, default=None,
                    help="with --mixed: the scheduler cuts steps a little over a multiple of this many tokens down "
                         "to the multiple (default: the engine's own, 256; 0: off)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--ceilings", action="store_true",
                    help="measure streaming-read bandwidth, back-to-back MFMA rates and a large square product "
                         "on this machine and stop")
    ap.add_argument("--sampling", default=None, metavar="K,P,T[,R]",
                    help="with --only decode: every request draws from the top K tokens (0: off) that hold a share "
                         "P of the probability (1: off) at temperature T, e.g. 50,0.95,0.8, instead of taking the "
                         "most likely one; R: a repetition penalty")
    ap.add_argument("--no-large-points", action="store_true",
                    help="skip the two points at the larger shapes (32 mixed requests at the 14B shape; batch 16 "
                         "at 8,192 tokens of context at the 32B shape), which the default run adds to 'points'")
    ap.add_argument("--no-long-points", action="store_true",
                    help="skip the points at long contexts (decode at batch 8 with 32,768 tokens of context and at "
                         "batch 128 with 8,192; prefill of 8,192 and of 32,768 tokens), which the default run adds")
    return ap.parse_args()


def build_model(cfg, seed):
    import torch
    from tffinfer_amd.models import build_model_skeleton, config_from_dict
    model = build_model_skeleton(config_from_dict(cfg))
    model.init_random(seed, torch.bfloat16, "cuda:0", on_device=True)
    torch.cuda.synchronize()
    return model


def large_points(args, gen) -> dict:
    """Two workloads at the larger shapes, each with a model of its own: 32 requests with prompts
    of 128 to 4,096 tokens in portions of 512 beside decoding requests at the 14B shape (all
    tokens, prompt and generated, a second), and decode steps of 16 requests at 8,192 tokens of
    context at the 32B shape (decoded tokens a second).  A point that fails is left null."""
    import gc
    import torch
    from tffinfer_amd import EngineOptions, LLMEngine
    from tffinfer_amd import measure as M
    out = {}

    def release():
        gc.collect()
        torch.cuda.empty_cache()

    try:
        cfg = dict(SHAPES["14b"][1])
        model = build_model(cfg, args.seed)
        opt = EngineOptions(dtype="bfloat16", page_size=args.page_size, kv_tokens=32 * (4096 + 256 + args.page_size),
                            max_num_seqs=32, prefill_chunk=512,      # (the token budget of a step: the engine's default)
                            max_model_len=cfg["max_position_embeddings"], use_graphs=not args.no_graphs)
        engine = LLMEngine(model, opt)
        # (a generator of its own: the same 32 prompts whatever was measured before, those of `--mixed 32 --shape 14b`)
        own = torch.Generator().manual_seed(args.seed)
        out["mixed32_14b_tokens_per_s"] = M.measure_mixed(engine, own, 32, cfg["vocab_size"])["total_tokens_per_s"]
        del engine, model
    except Exception as e:      # the headline figures must not be lost to a side measurement
        print(f"bench: the 14B point failed: {e}", file=sys.stderr)
        out["mixed32_14b_tokens_per_s"] = None
    release()
    try:
        cfg = dict(SHAPES["32b"][1])
        batch, context, steps, warmup = 16, 8192, 20, 4
        model = build_model(cfg, args.seed)
        total = steps + warmup + M.decode_slack(batch, context) + 16
        opt = EngineOptions(dtype="bfloat16", page_size=args.page_size,
                            kv_tokens=batch * (context + total + args.page_size), max_num_seqs=batch,
                            max_num_batched_tokens=4096, prefill_chunk=2048,
                            max_model_len=cfg["max_position_embeddings"], use_graphs=not args.no_graphs)
        engine = LLMEngine(model, opt)
        r = M.measure_decode(engine, gen, batch, context, steps, warmup, cfg["vocab_size"])
        out["decode_b16_ctx8192_32b"] = round(batch * steps / r["wall_s"], 1)
        del engine, model
    except Exception as e:
        print(f"bench: the 32B point failed: {e}", file=sys.stderr)
        out["decode_b16_ctx8192_32b"] = None
    release()
    return out


def long_points(args, model, cfg, gen) -> tuple[dict, dict]:
    """Further sizes at the benchmark shape, on an engine of their own whose length limit holds
    them (a decode graph's launches are sized for the limit, so the headline keeps its own):
    decode steps of 8 requests at 32,768 tokens of context, of 128 requests at 8,192 and of 64
    requests of which one has 32,768 tokens and the others 1,024 (as many keys as 64 requests of
    1,520), and prompts of 8,192 and 32,768 tokens in one step.  Returns (tokens a second, details) by
    point; a point that fails is left null."""
    import gc
    import torch
    from tffinfer_amd import EngineOptions, LLMEngine
    from tffinfer_amd import measure as M
    points, detail = {}, {}
    vocab = cfg["vocab_size"]
    L = cfg["num_hidden_layers"]
    for key, batch, context, steps, warmup in (("decode_b8_ctx32768", 8, 32768, 16, 4),
                                               ("decode_b128_ctx8192", 128, 8192, 12, 4),
                                               ("decode_b64_ctx1024_one_of_32768", 64, [32768] + [1024] * 63, 16, 4)):
        try:
            longest = max(context) if isinstance(context, list) else context
            mean = sum(context) / batch if isinstance(context, list) else context
            total = steps + warmup + M.decode_slack(batch, longest) + 16
            opt = EngineOptions(dtype="bfloat16", page_size=args.page_size,
                                kv_tokens=int(batch * (mean + total + args.page_size)), max_num_seqs=batch,
                                max_num_batched_tokens=4096, prefill_chunk=2048, max_model_len=longest + total + 16,
                                use_graphs=not args.no_graphs)
            engine = LLMEngine(model, opt)
            r = M.measure_decode(engine, gen, batch, context, steps, warmup, vocab)
            step = r["wall_s"] / steps
            nbytes = M.decode_bytes(model, batch, mean + warmup + steps / 2.0)
            points[key] = round(batch / step, 1)
            detail[key] = {"ms_per_step": round(1e3 * step, 4), "ms_per_step_median": round(1e3 * r["step_median_s"], 4),
                           "frac": round(nbytes / step / 1e9 / M.HBM_PEAK_GBS, 4)}
            del engine
        except Exception as e:      # the headline figures must not be lost to a side measurement
            print(f"bench: the point {key} failed: {e}", file=sys.stderr)
            points[key] = None
        gc.collect()
        torch.cuda.empty_cache()
    for key, T, reps in (("prefill_8192", 8192, 4), ("prefill_32768", 32768, 2)):
        try:
            opt = EngineOptions(dtype="bfloat16", page_size=args.page_size, kv_tokens=T + args.page_size, max_num_seqs=1,
                                max_num_batched_tokens=T, prefill_chunk=T, max_model_len=T + 16,
                                use_graphs=False)
            engine = LLMEngine(model, opt)
            r = M.measure_prefill(engine, gen, T, vocab, reps=reps, warm=1)
            points[key] = round(T / r["wall_s"], 1)
            detail[key] = {"ms": round(1e3 * r["wall_s"], 3), "ms_device": round(1e3 * r["device_s"], 3),
                           "frac": round(M.prefill_flops(model, T) / r["wall_s"] / M.MFMA_PEAK["bf16"], 4)}
            del engine
        except Exception as e:
            print(f"bench: the point {key} failed: {e}", file=sys.stderr)
            points[key] = None
        gc.collect()
        torch.cuda.empty_cache()
    return points, detail


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on a single GPU)")
        sys.exit(2)
    import torch
    from tffinfer_amd import EngineOptions, LLMEngine
    from tffinfer_amd import measure as M
    from tffinfer_amd.kernels import lib as kernel_lib

    kernel_lib.load()
    if args.ceilings:
        from tffinfer_amd.kernels import ops
        c = ops.measure_ceilings("cuda:0")
        c.update(M.square_product_rates("cuda:0"))
        print(json.dumps({"ceilings": c,
                          "published": {"hbm_GBps": M.HBM_PEAK_GBS, "bf16_TFLOPs": M.MFMA_PEAK["bf16"] / 1e12}}))
        return
    contexts = None
    if args.contexts:
        if args.only != "decode":
            raise SystemExit("--contexts goes with --only decode")
        contexts = []
        for part in args.contexts.split(","):
            n, _, c = part.rpartition("x")
            contexts += [int(c)] * (int(n) if n else 1)
        args.batch, args.context = len(contexts), max(contexts)
    shape_name, shape = SHAPES[args.shape]
    cfg = dict(shape)
    L_full = cfg["num_hidden_layers"]
    L = args.layers or L_full
    cfg["num_hidden_layers"] = L
    # a context beyond the shape's own limit: the limit grows with it (it sizes the rotation table only)
    longest = max(args.prefill_tokens,
                  args.context + args.steps + args.warmup + M.decode_slack(max(args.batch, 64), args.context) + 16)
    want_long = (args.shape == "8b" and args.layers is None and not args.only and not args.no_points
                 and not args.no_long_points and not args.mixed)
    if not args.mixed and longest > cfg["max_position_embeddings"]:
        cfg["max_position_embeddings"] = 1 << (longest - 1).bit_length()
    headline_limit = cfg["max_position_embeddings"]
    if want_long:
        # the model's own limit sizes the rotation table only; every engine below has its own
        cfg["max_position_embeddings"] = max(headline_limit, 65536)
    vocab = cfg["vocab_size"]
    gen = torch.Generator().manual_seed(args.seed)
    model = build_model(cfg, args.seed)
    if args.mixed:
        kv_tokens = args.mixed * (4096 + 256 + args.page_size)
        budget = {"max_num_batched_tokens": max(args.budget, args.chunk, args.mixed)} if args.budget else {}
        opt = EngineOptions(dtype="bfloat16", page_size=args.page_size, kv_tokens=kv_tokens,
                            max_num_seqs=args.mixed, prefill_chunk=args.chunk, max_model_len=cfg["max_position_embeddings"],
                            use_graphs=not args.no_graphs, token_quantum=args.token_quantum, **budget)
        engine = LLMEngine(model, opt)
        res = M.measure_mixed(engine, gen, args.mixed, vocab)
        print(json.dumps({"workload": "mixed", "model": shape_name, "layers_run": L, "chunk": args.chunk,
                          "budget": opt.max_num_batched_tokens, **res}))
        return
    max_batch = args.batch if (args.no_points or args.only) else max(args.batch, 64)
    total_steps = args.steps + args.warmup + M.decode_slack(max_batch, args.context) + 16
    kv_tokens = max_batch * (args.context + total_steps + args.page_size) + args.prefill_tokens
    if contexts:
        kv_tokens = sum(contexts) + max_batch * (total_steps + args.page_size)
    opt = EngineOptions(dtype="bfloat16", page_size=args.page_size, kv_tokens=kv_tokens, max_num_seqs=max_batch,
                        max_num_batched_tokens=max(4096, max_batch), prefill_chunk=2048,
                        max_model_len=headline_limit, use_graphs=not args.no_graphs)
    engine = LLMEngine(model, opt)

    pre = dec = None
    if args.only != "decode":
        pre = M.measure_prefill(engine, gen, args.prefill_tokens, vocab)
    if args.only != "prefill":
        sampling = None
        if args.sampling:
            if args.only != "decode":
                raise SystemExit("--sampling goes with --only decode (the benchmark line is greedy decoding)")
            from tffinfer_amd.sampling import SamplingConfig
            k, p, t, *rest = args.sampling.split(",")
            sampling = SamplingConfig(type="top_p", top_k=int(k), top_p=float(p), temperature=float(t), seed=args.seed,
                                      repetition_penalty=float(rest[0]) if rest else 1.0)
        dec = M.measure_decode(engine, gen, args.batch, contexts or args.context, args.steps, args.warmup, vocab, sampling)
    if args.only:
        part = ({"prefill_ms": round(1000 * pre["wall_s"], 3), "prefill_ms_device": round(1000 * pre["device_s"], 3)}
                if pre else
                {"decode_ms_per_step": round(1000 * dec["wall_s"] / args.steps, 4),
                 "decode_ms_per_step_median": round(1000 * dec["step_median_s"], 4)})
        if args.sampling:
            part["sampling"] = args.sampling
        print(json.dumps({"only": args.only, **part, "batch": args.batch, "context": args.contexts or args.context}))
        return
    points, detail = {}, {}
    if not args.no_points:
        for b, key in ((1, "decode_b1"), (64, "decode_b64")):
            k = min(args.steps, 32)
            w = min(args.warmup, 4)
            r = M.measure_decode(engine, gen, b, args.context, k, w, vocab)
            points[key] = round(b * k / r["wall_s"], 1)
            nb = M.decode_bytes(model, b, args.context + w + k / 2.0)
            detail[key] = {"ms_per_step": round(1e3 * r["wall_s"] / k, 4),
                           "ms_per_step_median": round(1e3 * r["step_median_s"], 4),
                           "frac": round(nb / (r["wall_s"] / k) / 1e9 / M.HBM_PEAK_GBS, 4)}
        # the headline batch again with every request drawing from the top 50 tokens at top-p 0.95 and
        # temperature 0.8 instead of taking the most likely one
        from tffinfer_amd.sampling import SamplingConfig
        k = min(args.steps, 32)
        r = M.measure_decode(engine, gen, args.batch, args.context, k, min(args.warmup, 4), vocab,
                             SamplingConfig(type="top_p", top_k=50, top_p=0.95, temperature=0.8, seed=args.seed))
        points[f"decode_b{args.batch}_top_k50_top_p0.95"] = round(args.batch * k / r["wall_s"], 1)
    ceilings = M.quick_ceilings("cuda:0")

    t_decode, t_prefill = dec["wall_s"], pre["wall_s"]
    ms_step = 1000.0 * t_decode / args.steps
    value = args.batch * args.steps / t_decode
    mean_context = args.context + args.warmup + args.steps / 2.0
    nbytes = M.decode_bytes(model, args.batch, mean_context)
    achieved = nbytes / (t_decode / args.steps) / 1e9
    pf = M.prefill_flops(model, args.prefill_tokens)
    out = {
        "metric": "decode_tokens_per_s", "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        # the same steps by device events, step by step: their median (the wall clock above is their mean
        # plus what the host adds)
        "ms_per_step_median": round(1000.0 * dec["step_median_s"], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (seeded random weights and token ids)",
        "config": {
            "model": shape_name, "layers": L_full, "layers_run": L, "hidden": cfg["hidden_size"],
            "q_heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["head_dim"], "intermediate": cfg["intermediate_size"], "vocab": vocab,
            "rope_theta": cfg["rope_theta"], "rms_norm_eps": cfg["rms_norm_eps"],
            "max_context": headline_limit, "global_batch": args.batch,
            "seq_len": args.context, "prefill_tokens": args.prefill_tokens, "page_size": args.page_size,
            "hip_graphs": not args.no_graphs, "parallelism": "single GPU",
        },
        "prefill": {"value": round(args.prefill_tokens / t_prefill, 1), "tokens": args.prefill_tokens,
                    "ms": round(1000.0 * t_prefill, 3), "frac": round(pf / t_prefill / M.MFMA_PEAK["bf16"], 4),
                    "ms_device": round(1000.0 * pre["device_s"], 3),
                    "frac_of_measured": round(pf / t_prefill / (ceilings["mfma_bf16_TFLOPs"] * 1e12), 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": M.HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / M.HBM_PEAK_GBS, 4),
                     "frac_of_measured": round(achieved / ceilings["stream_read_GBps"], 4)},
        # what this machine gives, in this process, to a kernel that only reads and to one that only
        # issues bfloat16 MFMAs from registers
        "ceilings": ceilings,
        "points": points,
        # per point: the step's (or the prompt's) time and its share of the published peak (HBM for decode
        # steps, bf16 MFMA for prompts)
        "points_detail": detail,
    }
    if want_long:
        del engine
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        engine = None
        lp, ld = long_points(args, model, cfg, gen)
        out["points"].update(lp)
        out["points_detail"].update(ld)
    if args.shape == "8b" and args.layers is None and not args.no_points and not args.no_large_points:
        del engine, model
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        out["points"].update(large_points(args, gen))
    print(json.dumps(out))


if __name__ == "__main__":
    main()
