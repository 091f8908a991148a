"""Command line: generate from token ids with a model folder, or with seeded
random weights for a configuration file; dump the logits; measure.

The reference's programs take the model path as their first argument and keep
everything else in constants (test/main.cu:17-66: ``n_predict = 64``,
``max_batches = 1``, the options of its ModelConfig; a second argument for a
configuration file is commented out there, :19;
example/load_model/load_model.cu:8-25 stops after loading).  Here the model
path is still the first argument and those constants are options under the
reference's names.

    tffinfer MODEL_DIR --prompt-ids 1,2,3 --n-predict 16
    tffinfer --config config.json --random-weights --seed 7 --random-prompts 2:40 --dump-logits out.f32
    tffinfer --config config.json --random-weights --bench decode --batch 8 --context 2048 --gen 64
"""
from __future__ import annotations

import argparse
import json
import sys
import time

from . import log


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="tffinfer", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("model", nargs="?", default=None, help="model folder: config.json and model.safetensors")
    ap.add_argument("--load-only", action="store_true",
                    help="load the model and stop (example/load_model of the reference)")
    g = ap.add_argument_group("random weights instead of a model folder")
    g.add_argument("--config", metavar="FILE", help="a config.json; needs --random-weights")
    g.add_argument("--random-weights", action="store_true",
                   help="weights drawn from --seed (matrices N(0, 0.02), norm weights 1 + N(0, 0.1))")
    g.add_argument("--random-on-device", action="store_true",
                   help="draw them on the GPU (another stream of numbers; for large models)")
    g.add_argument("--save-model", metavar="DIR",
                   help="also write config.json and model.safetensors with these weights to DIR")
    g = ap.add_argument_group("model options (the reference's ModelConfig)")
    g.add_argument("--use-f16", dest="use_f16", action="store_true", default=True,
                   help="16-bit path, bfloat16 here (_use_f16, default)")
    g.add_argument("--no-use-f16", "--fp32", dest="use_f16", action="store_false",
                   help="true 32-bit path of the whole model")
    g.add_argument("--dtype", choices=["bf16", "bfloat16", "fp32", "float32"], default=None,
                   help="the same choice by name")
    g.add_argument("--device", default="hip", help="hip (or cuda:0): the GPU; there is no other path")
    g.add_argument("--n-ctx", type=int, default=8192, help="longest sequence (_n_ctx)")
    g.add_argument("--rope-freq-base", type=float, default=None,
                   help="rotation base; default: config.json's rope_theta (_rope_freq_base)")
    g = ap.add_argument_group("requests")
    g.add_argument("--prompt-ids", action="append", default=[],
                   help="a prompt as comma-separated token ids; may be given several times")
    g.add_argument("--prompt-file", help="file with one prompt per line (ids separated by spaces or commas)")
    g.add_argument("--random-prompts", help="N:LEN, N random prompts of LEN tokens (seeded by --seed)")
    g.add_argument("--n-predict", "--max-new-tokens", dest="n_predict", type=int, default=64,
                   help="new tokens per prompt (n_predict, 64)")
    g.add_argument("--max-batches", "--max-num-seqs", dest="max_batches", type=int, default=8,
                   help="most sequences in flight (max_batches)")
    g.add_argument("--eos-id", type=int, default=None, help="token that ends a generation")
    g.add_argument("--ignore-eos", action="store_true")
    g = ap.add_argument_group("sampling (the reference's SamplingConfig)")
    g.add_argument("--sample-type", default="greedy", choices=["default", "greedy", "random", "top_k", "top_p"])
    g.add_argument("--temperature", type=float, default=1.0)
    g.add_argument("--top-k", type=int, default=0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--min-p", type=float, default=0.0)
    g.add_argument("--repetition-penalty", type=float, default=1.0)
    g.add_argument("--seed", type=int, default=0, help="seed of random weights and random prompts")
    g.add_argument("--sample-seed", type=int, default=None, help="seed of the random draws (default: --seed)")
    g = ap.add_argument_group("engine")
    g.add_argument("--page-size", type=int, default=16)
    g.add_argument("--kv-tokens", type=int, default=None, help="tokens the cache holds, or")
    g.add_argument("--num-pages", type=int, default=None, help="pages of every group of layers, or")
    g.add_argument("--kv-bytes", type=int, default=None, help="bytes of device memory for keys and values")
    g.add_argument("--max-batch-tokens", "--max-batched-tokens", dest="max_batch_tokens", type=int, default=2048,
                   help="token budget of a step")
    g.add_argument("--prefill-chunk", type=int, default=512, help="longest portion of a prompt in a step")
    g.add_argument("--no-graphs", action="store_true", help="launch decode steps kernel by kernel")
    g.add_argument("--warm-up", action="store_true",
                   help="capture the decode graphs of all batch sizes before the first request")
    g = ap.add_argument_group("output")
    g.add_argument("--json", action="store_true", help="print one JSON object per prompt")
    g.add_argument("--dump-logits", metavar="FILE",
                   help="float32 logits of every sampled position, little-endian [positions, vocab]: the prompts "
                        "in the order given, each one's positions in order; FILE.json says which rows are whose")
    g.add_argument("--log-level", default=None, help="debug, info, warning, error, off (default: info, or $TFFINFER_LOG)")
    g = ap.add_argument_group("measuring (one JSON line; no generation)")
    g.add_argument("--bench", choices=["decode", "prefill"], help="decode steps of --batch requests at --context "
                   "tokens each, or one prompt of --context tokens")
    g.add_argument("--batch", type=int, default=8)
    g.add_argument("--context", type=int, default=2048)
    g.add_argument("--gen", type=int, default=64, help="decode steps that are timed (prefill: repetitions)")
    return ap


def _parse_ids(text: str) -> list[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def _bench(args, rt, cfg) -> int:
    """``--bench``: the functions that ``bench.py`` uses, on the model just loaded."""
    import torch
    from . import measure as M
    from .engine.llm_engine import EngineOptions, LLMEngine
    model = rt._model
    mc = model.config
    vocab = mc.vocab_size
    gen = torch.Generator().manual_seed(args.seed)
    dtype = "bf16" if args.use_f16 else "fp32"
    warmup = 4
    if args.bench == "decode":
        total = args.gen + warmup + M.decode_slack(args.batch, args.context) + 16
        if args.context + total > mc.max_position_embeddings:
            log.error("--context %d plus %d steps exceed the model's %d positions", args.context, total,
                      mc.max_position_embeddings)
            return 1
        kv_tokens = args.batch * (args.context + total + args.page_size)
        chunk = 2048
    else:
        if args.context > mc.max_position_embeddings:
            log.error("--context %d exceeds the model's %d positions", args.context, mc.max_position_embeddings)
            return 1
        kv_tokens, chunk = args.context + args.page_size, args.context
    opt = EngineOptions(dtype=model.dtype, page_size=args.page_size, max_num_seqs=max(1, args.batch),
                        max_num_batched_tokens=max(4096, args.batch, chunk), prefill_chunk=chunk,
                        max_model_len=mc.max_position_embeddings, use_graphs=not args.no_graphs, warm_up=args.warm_up,
                        kv_tokens=None if (args.num_pages or args.kv_bytes) else kv_tokens,
                        num_pages=args.num_pages, kv_bytes=args.kv_bytes)
    engine = LLMEngine(model, opt)
    rec = {"bench": args.bench, "dtype": dtype, "batch": args.batch, "context": args.context}
    if args.bench == "decode":
        r = M.measure_decode(engine, gen, args.batch, args.context, args.gen, warmup, vocab)
        step = r["wall_s"] / args.gen
        rec.update(steps=args.gen, tokens_per_s=round(args.batch / step, 1), ms_per_step=round(1e3 * step, 4),
                   ms_per_step_median=round(1e3 * r["step_median_s"], 4))
        nbytes = M.decode_bytes(model, args.batch, args.context + warmup + args.gen / 2.0, 2 if args.use_f16 else 4)
        rec["hbm_GBps"] = round(nbytes / step / 1e9, 1)
        rec["hbm_frac"] = round(nbytes / step / 1e9 / M.HBM_PEAK_GBS, 4)
    else:
        r = M.measure_prefill(engine, gen, args.context, vocab, reps=max(1, min(args.gen, 20)))
        flops = M.prefill_flops(model, args.context)
        rec.update(tokens_per_s=round(args.context / r["wall_s"], 1), ms=round(1e3 * r["wall_s"], 3),
                   ms_device=round(1e3 * r["device_s"], 3),
                   mfma_frac=round(flops / r["wall_s"] / M.MFMA_PEAK[dtype], 6))
    print(json.dumps(rec))
    return 0


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    log.init("tffinfer", args.log_level)
    from .runtime import LLMInferRuntime, ModelConfig
    from .sampling import SamplingConfig

    if args.dtype is not None:
        args.use_f16 = args.dtype in ("bf16", "bfloat16")
    if args.device not in ("hip", "gpu", "cuda", "cuda:0"):
        log.error("--device %s: the engine runs on the GPU only (hip); it has no CPU path", args.device)
        return 2
    if bool(args.model) == bool(args.config):
        log.error("give a model folder, or --config FILE --random-weights")
        return 2
    if args.config and not args.random_weights:
        log.error("--config FILE names no weights: add --random-weights (and --seed N)")
        return 2
    if sum(x is not None for x in (args.kv_tokens, args.num_pages, args.kv_bytes)) > 1:
        log.error("give one of --kv-tokens, --num-pages and --kv-bytes")
        return 2

    cfg = ModelConfig()
    cfg._use_f16 = args.use_f16
    cfg._n_ctx = args.n_ctx
    cfg._rope_freq_base = args.rope_freq_base
    cfg._page_size = args.page_size
    cfg._max_batches = args.max_batches
    cfg._max_batch_tokens = args.max_batch_tokens
    cfg._prefill_chunk = args.prefill_chunk
    cfg._kv_tokens = args.kv_tokens
    cfg._num_pages = args.num_pages
    cfg._kv_bytes = args.kv_bytes
    cfg._use_graphs = not args.no_graphs
    cfg._warm_up = args.warm_up
    stype = args.sample_type
    if stype == "greedy" and (args.temperature != 1.0 or args.top_k or args.top_p < 1 or args.min_p > 0):
        stype = "random"   # sampling options without a type mean a random draw
    sample_seed = args.seed if args.sample_seed is None else args.sample_seed
    cfg._sampling_config = SamplingConfig(stype, args.temperature, args.top_k, args.top_p, args.min_p,
                                          args.repetition_penalty, sample_seed)
    rt = LLMInferRuntime()
    t0 = time.time()
    if args.config:
        if args.save_model:
            from .weights import write_random_model
            with open(args.config) as f:
                write_random_model(args.save_model, json.load(f), args.seed)
            log.info("wrote %s", args.save_model)
        rt.random_model(args.config, args.seed, cfg, on_device=args.random_on_device)
        log.info("random weights for %s from seed %d in %.1f s", args.config, args.seed, time.time() - t0)
    else:
        rt.load_model([args.model], cfg)
        log.info("loaded %s in %.1f s", args.model, time.time() - t0)
    if args.load_only:
        return 0
    if args.bench:
        return _bench(args, rt, cfg)
    if not rt.init_runtime_context():
        log.error("init_runtime_context failed")
        return 1
    prompts = [_parse_ids(p) for p in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts += [_parse_ids(line) for line in f if line.strip()]
    if args.random_prompts:
        import torch
        n, length = (int(x) for x in args.random_prompts.split(":"))
        gen = torch.Generator().manual_seed(args.seed)
        V = rt.engine.model.config.vocab_size
        prompts += [torch.randint(0, V, (length,), generator=gen).tolist() for _ in range(n)]
    if not prompts:
        log.error("no prompt given (--prompt-ids, --prompt-file or --random-prompts)")
        return 1
    rt.encode(prompts)
    eng = rt.engine
    eng.keep_logits = bool(args.dump_logits)
    t0 = time.time()
    res = eng.generate(prompts, cfg._sampling_config, max_new_tokens=args.n_predict,
                       eos_token_id=args.eos_id, ignore_eos=args.ignore_eos)
    dt = time.time() - t0
    for r in res:
        if args.json:
            print(json.dumps({"prompt": r.prompt, "output": r.output, "finish_reason": r.finish_reason}))
        else:
            print(" ".join(str(t) for t in r.output))
    if args.dump_logits:
        import torch
        rows = [row for r in res for row in r.logits]
        index, at = [], 0
        for i, r in enumerate(res):
            # row j of a prompt holds the logits at position len(prompt) - 1 + j, which chose output j
            index.append({"prompt": i, "first_row": at, "rows": len(r.logits), "first_position": len(r.prompt) - 1})
            at += len(r.logits)
        V = eng.model.config.vocab_size
        data = torch.stack(rows).to(torch.float32).contiguous() if rows else torch.empty(0, V)
        with open(args.dump_logits, "wb") as f:
            f.write(data.numpy().astype("<f4", copy=False).tobytes())
        with open(args.dump_logits + ".json", "w") as f:
            json.dump({"dtype": "float32", "shape": [at, V], "requests": index}, f)
        log.info("wrote %d rows of %d logits to %s", at, V, args.dump_logits)
    n_out = sum(len(r.output) for r in res)
    st = eng.scheduler.stats
    log.info("%d tokens in %.2f s (%.1f tok/s), %d steps, %d preemptions", n_out, dt, n_out / max(dt, 1e-9),
             st.steps, st.preemptions)
    log.exit()
    return 0


if __name__ == "__main__":
    sys.exit(main())
