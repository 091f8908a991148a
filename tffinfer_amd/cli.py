"""Command line: generate from token ids with a model folder.

The reference's programs take the model path as their first argument and keep
everything else in constants (test/main.cu:17-66: ``n_predict = 64``,
``max_batches = 1``, the options of its ModelConfig;
example/load_model/load_model.cu:8-25 stops after loading).  Here the model
path is still the first argument and those constants are options under the
reference's names.
"""
from __future__ import annotations

import argparse
import json
import sys
import time


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="tffinfer", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("model", help="model folder: config.json and model.safetensors")
    ap.add_argument("--load-only", action="store_true",
                    help="load the model and stop (example/load_model of the reference)")
    g = ap.add_argument_group("model options (the reference's ModelConfig)")
    g.add_argument("--use-f16", dest="use_f16", action="store_true", default=True,
                   help="16-bit path, bfloat16 here (_use_f16, default)")
    g.add_argument("--no-use-f16", "--fp32", dest="use_f16", action="store_false",
                   help="true 32-bit path of the whole model")
    g.add_argument("--n-ctx", type=int, default=8192, help="longest sequence (_n_ctx)")
    g.add_argument("--rope-freq-base", type=float, default=None,
                   help="rotation base; default: config.json's rope_theta (_rope_freq_base)")
    g = ap.add_argument_group("requests")
    g.add_argument("--prompt-ids", action="append", default=[],
                   help="a prompt as comma-separated token ids; may be given several times")
    g.add_argument("--prompt-file", help="file with one prompt per line (ids separated by spaces or commas)")
    g.add_argument("--random-prompts", help="N:LEN, N random prompts of LEN tokens (seeded by --seed)")
    g.add_argument("--n-predict", type=int, default=64, help="new tokens per prompt (n_predict, 64)")
    g.add_argument("--max-batches", type=int, default=8, help="most sequences in flight (max_batches)")
    g.add_argument("--eos-id", type=int, default=None, help="token that ends a generation")
    g.add_argument("--ignore-eos", action="store_true")
    g = ap.add_argument_group("sampling (the reference's SamplingConfig)")
    g.add_argument("--sample-type", default="greedy", choices=["default", "greedy", "random", "top_k", "top_p"])
    g.add_argument("--temperature", type=float, default=1.0)
    g.add_argument("--top-k", type=int, default=0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--min-p", type=float, default=0.0)
    g.add_argument("--repetition-penalty", type=float, default=1.0)
    g.add_argument("--seed", type=int, default=0)
    g = ap.add_argument_group("engine")
    g.add_argument("--page-size", type=int, default=16)
    g.add_argument("--kv-tokens", type=int, default=None, help="tokens the cache holds")
    g.add_argument("--max-batch-tokens", type=int, default=2048, help="token budget of a step")
    g.add_argument("--prefill-chunk", type=int, default=512, help="longest portion of a prompt in a step")
    g.add_argument("--json", action="store_true", help="print one JSON object per prompt")
    return ap


def _parse_ids(text: str) -> list[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    from .runtime import LLMInferRuntime, ModelConfig
    from .sampling import SamplingConfig

    cfg = ModelConfig()
    cfg._use_f16 = args.use_f16
    cfg._n_ctx = args.n_ctx
    cfg._rope_freq_base = args.rope_freq_base
    cfg._page_size = args.page_size
    cfg._max_batches = args.max_batches
    cfg._max_batch_tokens = args.max_batch_tokens
    cfg._prefill_chunk = args.prefill_chunk
    cfg._kv_tokens = args.kv_tokens
    stype = args.sample_type
    if stype == "greedy" and (args.temperature != 1.0 or args.top_k or args.top_p < 1 or args.min_p > 0):
        stype = "random"   # sampling options without a type mean a random draw
    cfg._sampling_config = SamplingConfig(stype, args.temperature, args.top_k, args.top_p, args.min_p,
                                          args.repetition_penalty, args.seed)
    rt = LLMInferRuntime()
    t0 = time.time()
    rt.load_model([args.model], cfg)
    print(f"loaded {args.model} in {time.time() - t0:.1f} s", file=sys.stderr)
    if args.load_only:
        return 0
    if not rt.init_runtime_context():
        print("init_runtime_context failed", file=sys.stderr)
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
        print("no prompt given (--prompt-ids, --prompt-file or --random-prompts)", file=sys.stderr)
        return 1
    rt.encode(prompts)
    eng = rt.engine
    t0 = time.time()
    res = eng.generate(prompts, cfg._sampling_config, max_new_tokens=args.n_predict,
                       eos_token_id=args.eos_id, ignore_eos=args.ignore_eos)
    dt = time.time() - t0
    for r in res:
        if args.json:
            print(json.dumps({"prompt": r.prompt, "output": r.output, "finish_reason": r.finish_reason}))
        else:
            print(" ".join(str(t) for t in r.output))
    n_out = sum(len(r.output) for r in res)
    st = eng.scheduler.stats
    print(f"{n_out} tokens in {dt:.2f} s ({n_out / max(dt, 1e-9):.1f} tok/s), {st.steps} steps, "
          f"{st.preemptions} preemptions", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
