"""Command line in the manner of the reference's example.py and bench.py: the engine's
options carry the names of its Config fields (nanovllm/config.py:6-19), the sampling
options those of SamplingParams (nanovllm/sampling_params.py:4-11).

    python -m nano_vllm_amd.cli generate --model DIR --prompt-ids 1,2,3 [--prompt "text"] ...
    python -m nano_vllm_amd.cli random-model --config config.json --seed 0 --out DIR
    python -m nano_vllm_amd.cli throughput --model DIR [--random-weights SEED] --num-seqs 256 ...
"""
from __future__ import annotations

import argparse
import json
import sys


def add_engine_options(ap: argparse.ArgumentParser) -> None:
    ap.add_argument("--model", required=True, help="folder with config.json and *.safetensors")
    ap.add_argument("--max-num-batched-tokens", type=int, default=16384)
    ap.add_argument("--max-num-seqs", type=int, default=512)
    ap.add_argument("--max-model-len", type=int, default=4096)
    ap.add_argument("--gpu-memory-utilization", type=float, default=0.9)
    ap.add_argument("--enforce-eager", action="store_true")
    ap.add_argument("--kvcache-block-size", type=int, default=256)
    ap.add_argument("--num-kvcache-blocks", type=int, default=-1)
    ap.add_argument("--dtype", default=None, choices=[None, "bfloat16", "float32"])
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--schedule", default="prefill_first", choices=["prefill_first", "mixed"])
    ap.add_argument("--no-prefix-caching", action="store_true")
    ap.add_argument("--decode-burst", type=int, default=16, help="decode steps in a row without the host (1: never)")
    ap.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                    help="draw the weights on the device from this seed: the folder needs config.json only")


def engine_kwargs(args) -> dict:
    return dict(max_num_batched_tokens=args.max_num_batched_tokens, max_num_seqs=args.max_num_seqs,
                max_model_len=args.max_model_len, gpu_memory_utilization=args.gpu_memory_utilization,
                enforce_eager=args.enforce_eager, kvcache_block_size=args.kvcache_block_size,
                num_kvcache_blocks=args.num_kvcache_blocks, dtype=args.dtype, seed=args.seed,
                schedule=args.schedule, enable_prefix_caching=not args.no_prefix_caching,
                random_weights=args.random_weights, decode_burst=args.decode_burst)


def cmd_generate(args) -> int:
    from . import LLM, SamplingParams
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids] + list(args.prompt)
    if not prompts:
        print("give at least one --prompt-ids or --prompt", file=sys.stderr)
        return 2
    llm = LLM(args.model, **engine_kwargs(args))
    sp = SamplingParams(temperature=args.temperature, max_tokens=args.max_tokens, ignore_eos=args.ignore_eos)
    outs = llm.generate(prompts, sp, use_tqdm=not args.json)
    if args.json:
        print(json.dumps(outs))
    else:
        for p, o in zip(prompts, outs):
            print(f"\nPrompt: {p!r}")
            print(f"Completion: {o['text']!r}" if o["text"] is not None else f"Completion ids: {o['token_ids']}")
    return 0


def cmd_throughput(args) -> int:
    """The workload of the reference's bench.py (bench.py:9-28 there): num_seqs requests of
    random token ids, prompt and output lengths uniform in [min, max], sampled at a
    temperature with ignore_eos, after one short warm-up request; prints the reference's line
    (generated tokens, seconds, tokens a second) and, with --json, the engine's own counts."""
    import random
    import time
    from . import LLM, SamplingParams
    for what, low, high in (("input", args.min_input_len, args.max_input_len),
                            ("output", args.min_output_len, args.max_output_len)):
        if not 1 <= low <= high:
            print(f"throughput: --min-{what}-len {low} and --max-{what}-len {high} must satisfy 1 <= min <= max",
                  file=sys.stderr)
            return 2
    rng = random.Random(args.workload_seed)
    llm = LLM(args.model, **engine_kwargs(args))
    vocab = llm.model.spec.vocab_size
    top = min(vocab, args.max_token_id)
    prompts = [[rng.randrange(top) for _ in range(rng.randint(args.min_input_len, args.max_input_len))]
               for _ in range(args.num_seqs)]
    params = [SamplingParams(temperature=args.temperature, ignore_eos=True,
                             max_tokens=rng.randint(args.min_output_len, args.max_output_len))
              for _ in range(args.num_seqs)]
    llm.generate([[1, 2, 3, 4]], SamplingParams(temperature=args.temperature, max_tokens=8, ignore_eos=True),
                 use_tqdm=False)
    for k in llm.stats:
        llm.stats[k] = 0 if isinstance(llm.stats[k], int) else 0.0
    t0 = time.perf_counter()
    llm.generate(prompts, params, use_tqdm=False)
    dt = time.perf_counter() - t0
    total = sum(p.max_tokens for p in params)
    print(f"Total: {total}tok, Time: {dt:.2f}s, Throughput: {total / dt:.2f}tok/s")
    if args.json:
        print(json.dumps({"generated_tokens": total, "prompt_tokens": sum(len(p) for p in prompts), "seconds": dt,
                          "tokens_per_second": total / dt, "num_seqs": args.num_seqs, **llm.stats}))
    return 0


def cmd_random_model(args) -> int:
    from .weights import write_random_model
    import os
    if (args.config is None) == (args.shape is None):
        print("give either --config FILE or --shape NAME", file=sys.stderr)
        return 2
    if args.shape is not None:
        from .models.shapes import shape
        config = shape(args.shape)
    else:
        with open(args.config) as f:
            config = json.load(f)
    if args.config_only:                 # for engines started with random_weights: the weights are drawn on the device
        if args.dtype:
            config["torch_dtype"] = args.dtype
        os.makedirs(args.out, exist_ok=True)
        with open(os.path.join(args.out, "config.json"), "w") as f:
            json.dump(config, f, indent=2)
        print(f"wrote {args.out}/config.json")
        return 0
    write_random_model(args.out, config, args.seed, std=args.std, norm_std=args.norm_std, dtype=args.dtype)
    print(f"wrote {args.out}/config.json and {args.out}/model.safetensors")
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="nano_vllm_amd")
    sub = ap.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("generate", help="generate from prompts (example.py of the reference)")
    add_engine_options(g)
    g.add_argument("--prompt", action="append", default=[], help="a text prompt (needs the folder's tokenizer)")
    g.add_argument("--prompt-ids", action="append", default=[], help="a prompt as comma-separated token ids")
    g.add_argument("--temperature", type=float, default=0.6)
    g.add_argument("--max-tokens", type=int, default=256)
    g.add_argument("--ignore-eos", action="store_true")
    g.add_argument("--json", action="store_true", help="print the outputs as one JSON line")
    g.set_defaults(fn=cmd_generate)
    t = sub.add_parser("throughput", help="requests of random tokens through generate (bench.py of the reference)")
    add_engine_options(t)
    t.add_argument("--num-seqs", type=int, default=256)
    t.add_argument("--min-input-len", type=int, default=100)
    t.add_argument("--max-input-len", type=int, default=1024)
    t.add_argument("--min-output-len", type=int, default=100)
    t.add_argument("--max-output-len", type=int, default=1024)
    t.add_argument("--max-token-id", type=int, default=10000, help="prompt ids are drawn below this (and the vocabulary)")
    t.add_argument("--temperature", type=float, default=0.6)
    t.add_argument("--workload-seed", type=int, default=0)
    t.add_argument("--json", action="store_true", help="also print the counts as one JSON line")
    t.set_defaults(fn=cmd_throughput)
    r = sub.add_parser("random-model", help="write a model folder with seeded random weights")
    r.add_argument("--config", default=None, help="a config.json of the architecture")
    r.add_argument("--shape", default=None, help="a named shape instead: tiny-a, tiny-b, qwen3-0.6b, qwen3-1.7b, qwen3-4b, qwen3-8b, qwen3-14b, qwen3-32b")
    r.add_argument("--config-only", action="store_true", help="write config.json only (for --random-weights)")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--out", required=True)
    r.add_argument("--std", type=float, default=0.02)
    r.add_argument("--norm-std", type=float, default=0.0, help="norm weights are 1 + N(0, this)")
    r.add_argument("--dtype", default=None, choices=[None, "bfloat16", "float32"])
    r.set_defaults(fn=cmd_random_model)
    args = ap.parse_args(argv)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
