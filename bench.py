#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

The default run has the layer sizes of the Qwen3-8B shape (36 layers, hidden 4096, 32 query
and 8 kv heads of 128, inner 12288, vocabulary 151936, bfloat16) with seeded random weights,
a batch of 8 requests and a context of 4096 tokens: after W untimed steps, K decode steps
(one token per request and step, through the engine's step function and sampler) are timed
so that the last one ends at the context length.  The cache in front of the timed steps is
filled with random keys and values (a decode step's work does not depend on their values).
Also measured: a prefill of 2,048 tokens, decoding at batch 1 and 64, decoding at the default
batch with a context of 32,768 tokens, and ("serve_256") the reference's own benchmark workload
(bench.py:8-28 there: 256 requests of random ids, prompts and outputs of 100 to 1024 tokens,
temperature 0.6, ignore_eos, one `generate` call after a short warm-up request) through
`LLM.generate`: scheduler, chunked prefill, sampling and the host's round trips included.

One JSON line is printed: `value` is decoded tokens a second at the default batch.
The reference measures throughput the same way on synthetic token ids (bench.py:8-28 there).
"""
import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0                      # MI355X HBM3E, published
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}      # dense MFMA, published


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--shape", default="qwen3-8b", help="a named shape of nano_vllm_amd.models.shapes (qwen3-0.6b ... qwen3-32b)")
    ap.add_argument("--layers", type=int, default=None, help="layers to build (default: all the shape has)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--page-size", type=int, default=256)
    ap.add_argument("--points", default="1,64", help="further decode batch sizes")
    ap.add_argument("--eager", action="store_true", help="no captured decode graph")
    ap.add_argument("--burst", type=int, default=None,
                    help="decode steps in a row without the host in between (default: the engine's decode_burst; 1: one)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--long-context", type=int, default=32768,
                    help="context of one more decode point at the default batch (0: none)")
    ap.add_argument("--serve-seqs", type=int, default=256,
                    help="requests of the reference's benchmark workload through LLM.generate (0: not run)")
    return ap.parse_args()


def serve_run(args, config_json):
    """The reference's benchmark (bench.py:8-28 there) on this model shape with random weights:
    generated tokens a second of one generate call, and the engine's own split of it."""
    import json as _json
    import os
    import random
    import tempfile
    from nano_vllm_amd import LLM, SamplingParams
    rng = random.Random(0)
    n = args.serve_seqs
    prompts = [[rng.randint(0, 10000) for _ in range(rng.randint(100, 1024))] for _ in range(n)]
    params = [SamplingParams(temperature=0.6, ignore_eos=True, max_tokens=rng.randint(100, 1024)) for _ in range(n)]
    with tempfile.TemporaryDirectory() as folder:
        with open(os.path.join(folder, "config.json"), "w") as f:
            _json.dump(config_json, f)
        llm = LLM(folder, random_weights=args.seed, max_model_len=4096, kvcache_block_size=args.page_size,
                  enforce_eager=args.eager, **({} if args.burst is None else {"decode_burst": max(1, args.burst)}))
        llm.generate([[1, 2, 3, 4]], SamplingParams(temperature=0.6, max_tokens=8, ignore_eos=True), use_tqdm=False)
        for k in llm.stats:
            llm.stats[k] = 0 if isinstance(llm.stats[k], int) else 0.0
        t0 = time.perf_counter()
        llm.generate(prompts, params, use_tqdm=False)
        dt = time.perf_counter() - t0
        st = llm.stats
    total = sum(p.max_tokens for p in params)
    out = {"value": round(total / dt, 1), "unit": "generated tok/s", "seconds": round(dt, 2), "generated_tokens": total,
           "prompt_tokens": sum(len(p) for p in prompts),
           "prefill_tok_s": round(st["prefill_tokens"] / max(st["prefill_time"], 1e-9), 1),
           "decode_tok_s": round(st["decode_tokens"] / max(st["decode_time"], 1e-9), 1), "steps": st["steps"]}
    print(f"# serve {n} requests: {total} tokens in {dt:.2f} s = {total / dt:.0f} tok/s (prefill {out['prefill_tok_s']:.0f}, "
          f"decode {out['decode_tok_s']:.0f} tok/s by the engine's own clock)", file=sys.stderr, flush=True)
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not measured")
        return 2

    import torch
    from nano_vllm_amd.config import EngineConfig, Qwen3Config
    from nano_vllm_amd.engine.batch import StepEntry
    from nano_vllm_amd.engine.runner import ModelRunner
    from nano_vllm_amd.kernels import HipKernels
    from nano_vllm_amd.models.qwen3 import build_spec
    from nano_vllm_amd.parts.model import Model, torch_dtype
    from nano_vllm_amd.sampling.sampler import Sampler
    from nano_vllm_amd.weights import fill_random_

    from nano_vllm_amd.models.shapes import shape
    config_json = shape(args.shape)                     # the default is the benchmark's model: layer sizes of Qwen3-8B
    full_layers = config_json["num_hidden_layers"]
    if args.burst is None:
        args.burst = EngineConfig.decode_burst
    config_json.update(num_hidden_layers=args.layers or full_layers, torch_dtype=args.dtype)
    cfg = Qwen3Config.from_dict(config_json)
    device = "cuda:0"
    dtype = torch_dtype(args.dtype)
    itemsize = 2 if args.dtype == "bfloat16" else 4
    kernels = HipKernels(device, dtype)
    model = Model(build_spec(cfg), kernels, device, dtype)
    fill_random_(model, args.seed)
    torch.cuda.synchronize()

    points = sorted({args.batch} | {int(b) for b in args.points.split(",") if b})
    page = args.page_size
    pages_per_request = (args.context + page - 1) // page + 1
    num_pages = max(points) * pages_per_request + (args.prefill_tokens + page - 1) // page + 1
    runner = ModelRunner(model, page, num_pages, max(points) + 1, enable_prefix_caching=False)
    if not args.eager and hasattr(runner, "enable_decode_graphs"):
        runner.enable_decode_graphs(max(points), args.context + page)
    for lc in runner.layer_caches:                      # random keys and values in every page
        lc.k.normal_(0, 1)
        lc.v.normal_(0, 1)
    sampler = Sampler(kernels, model.device)
    gen = torch.Generator().manual_seed(args.seed)

    # ------------------------------------------------------------------ what a decode step must read
    H, I, V, D = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.head_dim
    Hq, Hkv, L = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.num_hidden_layers
    layer_matrix_params = (Hq + 2 * Hkv) * D * H + H * Hq * D + 2 * I * H + H * I
    layer_params = layer_matrix_params + 2 * H + 2 * D
    weight_bytes = (L * layer_params + H + V * H) * itemsize            # every weight a step uses, once
    kv_bytes_per_token = 2 * L * Hkv * D * itemsize

    def decode_run(batch, steps, warmup, runner=runner, context=args.context):
        """Timed decode steps that end with `context` tokens in each request's cache."""
        start = context - (steps + warmup)
        ids = [f"d{batch}-{i}" for i in range(batch)]
        for rid in ids:
            runner.cache.admit(rid)
            runner.cache.reserve(rid, start)
        tokens = torch.randint(0, V, (batch,), generator=gen).tolist()
        pos = start
        temps, seeds, reqs = [0.0] * batch, [0] * batch, list(range(batch))

        def some_steps(count):
            """`count` decode steps: through the host one by one, or as bursts on the device."""
            nonlocal tokens, pos
            burst = 1 if args.eager else max(1, args.burst)
            while count > 0:
                n = min(burst, count)
                entries = []
                for rid, tok in zip(ids, tokens):
                    runner.cache.reserve(rid, pos + n)
                    entries.append(StepEntry(rid, [tok], pos, [0]))
                if n == 1:
                    logits = runner.step(entries)
                    tokens = sampler.sample(logits, temps, seeds, reqs, [pos + 1] * batch)
                else:
                    tokens = runner.decode_burst(entries, n, sampler, temps, seeds, reqs)[-1]
                pos += n
                count -= n

        some_steps(warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        some_steps(steps)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert pos == context
        for rid in ids:
            runner.cache.release(rid)
        # keys read per step: the mean context over the timed steps
        mean_ctx = context - (steps - 1) / 2.0
        step_bytes = weight_bytes + batch * H * itemsize + batch * mean_ctx * kv_bytes_per_token
        return dt, step_bytes

    def prefill_run(tokens_n, reps, warmup):
        toks = torch.randint(0, V, (tokens_n,), generator=gen).tolist()
        times = []
        for r in range(warmup + reps):
            runner.cache.admit("p")
            runner.cache.reserve("p", tokens_n)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            runner.step([StepEntry("p", toks, 0, [tokens_n - 1])])
            torch.cuda.synchronize()
            if r >= warmup:
                times.append(time.perf_counter() - t0)
            runner.cache.release("p")
        return sum(times) / len(times)

    results = {}
    for b in points:
        steps = args.steps if b == args.batch else max(8, args.steps // 2)
        dt, step_bytes = decode_run(b, steps, args.warmup)
        results[b] = (b * steps / dt, dt / steps, step_bytes)
        print(f"# decode batch {b}: {results[b][0]:.1f} tok/s, {results[b][1] * 1e3:.3f} ms/step", file=sys.stderr,
              flush=True)

    T = args.prefill_tokens
    pre_s = prefill_run(T, reps=3, warmup=2)
    # matrix products of every token, the head for the one wanted row, causal attention
    prefill_flops = 2.0 * T * L * layer_matrix_params + 2.0 * V * H + L * 4.0 * Hq * D * T * (T + 1) / 2.0
    print(f"# prefill {T} tokens: {T / pre_s:.0f} tok/s, {pre_s * 1e3:.2f} ms", file=sys.stderr, flush=True)
    kernels.check_faults()

    extra_points = {}
    if args.long_context > args.context and args.dtype == "bfloat16":
        # the default batch at a long context, on a runner of its own (its captured steps are sized
        # for that length; the headline's runner stays as it was)
        ctx = args.long_context
        del runner
        torch.cuda.empty_cache()
        long_runner = ModelRunner(model, page, args.batch * ((ctx + page - 1) // page + 1), args.batch + 1,
                                  enable_prefix_caching=False)
        if not args.eager:
            long_runner.enable_decode_graphs(args.batch, ctx + page)
        for lc in long_runner.layer_caches:
            lc.k.normal_(0, 1)
            lc.v.normal_(0, 1)
        steps = max(8, args.steps // 2)
        dt, step_bytes = decode_run(args.batch, steps, args.warmup, runner=long_runner, context=ctx)
        extra_points[f"decode_b{args.batch}_ctx{ctx}"] = round(args.batch * steps / dt, 2)
        print(f"# decode batch {args.batch} at context {ctx}: {args.batch * steps / dt:.1f} tok/s, {dt / steps * 1e3:.3f} "
              f"ms/step, {step_bytes / (dt / steps) / 1e9:.0f} GB/s", file=sys.stderr, flush=True)
        kernels.check_faults()
        del long_runner
        runner = None
    serve = None
    if args.serve_seqs > 0 and args.dtype == "bfloat16":
        serve = serve_run(args, config_json)
        torch.cuda.synchronize()

    value, step_s, step_bytes = results[args.batch]
    achieved = step_bytes / step_s / 1e9
    shape_name = args.shape.replace("qwen", "Qwen").replace("b", "B") if args.shape.startswith("qwen3-") else args.shape
    short_dtype = "bf16" if args.dtype == "bfloat16" else "fp32"
    line = {
        "metric": f"decode tok/s @ batch {args.batch}, context {args.context}, {shape_name} shape {short_dtype} "
                  f"(also batch {'/'.join(str(b) for b in points if b != args.batch) or '-'} and prefill tok/s @ {T} tok"
                  + (f"; serve_{args.serve_seqs}: the reference's bench.py workload through LLM.generate" if serve else "") + ")",
        "value": round(value, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short_dtype, "data": "synthetic",
        "config": {"model": f"{shape_name} shape, random weights", "global_batch": args.batch, "seq_len": args.context,
                   "parallelism": "single GPU", "layers": L, "layers_of_shape": full_layers, "hidden_size": H,
                   "num_attention_heads": Hq, "num_key_value_heads": Hkv, "head_dim": D, "intermediate_size": I,
                   "vocab_size": V, "kv_page_size": page, "prefill_tokens": T, "rope_theta": cfg.rope_theta,
                   "rms_norm_eps": cfg.rms_norm_eps, "decode_graph": not args.eager,
                   "decode_burst": 1 if args.eager else max(1, args.burst)},
        "prefill": {"value": round(T / pre_s, 1), "tokens": T, "ms": round(pre_s * 1e3, 3),
                    "frac": round(prefill_flops / pre_s / PEAK_FLOPS[args.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": {**{f"decode_b{b}": round(results[b][0], 2) for b in points if b != args.batch}, **extra_points},
    }
    if serve:
        line[f"serve_{args.serve_seqs}"] = serve
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
