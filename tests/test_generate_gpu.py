"""Generation through the Python entry point and the command line on the GPU."""
import json
import os
import subprocess
import sys

import pytest

import helpers as H
import plain_qwen3 as plain
from nano_vllm_amd import LLM, SamplingParams

pytestmark = pytest.mark.gpu


def _llm(name, dtype, **kw):
    opts = dict(dtype=dtype, kvcache_block_size=H.CONFIGS[name]["page"], num_kvcache_blocks=64,
                max_num_batched_tokens=16, max_num_seqs=4)
    opts.update(kw)
    return LLM(H.model_folder(name, dtype), **opts)


@pytest.mark.parametrize("name", ["a", "b"])
def test_greedy_generation_in_float32_is_the_plain_argmax_chain(name):
    lens = (5, 11, 17) if name == "a" else (3, 9, 24, 40)
    prompts = [H.random_tokens(H.CONFIGS[name]["cfg"].vocab_size, n, 100 + n) for n in lens]
    outs = _llm(name, "float32").generate(prompts, SamplingParams(temperature=0.0, max_tokens=8), use_tqdm=False)
    cfg, w = plain.read_folder(H.model_folder(name, "float32"))
    for p, o in zip(prompts, outs):
        assert o["token_ids"] == plain.greedy_generate(w, cfg, p, 8)


def test_greedy_generation_in_bfloat16_follows_the_plain_chain():
    name = "c"
    prompts = [H.random_tokens(1000, n, 200 + n) for n in (30, 77, 150)]
    outs = _llm(name, "bfloat16").generate(prompts, SamplingParams(temperature=0.0, max_tokens=12), use_tqdm=False)
    cfg, w = plain.read_folder(H.model_folder(name, "bfloat16"))
    same = total = 0
    for p, o in zip(prompts, outs):
        # teacher-forced on the engine's own tokens, so that one flipped near-tie does not
        # turn every later token: the plain logit of the engine's token must be within the
        # tolerance of the plain maximum
        toks = list(p)
        for t in o["token_ids"]:
            l = plain.logits(w, cfg, toks, "bfloat16")[-1]
            assert float(l.max() - l[t]) <= 2e-2 * float(l.abs().max())
            same += int(int(l.argmax()) == t)
            total += 1
            toks.append(t)
    assert same >= 0.8 * total


def test_schedules_and_page_shortage_do_not_change_greedy_tokens():
    name = "b"
    prompts = [H.random_tokens(384, n, 300 + n) for n in (3, 9, 24, 40, 33, 33)]
    prompts[5] = prompts[4][:32] + [1]                      # shares four pages with the one before
    sp = SamplingParams(temperature=0.0, max_tokens=10)
    base = [o["token_ids"] for o in _llm(name, "float32", enable_prefix_caching=False).generate(prompts, sp, use_tqdm=False)]
    for kw in (dict(schedule="mixed"), dict(num_kvcache_blocks=14), dict(num_kvcache_blocks=14, schedule="mixed")):
        llm = _llm(name, "float32", **kw)
        assert [o["token_ids"] for o in llm.generate(prompts, sp, use_tqdm=False)] == base, kw
        llm.runner.cache.check()
        if "num_kvcache_blocks" in kw:
            assert llm.scheduler.num_preemptions > 0


@pytest.mark.parametrize("seed", range(4))
def test_scheduling_options_drawn_at_random_do_not_change_the_tokens(tmp_path, seed):
    """A configuration, requests (some sharing a prefix) and sampling drawn at random; then schedule,
    pool size (down to what the longest request needs and one page), token budget, request limit, burst
    length and prefix reuse drawn at random: the tokens of a run with plenty of everything, in
    float32, where the logits do not depend on the batch by a bit."""
    import random
    from nano_vllm_amd.models.qwen3 import Qwen3Config
    from nano_vllm_amd.weights import write_random_model
    rng = random.Random(7000 + seed)
    hkv, group = rng.choice([1, 2, 4]), rng.choice([1, 2, 4, 8])
    cfg = Qwen3Config(vocab_size=rng.randint(50, 1500), hidden_size=8 * rng.randint(4, 30), num_hidden_layers=rng.randint(1, 3),
                      num_attention_heads=hkv * group, num_key_value_heads=hkv, head_dim=rng.choice([16, 32, 64, 128]),
                      intermediate_size=8 * rng.randint(4, 40), rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=512,
                      tie_word_embeddings=rng.random() < 0.5)
    page = rng.choice([4, 8, 16, 32, 64])
    folder = str(tmp_path / "model")
    write_random_model(folder, cfg, seed=seed, norm_std=0.1, dtype="float32")
    count = rng.randint(2, 7)
    prompts = [H.random_tokens(cfg.vocab_size, rng.randint(1, 150), 50 * seed + i) for i in range(count)]
    if count > 2:
        prompts[1] = prompts[0][:len(prompts[0]) // 2] + prompts[1][:5]
    params = [SamplingParams(temperature=rng.choice([0.0, 0.0, 0.8]), max_tokens=rng.randint(1, 40), seed=rng.randint(0, 5))
              for _ in prompts]
    pages = [(len(p) + sp.max_tokens + page - 1) // page for p, sp in zip(prompts, params)]
    plenty = dict(dtype="float32", kvcache_block_size=page, num_kvcache_blocks=sum(pages) + 4, max_num_batched_tokens=4096,
                  max_num_seqs=8, decode_burst=1, enable_prefix_caching=False, max_model_len=512)
    base = [o["token_ids"] for o in LLM(folder, **plenty).generate(prompts, params, use_tqdm=False)]
    for _ in range(2):
        kw = dict(plenty, schedule=rng.choice(["prefill_first", "mixed"]),
                  num_kvcache_blocks=rng.choice([sum(pages) + 4, max(pages) + 1, max(pages) + rng.randint(1, 6)]),
                  max_num_batched_tokens=rng.choice([4096, 16, rng.randint(2, 64)]), max_num_seqs=rng.choice([8, 1, 2, 3]),
                  decode_burst=rng.choice([1, 2, 4, 8, 16]), enable_prefix_caching=rng.random() < 0.5)
        llm = LLM(folder, **kw)
        assert [o["token_ids"] for o in llm.generate(prompts, params, use_tqdm=False)] == base, kw
        llm.runner.cache.check()


def test_temperature_sampling_is_reproducible_and_independent_of_the_batch():
    name = "b"
    prompts = [H.random_tokens(384, n, 400 + n) for n in (7, 19, 31)]
    sp = SamplingParams(temperature=0.7, max_tokens=10, seed=3)
    a = [o["token_ids"] for o in _llm(name, "float32").generate(prompts, sp, use_tqdm=False)]
    b = [o["token_ids"] for o in _llm(name, "float32", max_num_seqs=1).generate(prompts, sp, use_tqdm=False)]
    assert a == b
    c = [o["token_ids"] for o in _llm(name, "float32").generate(prompts, SamplingParams(temperature=0.7, max_tokens=10, seed=4), use_tqdm=False)]
    assert a != c


def test_cache_sized_from_free_memory():
    llm = LLM(H.model_folder("d", "bfloat16"), gpu_memory_utilization=0.05, max_num_batched_tokens=64, max_num_seqs=4)
    assert llm.config.num_kvcache_blocks > 0 and llm.config.kvcache_block_size == 256
    assert llm.warmup_peak_bytes > 0              # the largest step was run and measured
    out = llm.generate([[1, 2, 3]], SamplingParams(temperature=0.0, max_tokens=3), use_tqdm=False)
    assert len(out[0]["token_ids"]) == 3


def test_command_line_generates(tmp_path):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "example.py"), "--model", H.model_folder("b", "float32"),
                           "--prompt-ids", "5,6,7", "--prompt-ids", "9,8", "--temperature", "0", "--max-tokens", "4",
                           "--kvcache-block-size", "8", "--num-kvcache-blocks", "16", "--json"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    outs = json.loads(proc.stdout.strip().split("\n")[-1])
    cfg, w = plain.read_folder(H.model_folder("b", "float32"))
    assert [o["token_ids"] for o in outs] == [plain.greedy_generate(w, cfg, p, 4) for p in ([5, 6, 7], [9, 8])]


def test_throughput_command_with_weights_drawn_on_the_device(tmp_path, capsys):
    """The reference's bench.py workload in small: requests of random ids through generate, with
    the weights drawn from a seed (the folder holds config.json only), padded decode graphs and
    so few pages that requests wait and are preempted."""
    from nano_vllm_amd.cli import main
    folder = tmp_path / "config_only"
    folder.mkdir()
    cj = H.CONFIGS["c"]["cfg"].to_dict()
    (folder / "config.json").write_text(json.dumps(cj))
    rc = main(["throughput", "--model", str(folder), "--random-weights", "4", "--num-seqs", "11", "--min-input-len", "5",
               "--max-input-len", "60", "--min-output-len", "4", "--max-output-len", "40", "--max-token-id", "500",
               "--kvcache-block-size", "16", "--num-kvcache-blocks", "24", "--max-num-seqs", "6",
               "--max-num-batched-tokens", "64", "--max-model-len", "128", "--json"])
    assert rc == 0
    lines = capsys.readouterr().out.strip().split("\n")
    assert lines[-2].startswith("Total: ") and "Throughput: " in lines[-2]
    stats = json.loads(lines[-1])
    assert stats["num_seqs"] == 11 and stats["decode_tokens"] > 0 and stats["prefill_tokens"] >= stats["prompt_tokens"]


def test_decode_bursts_do_not_change_the_tokens():
    """Generation with several decode steps in a row on the device (the default) against one step
    at a time: greedy and at a temperature, requests that end inside a burst by max_tokens and by
    an eos token, and a pool so small that bursts fall back to single steps."""
    name, dtype = "c", "bfloat16"
    prompts = [H.random_tokens(1000, n, 300 + n) for n in (12, 33, 57, 8)]
    params = [SamplingParams(temperature=t, max_tokens=m) for t, m in ((0.0, 23), (0.7, 9), (1.1, 30), (0.0, 14))]
    base = _llm(name, dtype, decode_burst=1, max_num_batched_tokens=256).generate(prompts, params, use_tqdm=False)
    eos = base[2]["token_ids"][11]                                  # request 2 ends here when this token ends requests
    for kw in (dict(), dict(eos=eos), dict(num_kvcache_blocks=9)):
        one = base if not kw else _llm(name, dtype, decode_burst=1, max_num_batched_tokens=256, **kw).generate(
            prompts, params, use_tqdm=False)
        llm = _llm(name, dtype, decode_burst=6, max_num_batched_tokens=256, **kw)
        many = llm.generate(prompts, params, use_tqdm=False)
        assert [o["token_ids"] for o in many] == [o["token_ids"] for o in one], kw
        if "num_kvcache_blocks" not in kw:                          # (a preempted request gets a token from a prompt step)
            assert llm.stats["decode_tokens"] == sum(len(o["token_ids"]) for o in many) - len(prompts)
        else:
            assert llm.scheduler.num_preemptions > 0
    assert len(_llm(name, dtype, decode_burst=6, eos=eos).generate(prompts, params, use_tqdm=False)[2]["token_ids"]) <= 12
