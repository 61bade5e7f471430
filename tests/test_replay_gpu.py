"""The engine on the GPU against the plain implementation, in float32 and bfloat16: each
request alone and whole; most of it in one step and the last 32 tokens one by one; in
portions of changing size, down to two tokens; mixed, up to four live requests on so few
pages that they are used again; long decoding; the first tokens; and the same through
bin/trace_run as a user calls it."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

# float32: summation order only.  bfloat16: both sides round at the same places (the plain
# implementation emulates them), but sum in different orders, so single roundings of about
# 2^-9 flip and travel through the layers; 2e-2 of the largest logit bounds what a few such
# flips per layer give and is far below the effect of any indexing fault.
TOL = {"float32": 2e-5, "bfloat16": 2e-2}
ROUNDING = {"float32": None, "bfloat16": "bfloat16"}


@pytest.fixture(scope="module")
def runners():
    made = {}

    def get(name, dtype, pages):
        key = (name, dtype, pages)
        if key not in made:
            made[key] = H.make_runner(H.model_folder(name, dtype), dtype, H.CONFIGS[name]["page"], pages)
        return made[key]
    return get


def _length(name):
    return min(H.CONFIGS[name]["cfg"].max_position_embeddings - 2, 250)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b", "c", "d", "e"])
@pytest.mark.parametrize("driving", ["whole", "last32", "portions"])
def test_one_request(runners, name, dtype, driving):
    n = _length(name)
    toks = H.random_tokens(H.CONFIGS[name]["cfg"].vocab_size, n, 21)
    want = H.plain_logits(H.model_folder(name, dtype), toks, ROUNDING[dtype])
    portions = {"whole": H.whole(n), "last32": H.last_one_by_one(n), "portions": H.changing_portions(n, 5)}[driving]
    r = runners(name, dtype, 80)
    got = H.run_portions(r, "x", toks, portions)
    assert H.rel_err(got, want) < TOL[dtype]
    if dtype == "float32":
        assert torch.equal(got.argmax(-1), want.argmax(-1))
    r.kernels.check_faults()


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Every size and option of the configuration drawn at random (head sizes in steps of 16, odd
    numbers of heads and groups, widths and vocabularies that are no power of two, with and without
    the bias on q/k/v and the tied head), a page size, a dtype and a length: whole, the last tokens
    one by one, and in portions, against the plain implementation."""
    import random
    from nano_vllm_amd.models.qwen3 import Qwen3Config
    from nano_vllm_amd.weights import write_random_model
    rng = random.Random(9000 + seed)
    hkv, group = rng.choice([1, 2, 3, 4]), rng.choice([1, 2, 3, 4, 8])
    cfg = Qwen3Config(vocab_size=rng.randint(50, 1500), hidden_size=8 * rng.randint(4, 40), num_hidden_layers=rng.randint(1, 3),
                      num_attention_heads=hkv * group, num_key_value_heads=hkv,
                      head_dim=rng.choice([16, 32, 48, 64, 80, 96, 128]), intermediate_size=8 * rng.randint(4, 60),
                      rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-4]), rope_theta=rng.choice([1e4, 5e5, 1e6]),
                      max_position_embeddings=512, tie_word_embeddings=rng.random() < 0.5,
                      attention_bias=rng.random() < 0.25)
    page = rng.choice([4, 8, 16, 24, 32, 64, 256])
    dtype = rng.choice(["float32", "bfloat16"])
    n = rng.randint(3, 300)
    folder = str(tmp_path / "model")
    write_random_model(folder, cfg, seed=seed, norm_std=0.1, dtype=dtype)
    toks = H.random_tokens(cfg.vocab_size, n, 40 + seed)
    want = H.plain_logits(folder, toks, ROUNDING[dtype])
    r = H.make_runner(folder, dtype, page, (512 + page - 1) // page + 4)
    for portions in (H.whole(n), H.last_one_by_one(n, rng.randint(1, 40)), H.changing_portions(n, seed)):
        got = H.run_portions(r, "x", toks, portions)
        r.kernels.check_faults()
        assert H.rel_err(got, want) < TOL[dtype], (cfg, page, dtype, n, portions[:4])


@pytest.mark.parametrize("name", ["b", "d"])
def test_decoding_with_the_kernel_for_wide_weights_forced(name):
    """At the tiny sizes no weight is wide enough for the kernel whose waves split k inside a
    workgroup, so the decoded tokens of these models never run it; here it takes every product
    of up to 16 rows (qkv, o, gate/up with the gating, down, the head; widths are multiples of 32
    in these two configurations)."""
    dtype = "bfloat16"
    n = _length(name)
    toks = H.random_tokens(H.CONFIGS[name]["cfg"].vocab_size, n, 23)
    want = H.plain_logits(H.model_folder(name, dtype), toks, ROUNDING[dtype])
    r = H.make_runner(H.model_folder(name, dtype), dtype, H.CONFIGS[name]["page"], 80)
    r.kernels.team_min_weight_rows = 0
    seen = []
    launch = r.kernels._linear_team
    r.kernels._linear_team = lambda *a: (seen.append(a[7]), launch(*a))[1]
    got = H.run_portions(r, "x", toks, [n - 40, 9, 5] + [1] * 26)
    assert H.rel_err(got, want) < TOL[dtype]
    assert {0, 1, 2} <= set(seen)                   # element, float and gated results all went through it
    r.kernels.check_faults()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b", "c", "d", "e"])
def test_mixed_requests_on_few_pages(runners, name, dtype):
    c = H.CONFIGS[name]
    top = _length(name)
    lens = [top, top // 2 + 3, top - 17, 40, top // 3, top - 40, 65]
    reqs = {f"r{i}": H.random_tokens(c["cfg"].vocab_size, n, 30 + i) for i, n in enumerate(lens)}
    need = sorted(((n + c["page"] - 1) // c["page"] for n in lens), reverse=True)
    pages = sum(need[:3]) + 1                      # room for about three of the seven at a time
    r = runners(name, dtype, pages)
    got = H.run_mixed(r, reqs, seed=4)
    for rid, toks in reqs.items():
        want = H.plain_logits(H.model_folder(name, dtype), toks, ROUNDING[dtype])
        assert H.rel_err(got[rid], want) < TOL[dtype], rid
    assert r.cache.pools[0].num_free == pages
    r.kernels.check_faults()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b"])
def test_mixed_requests_that_share_prefix_pages(name, dtype):
    """nanovllm/engine/block_manager.py:58-92,110-120 on the GPU, compared by logits: pages
    found by their hash while another request holds them, pages found after they were given
    back, pages that were taken again in between (the prefix is then computed again), on a
    pool that holds about three requests.  Every computed position against the plain model."""
    c = H.CONFIGS[name]
    folder = H.model_folder(name, dtype)
    r = H.make_runner(folder, dtype, c["page"], H.prefix_pool_pages(name, _length(name)), prefix_caching=True)
    H.check_prefix_reuse(r, name, _length(name), lambda toks: H.plain_logits(folder, toks, ROUNDING[dtype]), TOL[dtype])
    r.kernels.check_faults()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(runners, dtype):
    name = "c"
    n = 600
    toks = H.random_tokens(H.CONFIGS[name]["cfg"].vocab_size, n, 41)
    want = H.plain_logits(H.model_folder(name, dtype), toks, ROUNDING[dtype])
    r = runners(name, dtype, 80)
    got = H.run_portions(r, "x", toks, [1] * n)     # every token decoded, from the very first
    assert H.rel_err(got[:8], want[:8]) < TOL[dtype]
    assert H.rel_err(got, want) < TOL[dtype]


def test_logits_do_not_depend_on_pages_or_batch_mates(runners):
    """float32: the same request alone, beside others, and on other pages gives the same
    logits to the last bit (every sum runs in an order that the batch does not change)."""
    name = "b"
    c = H.CONFIGS[name]
    toks = H.random_tokens(c["cfg"].vocab_size, 90, 51)
    r = runners(name, "float32", 80)
    alone = H.run_portions(r, "x", toks, H.changing_portions(90, 1))
    others = {f"o{i}": H.random_tokens(c["cfg"].vocab_size, 50 + 9 * i, 60 + i) for i in range(3)}
    mixed = H.run_mixed(r, {"o0": others["o0"], "x": toks, "o1": others["o1"], "o2": others["o2"]}, seed=8)
    assert torch.equal(mixed["x"], alone)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_as_a_user_calls_it(tmp_path, dtype):
    """bin/trace_run in a process of its own: portions, single tokens, four live requests,
    a pool so small that pages are used again."""
    name = "b"
    c = H.CONFIGS[name]
    folder = H.model_folder(name, dtype)
    lens = {"a": 100, "b": 70, "c": 130, "d": 64, "e": 90}
    reqs = {k: H.random_tokens(c["cfg"].vocab_size, n, 70 + i) for i, (k, n) in enumerate(lens.items())}
    # steps: a and b start; c joins; a ends, d takes its pages; ...
    plan = [
        [("a", 60), ("b", 2)], [("a", 38), ("b", 33), ("c", 64)], [("a", 1), ("b", 1), ("c", 2)],
        [("a", 1), ("b", 34), ("c", 64)], "end:a", [("d", 63), ("b", 0), ("c", 0)], [("d", 1), ("e", 7)],
        "end:b", [("e", 83)], "end:c,d,e",
    ]
    pos = {k: 0 for k in reqs}
    lines, wants, step = [], {}, 0
    pending_end = []
    for item in plan:
        if isinstance(item, str):
            lines[-1]["end"] = item[4:].split(",")
            continue
        entries = []
        for rid, n in item:
            if n == 0:
                continue
            want = list(range(n)) if n <= 4 else [0, n // 2, n - 1]
            entries.append({"id": rid, "tokens": reqs[rid][pos[rid]:pos[rid] + n], "want": want})
            for w in want:
                wants.setdefault(step, []).append((rid, pos[rid] + w))
            pos[rid] += n
        lines.append({"step": step, "entries": entries, "end": []})
        step += 1
    out = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    # live at most: a 100->128, b 70->128, c 130->192 = 448; later d 64 + c 192 + e 128
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", str(out), "--max-tokens", "448"],
                          input="\n".join(json.dumps(l) for l in lines) + "\n", capture_output=True, text=True,
                          timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l] == [f"done {i}" for i in range(step)]
    plain_logits = {k: H.plain_logits(folder, v, ROUNDING[dtype]) for k, v in reqs.items()}
    V = c["cfg"].vocab_size
    for s, places in wants.items():
        got = torch.from_numpy(np.fromfile(out / f"{s}.f32", dtype="<f4").reshape(len(places), V))
        want = torch.stack([plain_logits[rid][p] for rid, p in places])
        assert H.rel_err(got, want) < TOL[dtype], (s, places)


def test_a_bfloat16_model_with_norm_weights_stored_in_float32(tmp_path):
    """A tensor stored in 32 bits stays so: norm weights that a checkpoint stores in float32 are
    used unrounded by the bfloat16 kernels (block norms, final norm, per-head q/k norms), whole and
    in portions with decoded tokens.  The weights are made so that rounding them would show: 1 + d
    with |d| below half a bfloat16 step, which rounds to exactly 1."""
    from safetensors.torch import load_file, save_file
    from nano_vllm_amd.weights import write_random_model
    c = H.CONFIGS["b"]
    folder = write_random_model(str(tmp_path / "m"), c["cfg"], seed=31, norm_std=0.0, dtype="bfloat16")
    file = os.path.join(folder, "model.safetensors")
    tensors = load_file(file)
    gen = torch.Generator().manual_seed(5)
    norms = [k for k in tensors if "norm" in k]
    assert len(norms) == 4 * 3 + 1
    for k in norms:
        d = (torch.rand(tensors[k].shape, generator=gen) - 0.5) * 2 ** -8        # |d| < 2^-9: rounds away in bfloat16
        tensors[k] = (1.0 + d).float()
        assert torch.equal(tensors[k].to(torch.bfloat16).float(), torch.ones_like(d))
    save_file(tensors, file, metadata={"format": "pt"})
    r = H.make_runner(folder, "bfloat16", c["page"], 64)
    assert all(r.model.params[k].dtype == torch.float32 for k in norms)
    assert r.model.params["model.layers.0.mlp.down_proj.weight"].dtype == torch.bfloat16
    toks = H.random_tokens(c["cfg"].vocab_size, 120, 8)
    want = H.plain_logits(folder, toks, "bfloat16")
    for portions in (H.whole(120), H.last_one_by_one(120), H.changing_portions(120, 2)):
        assert H.rel_err(H.run_portions(r, "x", toks, portions), want) < TOL["bfloat16"]
    r.kernels.check_faults()
