"""The engine's host logic (batching, block tables, slot mapping, scheduler, engine loop)
on the CPU: the device operations are replaced by their plain torch versions
(tests/torch_kernels.py), the model and everything above it is the product's.  Compared
with the plain implementation in float32."""
import json

import pytest
import torch

import helpers as H
import plain_qwen3 as plain
from nano_vllm_amd import LLM, SamplingParams
from nano_vllm_amd.cache import OutOfPages
from nano_vllm_amd.engine.batch import StepEntry
from torch_kernels import TorchKernels

TOL = 2e-5


def _runner(name, pages):
    c = H.CONFIGS[name]
    return H.make_runner(H.model_folder(name), "float32", c["page"], pages, device="cpu", kernels=TorchKernels())


@pytest.mark.parametrize("name", ["a", "b", "e"])
def test_every_cutting_gives_the_plain_logits(name):
    c = H.CONFIGS[name]
    n = 70
    toks = H.random_tokens(c["cfg"].vocab_size, n, 1)
    want = H.plain_logits(H.model_folder(name), toks)
    r = _runner(name, 32)
    for portions in (H.whole(n), H.last_one_by_one(n), H.changing_portions(n, 2)):
        got = H.run_portions(r, "x", toks, portions)
        assert H.rel_err(got, want) < TOL, portions


def test_mixed_batches_on_few_pages():
    c = H.CONFIGS["b"]
    lens = {"r0": 60, "r1": 41, "r2": 77, "r3": 35, "r4": 52, "r5": 66}
    reqs = {r: H.random_tokens(c["cfg"].vocab_size, n, i) for i, (r, n) in enumerate(lens.items())}
    r = _runner("b", 26)                  # 208 tokens of cache for 331 tokens of requests: pages are used again
    got = H.run_mixed(r, reqs, seed=3)
    for rid, toks in reqs.items():
        assert H.rel_err(got[rid], H.plain_logits(H.model_folder("b"), toks)) < TOL, rid
    assert r.cache.pools[0].num_free == 26


def test_step_refuses_what_the_cache_does_not_hold():
    r = _runner("a", 4)
    r.cache.admit("x")
    r.cache.reserve("x", 3)
    with pytest.raises(ValueError, match="not reserved"):
        r.step([StepEntry("x", [1, 2, 3, 4], 0, [])])
    with pytest.raises(ValueError, match="vocabulary"):
        r.step([StepEntry("x", [1, 2, 999], 0, [])])
    with pytest.raises(ValueError, match="twice"):
        r.step([StepEntry("x", [1], 0, []), StepEntry("x", [2], 1, [])])
    with pytest.raises(ValueError, match="wanted place"):
        r.step([StepEntry("x", [1, 2], 0, [2])])
    assert r.step([StepEntry("x", [1, 2], 0, [])]) is None
    with pytest.raises(OutOfPages):
        r.cache.reserve("x", 17)


def test_logits_come_back_in_the_callers_order():
    c = H.CONFIGS["a"]
    r = _runner("a", 16)
    t1, t2 = H.random_tokens(256, 9, 1), H.random_tokens(256, 6, 2)
    w1, w2 = H.plain_logits(H.model_folder("a"), t1), H.plain_logits(H.model_folder("a"), t2)
    for rid, n in (("p", 9), ("q", 6)):
        r.cache.admit(rid)
        r.cache.reserve(rid, n)
    r.step([StepEntry("q", t2[:5], 0, [])])
    # a portion first, a single token second: the step reorders, the answer does not
    out = r.step([StepEntry("p", t1, 0, [8, 0, 3]), StepEntry("q", t2[5:], 5, [0])])
    want = torch.stack([w1[8], w1[0], w1[3], w2[5]])
    assert H.rel_err(out, want) < TOL


def test_a_padded_batch_of_decoded_tokens_reads_what_the_first_request_reads():
    """The captured decode graphs run a few fixed batch sizes: the rows beyond the real requests
    are copies of the first entry that write nothing, and the real rows are not changed by them."""
    from nano_vllm_amd.engine.batch import build_batch
    r = _runner("a", 16)
    toks = {rid: H.random_tokens(256, 9, s) for s, rid in enumerate("pqr")}
    for rid, t in toks.items():
        r.cache.admit(rid)
        r.cache.reserve(rid, 9)
        r.step([StepEntry(rid, t[:8], 0, [])])
    entries = [StepEntry(rid, t[8:], 8, [0]) for rid, t in toks.items()]
    b = build_batch(entries, r.cache, r.page_size, 256, "cpu", table_width=5, pad_to=4)
    assert (b.num_seqs, b.num_tokens, b.num_decode) == (4, 4, 4)
    assert b.input_ids.tolist() == [toks["p"][8], toks["q"][8], toks["r"][8], toks["p"][8]]
    assert b.positions.tolist() == [8, 8, 8, 8] and b.logits_rows.tolist() == [0, 1, 2, 3]
    assert b.groups[0].slot_mapping.tolist()[3] == -1 and b.groups[0].slot_mapping.tolist()[0] >= 0
    assert b.groups[0].block_tables[3].tolist() == b.groups[0].block_tables[0].tolist()
    assert b.groups[0].block_tables.shape == (4, 5)
    padded = r.model.logits(r.model.forward(b, r.layer_caches), b.logits_rows)
    plain_rows = r.step(entries)
    assert torch.equal(padded[:3], plain_rows) and torch.equal(padded[3], padded[0])
    with pytest.raises(ValueError, match="decoded"):
        build_batch([StepEntry("p", toks["p"][7:], 7, [])], r.cache, r.page_size, 256, "cpu", pad_to=2)


def test_the_batch_builder_uploads_what_the_kernels_ask_for_and_knows_no_kernel():
    """Lists that a kernel wants on the device for a step (the prefill attention's tile order is
    one) are asked of the kernels object and travel in the batch's one copy; the builder itself
    imports nothing of the kernels."""
    import ast
    import nano_vllm_amd.engine.batch as batch_module
    from nano_vllm_amd.engine.batch import build_batch
    tree = ast.parse(open(batch_module.__file__).read())
    imported = [n.module or "" for n in ast.walk(tree) if isinstance(n, ast.ImportFrom)]
    assert not any("kernels" in m for m in imported), imported
    r = _runner("a", 16)
    for rid, n in (("p", 9), ("q", 6)):
        r.cache.admit(rid)
        r.cache.reserve(rid, n)
    asked = []

    def extras(q_lens, starts, num_decode):
        asked.append((list(q_lens), list(starts), num_decode))
        return {"first": [7, 8, 9], "none": [], "second": [len(q_lens)]}

    entries = [StepEntry("p", list(range(9)), 0, [8]), StepEntry("q", [3], 0, [0])]
    b = build_batch(entries, r.cache, r.page_size, 256, "cpu", extras=extras)
    assert asked == [([1, 9], [0, 0], 1)]                  # single tokens first
    assert b.extras["first"].tolist() == [7, 8, 9] and b.extras["second"].tolist() == [2]
    assert b.extras["none"].numel() == 0 and b.extras["first"].dtype == torch.int32
    assert b.logits_rows.tolist() == [9, 0] and b.groups[0].slot_mapping.numel() == 10
    assert build_batch(entries, r.cache, r.page_size, 256, "cpu").extras == {}


def _llm(name, **kw):
    c = H.CONFIGS[name]
    opts = dict(kernels=TorchKernels(), device="cpu", dtype="float32", kvcache_block_size=c["page"],
                num_kvcache_blocks=64, max_num_batched_tokens=16, max_num_seqs=4)
    opts.update(kw)
    return LLM(H.model_folder(name), **opts)


def _prompts(name, lens):
    return [H.random_tokens(H.CONFIGS[name]["cfg"].vocab_size, n, 100 + n) for n in lens]


def test_greedy_generation_is_the_plain_argmax_chain():
    prompts = _prompts("b", (3, 9, 24, 40))
    outs = _llm("b").generate(prompts, SamplingParams(temperature=0.0, max_tokens=8), use_tqdm=False)
    cfg, w = plain.read_folder(H.model_folder("b"))
    for p, o in zip(prompts, outs):
        assert o["token_ids"] == plain.greedy_generate(w, cfg, p, 8)
        assert o["finish_reason"] == "max_tokens" and o["text"] is None


def test_schedules_prefix_cache_and_page_shortage_do_not_change_the_tokens():
    prompts = _prompts("b", (3, 9, 24, 40))
    shared = prompts[3][:32]
    prompts += [shared + [5, 6, 7], shared + [9]]            # two requests with four pages in common
    sp = [SamplingParams(temperature=0.0, max_tokens=10), SamplingParams(temperature=0.7, max_tokens=10)] * 3
    base = _llm("b", enable_prefix_caching=False).generate(prompts, sp, use_tqdm=False)
    for kw in (dict(schedule="mixed"), dict(enable_prefix_caching=True), dict(num_kvcache_blocks=14),
               dict(num_kvcache_blocks=14, schedule="mixed"), dict(max_num_batched_tokens=5, max_num_seqs=2)):
        llm = _llm("b", **kw)
        outs = llm.generate(prompts, sp, use_tqdm=False)
        assert [o["token_ids"] for o in outs] == [o["token_ids"] for o in base], kw
        llm.runner.cache.check()
        assert llm.runner.cache.pools[0].num_free == llm.config.num_kvcache_blocks
        if kw.get("num_kvcache_blocks") == 14:
            assert llm.scheduler.num_preemptions > 0


def test_the_engines_counts_tell_prompt_tokens_from_decoded_ones_in_either_schedule():
    prompts = _prompts("a", (3, 9, 24, 40))
    for kw in (dict(), dict(schedule="mixed"), dict(schedule="mixed", decode_burst=1)):
        llm = _llm("a", enable_prefix_caching=False, **kw)
        llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=7, ignore_eos=True), use_tqdm=False)
        # a request's first token comes out of the step that holds the end of its prompt
        assert llm.stats["prefill_tokens"] == sum(len(p) for p in prompts), kw
        assert llm.stats["decode_tokens"] == len(prompts) * 6, kw


def test_temperature_sampling_is_the_plain_draw_and_is_reproducible():
    prompts = _prompts("a", (5, 11))
    sp = SamplingParams(temperature=0.7, max_tokens=5, seed=42)
    llm = _llm("a")
    outs = llm.generate(prompts, sp, use_tqdm=False)
    cfg, w = plain.read_folder(H.model_folder("a"))
    # by hand: the same seed, request number and position give the same noise
    for k, (p, o) in enumerate(zip(prompts, outs)):
        toks = list(p)
        for _ in range(5):
            l = plain.logits(w, cfg, toks)[-1]
            toks.append(plain.sample(l, 0.7, seed=42, request=k, position=len(toks)))
        assert o["token_ids"] == toks[len(p):]
    assert [o["token_ids"] for o in _llm("a").generate(prompts, sp, use_tqdm=False)] == [o["token_ids"] for o in outs]


def test_unknown_option_is_an_error():
    with pytest.raises(TypeError, match="unknown engine options"):
        _llm("a", max_batch=3)


def test_step_refuses_a_position_the_model_does_not_know():
    """The rotary table has max_position_embeddings rows and the kernels read it unchecked:
    the step function refuses an entry that reaches beyond, whoever calls it."""
    r = _runner("a", 80)                                   # configuration a knows 128 positions
    r.cache.admit("x")
    r.cache.reserve("x", 130)
    toks = H.random_tokens(256, 130, 3)
    r.step([StepEntry("x", toks[:128], 0, [127])])         # positions 0..127 are all there
    with pytest.raises(ValueError, match="beyond the model's 128 positions"):
        r.step([StepEntry("x", toks[128:129], 128, [0])])
    r.cache.admit("y")
    r.cache.reserve("y", 130)
    with pytest.raises(ValueError, match="beyond the model's 128 positions"):
        r.step([StepEntry("y", toks, 0, [])])
    with pytest.raises(ValueError, match="positions"):
        r.enable_decode_graphs(2, 129)


def test_trace_run_refuses_a_trace_longer_than_the_model_knows(tmp_path):
    """bin/trace_run drives the step function without the scheduler's length limit: a trace
    that runs past max_position_embeddings ends with an error, not with a read past the table."""
    import importlib.machinery
    import importlib.util
    import io
    import json
    import os
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "trace_run")
    loader = importlib.machinery.SourceFileLoader("trace_run_program", path)
    trace_run = importlib.util.module_from_spec(importlib.util.spec_from_loader("trace_run_program", loader))
    loader.exec_module(trace_run)
    toks = H.random_tokens(256, 130, 4)
    lines = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:126], "want": [125]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[126:128], "want": [1]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": toks[128:130], "want": [0]}], "end": ["a"]}]
    argv = ["--model", H.model_folder("a"), "--dtype", "float32", "--out", str(tmp_path), "--max-tokens", "256",
            "--device", "cpu"]
    with pytest.raises(ValueError, match="beyond the model's 128 positions"):
        trace_run.main(argv, io.StringIO("\n".join(json.dumps(l) for l in lines) + "\n"), TorchKernels())
    assert sorted(os.listdir(tmp_path)) == ["0.f32", "1.f32"]          # the steps before it ran
    want = H.plain_logits(H.model_folder("a"), toks[:128])
    import numpy as np
    got = torch.from_numpy(np.fromfile(os.path.join(tmp_path, "1.f32"), dtype="<f4").reshape(1, 256))
    assert H.rel_err(got, want[127:128]) < TOL


def test_a_burst_reserves_for_all_its_requests_or_for_none():
    """Several decode steps in a row need pages for all of them: when the pool cannot give them
    to every request of the batch, no request keeps any (single steps follow), and a model
    with more cache groups than the metadata kernel takes never bursts."""
    llm = _llm("a", num_kvcache_blocks=6, decode_burst=4, max_num_batched_tokens=32)           # pages of 4 tokens
    sp = SamplingParams(temperature=0.0, max_tokens=20)
    for p in _prompts("a", (7, 11)):
        llm.add_request(p, sp)
    llm.step()                                                         # both prompts: 2 and 3 pages, 1 free
    llm.model.kernels.max_burst_groups = 4
    llm.runner._graph_max_batch = 8                                    # as if decode steps were captured
    llm.runner._graph_takes = lambda entries: True
    seqs, is_prefill = llm.scheduler.schedule()                        # decode at positions 7 and 11: no new page
    assert not is_prefill and len(seqs) == 2
    entries = [StepEntry(s.seq_id, s.token_ids[-1:], s.num_cached_tokens, [0]) for s in seqs]
    tables = [list(llm.runner.cache.table(s.seq_id, 0)) for s in seqs]
    free = llm.runner.cache.pools[0].num_free
    assert free == 1
    # steps 2..4 need a third page for the first request (positions 8..10), which is there, and a
    # fourth for the second (12..14), which is not: the first must not keep the one it could have
    assert llm._burst_steps(seqs, entries, False) == 1
    assert llm.runner.cache.pools[0].num_free == free
    assert [list(llm.runner.cache.table(s.seq_id, 0)) for s in seqs] == tables
    llm.runner.cache.check()
    # with pages enough the same call reserves for all steps
    big = _llm("a", num_kvcache_blocks=16, decode_burst=4)
    for p in _prompts("a", (7, 8)):
        big.add_request(p, sp)
    big.step()
    big.model.kernels.max_burst_groups = 4
    big.runner._graph_max_batch = 8
    big.runner._graph_takes = lambda entries: True
    seqs, _ = big.scheduler.schedule()
    entries = [StepEntry(s.seq_id, s.token_ids[-1:], s.num_cached_tokens, [0]) for s in seqs]
    assert big._burst_steps(seqs, entries, False) == 4
    assert all(big.runner.cache.requests[s.seq_id].num_tokens == s.num_tokens + 3 for s in seqs)
    big.model.kernels.max_burst_groups = 0
    assert big._burst_steps(seqs, entries, False) == 1


@pytest.mark.parametrize("name", ["a", "b"])
def test_requests_that_share_prefix_pages_give_the_plain_logits(name):
    """The drive of tests/test_replay_gpu.py's prefix test on the host side alone: hashed pages are
    found while in use, found after they were given back, and lost to other requests."""
    c = H.CONFIGS[name]
    top = min(c["cfg"].max_position_embeddings - 2, 250)
    folder = H.model_folder(name)
    r = H.make_runner(folder, "float32", c["page"], H.prefix_pool_pages(name, top), device="cpu",
                      kernels=TorchKernels(), prefix_caching=True)
    H.check_prefix_reuse(r, name, top, lambda toks: H.plain_logits(folder, toks), TOL)


def test_another_embedding_and_head_are_registered_not_edited_in(tmp_path):
    """Embedding and head are parts chosen by kind: an embedding that scales its rows and a head
    that caps its logits are registered here and run through Model.forward unchanged.  Checked
    against the package's own kinds: the scaled embedding on a table equals the plain embedding
    on the table times the scale, and the capped logits are cap * tanh(logits / cap)."""
    import dataclasses
    import os
    from safetensors.torch import load_file, save_file
    from nano_vllm_amd.config.registry import register_architecture
    from nano_vllm_amd.models.qwen3 import build_spec
    from nano_vllm_amd.parts import PartSpec, register_part
    from nano_vllm_amd.parts.embedding import OutputHead, TokenEmbedding
    from nano_vllm_amd.weights import write_random_model

    scale, cap = 3.0, 0.05

    class ScaledEmbedding(TokenEmbedding):
        told = 0

        def on_weights_loaded(self):                  # called once, after every parameter is there
            assert self.weights["weight"].shape == (384, 96)
            type(self).told += 1
            self.factor = torch.tensor(float(self.params["scale"]))

        def forward(self, ids):
            return super().forward(ids) * self.factor

    class CappedHead(OutputHead):
        def forward(self, x):
            c = float(self.params["cap"])
            return torch.tanh(super().forward(x) / c) * c

    def toy_spec(cfg):
        s = build_spec(cfg)
        return dataclasses.replace(
            s, embedding=PartSpec("toy_scaled_embedding", {**s.embedding.params, "scale": scale}),
            head=PartSpec("toy_capped_head", {**s.head.params, "cap": cap}))

    register_part("embedding", "toy_scaled_embedding", ScaledEmbedding, replace=True)
    register_part("head", "toy_capped_head", CappedHead, replace=True)
    register_architecture("ToyScaledCappedLM", H.CONFIGS["b"]["cfg"].from_dict, toy_spec, replace=True)

    base = str(tmp_path / "base")
    write_random_model(base, H.CONFIGS["b"]["cfg"], seed=5, norm_std=0.1, dtype="float32")
    tensors = load_file(os.path.join(base, "model.safetensors"))
    with open(os.path.join(base, "config.json")) as f:
        cfg_json = json.load(f)
    # the toy architecture on the same tensors
    toy = str(tmp_path / "toy")
    os.makedirs(toy)
    save_file(tensors, os.path.join(toy, "model.safetensors"), metadata={"format": "pt"})
    with open(os.path.join(toy, "config.json"), "w") as f:
        json.dump({**cfg_json, "architectures": ["ToyScaledCappedLM"]}, f)
    # the package's own kinds on a table that is already scaled
    scaled = str(tmp_path / "scaled")
    os.makedirs(scaled)
    save_file({k: t * scale if k == "model.embed_tokens.weight" else t for k, t in tensors.items()},
              os.path.join(scaled, "model.safetensors"), metadata={"format": "pt"})
    with open(os.path.join(scaled, "config.json"), "w") as f:
        json.dump(cfg_json, f)

    toks = H.random_tokens(384, 40, 9)
    runs = {}
    for name, folder in (("toy", toy), ("scaled", scaled), ("base", base)):
        r = H.make_runner(folder, "float32", 8, 16, device="cpu", kernels=TorchKernels())
        runs[name] = H.run_portions(r, "x", toks, [25, 1, 14])
    want = torch.tanh(runs["scaled"] / cap) * cap
    assert ScaledEmbedding.told == 1
    assert H.rel_err(runs["toy"], want) < TOL
    assert H.rel_err(runs["base"], runs["scaled"]) > 1e-2        # the scale moves the logits: the check above can fail
    assert (runs["scaled"].abs() > cap).any()                    # and so does the cap
