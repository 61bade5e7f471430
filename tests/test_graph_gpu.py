"""Captured decode steps: every replay is compared with the same step run eagerly, with the
program's own eager work (prompt portions of other requests, a changed batch) and
synchronisations between the replays."""
import pytest
import torch

import helpers as H
from nano_vllm_amd.engine.batch import StepEntry

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["b", "d"])
def test_graph_replays_equal_eager_steps(name, dtype):
    c = H.CONFIGS[name]
    folder = H.model_folder(name, dtype)
    eager = H.make_runner(folder, dtype, c["page"], 64)
    graphed = H.make_runner(folder, dtype, c["page"], 64)
    graphed.enable_decode_graphs(max_batch=8, max_len=c["cfg"].max_position_embeddings)
    V = c["cfg"].vocab_size
    reqs = {f"r{i}": H.random_tokens(V, n, 80 + i) for i, n in enumerate((70, 60, 55))}
    extra = H.random_tokens(V, 37, 99)
    pos = {}
    for r in (eager, graphed):
        for rid, toks in reqs.items():
            r.cache.admit(rid)
            r.cache.reserve(rid, 20)
            r.step([StepEntry(rid, toks[:20], 0, [])])
    for rid in reqs:
        pos[rid] = 20
    live = list(reqs)
    for step in range(24):
        if step == 9:
            live = live[:2]                     # the batch size changes: another graph
        if step == 15:
            live = list(reqs)
        outs = []
        for r in (eager, graphed):
            entries = []
            for rid in live:
                r.cache.reserve(rid, pos[rid] + 1)
                entries.append(StepEntry(rid, [reqs[rid][pos[rid]]], pos[rid], [0]))
            outs.append(r.step(entries).clone())
            if step % 4 == 1:                   # eager work between the replays: a prompt portion
                r.cache.admit("x")
                r.cache.reserve("x", len(extra))
                r.step([StepEntry("x", extra, 0, [len(extra) - 1])])
                r.cache.release("x")
            torch.cuda.synchronize()
        for rid in live:
            pos[rid] += 1
        if dtype == "float32":
            assert torch.equal(outs[0], outs[1]), f"replay {step} differs from the eager step"
        else:
            assert H.rel_err(outs[1], outs[0]) < 1e-5, f"replay {step} differs from the eager step"
    assert sorted(graphed._graphs) == [2, 4]           # three requests run the graph of four, one row of padding
    want = H.plain_logits(folder, reqs["r0"][:pos["r0"]], None if dtype == "float32" else "bfloat16")
    assert H.rel_err(outs[1][0].cpu(), want[-1]) < (2e-5 if dtype == "float32" else 2e-2)
    graphed.kernels.check_faults()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_burst_of_decode_steps_gives_the_tokens_of_single_steps(dtype):
    """Several captured steps in a row with sampling and the next step's metadata made on the
    device: the same tokens as step by step through the host, across page edges, with a row of
    padding, greedy and at a temperature."""
    from nano_vllm_amd.sampling.sampler import Sampler
    c = H.CONFIGS["b"]
    folder = H.model_folder("b", dtype)
    V = c["cfg"].vocab_size
    reqs = {i: H.random_tokens(V, n, 60 + i) for i, n in enumerate((21, 30, 13))}
    temps, seeds = [0.0, 0.8, 1.3], [5, 5, 11]
    runs = []
    for burst in (False, True):
        r = H.make_runner(folder, dtype, c["page"], 64)
        r.enable_decode_graphs(max_batch=8, max_len=c["cfg"].max_position_embeddings)
        sampler = Sampler(r.kernels, r.device)
        toks = {}
        for rid, t in reqs.items():
            r.cache.admit(rid)
            r.cache.reserve(rid, len(t))
            logits = r.step([StepEntry(rid, t, 0, [len(t) - 1])])
            toks[rid] = list(t) + sampler.sample(logits, [temps[rid]], [seeds[rid]], [rid], [len(t)])
        steps = 19                                                  # pages of 8: every request crosses two edges
        if burst:
            for lo, n in ((0, 7), (7, 1), (8, 11)):                 # three bursts, one of a single step
                entries = []
                for rid in reqs:
                    r.cache.reserve(rid, len(toks[rid]) + n - 1)
                    entries.append(StepEntry(rid, [toks[rid][-1]], len(toks[rid]) - 1, [0]))
                out = r.decode_burst(entries, n, sampler, temps, seeds, list(reqs))
                for row in out:
                    for rid, tok in zip(reqs, row):
                        toks[rid].append(tok)
        else:
            for _ in range(steps):
                entries = []
                for rid in reqs:
                    r.cache.reserve(rid, len(toks[rid]))
                    entries.append(StepEntry(rid, [toks[rid][-1]], len(toks[rid]) - 1, [0]))
                logits = r.step(entries)
                out = sampler.sample(logits, temps, seeds, list(reqs), [len(toks[rid]) for rid in reqs])
                for rid, tok in zip(reqs, out):
                    toks[rid].append(tok)
        r.kernels.check_faults()
        runs.append(toks)
    assert runs[0] == runs[1]
    assert all(len(runs[1][rid]) == len(reqs[rid]) + 1 + 19 for rid in reqs)


def test_graphs_captured_at_start_give_the_eager_steps():
    """Every batch size captured up front with stand-in requests (largest first, one memory pool):
    no page or slot stays held, and a later step of real requests replays what an eager step gives."""
    c = H.CONFIGS["b"]
    folder = H.model_folder("b", "float32")
    eager = H.make_runner(folder, "float32", c["page"], 40)
    graphed = H.make_runner(folder, "float32", c["page"], 40)
    graphed.enable_decode_graphs(max_batch=8, max_len=c["cfg"].max_position_embeddings)
    assert graphed.capture_decode_graphs() == 4 and sorted(graphed._graphs) == [1, 2, 4, 8]
    graphed.cache.check()
    assert graphed.cache.pools[0].num_free == 40
    assert graphed.capture_decode_graphs() == 0                        # nothing left to capture
    V = c["cfg"].vocab_size
    reqs = {f"r{i}": H.random_tokens(V, 30, 50 + i) for i in range(3)}
    for r in (eager, graphed):
        for rid, toks in reqs.items():
            r.cache.admit(rid)
            r.cache.reserve(rid, 25)
            r.step([StepEntry(rid, toks[:25], 0, [])])
    for pos in range(25, 30):
        outs = []
        for r in (eager, graphed):
            entries = []
            for rid in reqs:
                r.cache.reserve(rid, pos + 1)
                entries.append(StepEntry(rid, [reqs[rid][pos]], pos, [0]))
            outs.append(r.step(entries).clone())
            torch.cuda.synchronize()
        assert torch.equal(outs[0], outs[1]), f"replay at position {pos} differs from the eager step"
    # too few pages for the largest sizes: they are left for their first occurrence
    small = H.make_runner(folder, "float32", c["page"], 5)
    small.enable_decode_graphs(max_batch=8, max_len=c["cfg"].max_position_embeddings)
    assert small.capture_decode_graphs() == 3 and sorted(small._graphs) == [1, 2, 4]
    graphed.kernels.check_faults()


def test_a_captured_step_of_more_rows_than_the_engines_own_products_take():
    """More than 256 single tokens: the products are the library's, the residual sum runs in their
    epilogue, the logits come from the library's product with a float result, all inside the
    captured step.  Every replay against the eager step, eager work between the replays."""
    name, dtype, n = "b", "bfloat16", 272
    c = H.CONFIGS[name]
    folder = H.model_folder(name, dtype)
    eager = H.make_runner(folder, dtype, c["page"], 2 * n + 8, max_requests=n + 1)
    graphed = H.make_runner(folder, dtype, c["page"], 2 * n + 8, max_requests=n + 1)
    graphed.enable_decode_graphs(max_batch=n, max_len=c["cfg"].max_position_embeddings)
    V = c["cfg"].vocab_size
    reqs = {f"r{i}": H.random_tokens(V, 3 + i % 5 + 6, 300 + i) for i in range(n)}
    extra = H.random_tokens(V, 37, 99)
    pos = {}
    for r in (eager, graphed):
        for rid, toks in reqs.items():
            r.cache.admit(rid)
            r.cache.reserve(rid, len(toks) - 6)
        r.step([StepEntry(rid, toks[:-6], 0, []) for rid, toks in reqs.items()])
    for rid, toks in reqs.items():
        pos[rid] = len(toks) - 6
    for step in range(5):
        outs = []
        for r in (eager, graphed):
            entries = []
            for rid in reqs:
                r.cache.reserve(rid, pos[rid] + 1)
                entries.append(StepEntry(rid, [reqs[rid][pos[rid]]], pos[rid], [0]))
            outs.append(r.step(entries).clone())
            if step % 2 == 1:
                r.cache.admit("x")
                r.cache.reserve("x", len(extra))
                r.step([StepEntry("x", extra, 0, [len(extra) - 1])])
                r.cache.release("x")
            torch.cuda.synchronize()
        for rid in reqs:
            pos[rid] += 1
        assert H.rel_err(outs[1], outs[0]) < 1e-5, f"replay {step} differs from the eager step"
    assert sorted(graphed._graphs) == [n]
    rid = "r7"
    want = H.plain_logits(folder, reqs[rid][:pos[rid]], "bfloat16")
    assert H.rel_err(outs[1][7].cpu(), want[-1]) < 2e-2
    graphed.kernels.check_faults()
