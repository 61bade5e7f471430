"""Each part alone against the plain implementation's function for it, and a toy mixer with
state of its own, defined here, that is registered, built, loaded and stepped without a
change to the package's files."""
import json
import os

import pytest
import torch

import helpers as H
import plain_qwen3 as plain
from nano_vllm_amd.cache import CacheGroup, CacheManager
from nano_vllm_amd.config import register_architecture
from nano_vllm_amd.engine.batch import StepEntry, build_batch
from nano_vllm_amd.engine.runner import ModelRunner
from nano_vllm_amd.parts import (BuildContext, FixedState, LayerCache, LayerRun, LayerSpec, ModelSpec, ParamDecl,
                                 Part, PartSpec, make_part, register_part)
from nano_vllm_amd.weights import write_random_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 1e-5, "bfloat16": 2.0 ** -6}


def _ctx(dtype, hidden=96, max_position=256):
    from nano_vllm_amd.kernels import HipKernels
    return BuildContext(HipKernels(DEV, dtype, quiet=True), torch.device(DEV), dtype, hidden, max_position)


def _rand(shape, seed, scale=1.0):
    return scale * torch.randn(shape, generator=torch.Generator().manual_seed(seed))


def _err(got, want):
    return float((got.float().cpu() - want).abs().max() / want.abs().max())


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_norm_part(dt):
    dtype = DTYPES[dt]
    part = make_part("norm", PartSpec("rms_norm", {"dim": 120, "eps": 3e-5}), _ctx(dtype))
    assert part.param_decls()["weight"].shape == (120,)
    w = (1 + _rand((120,), 1, 0.1)).to(dtype)
    part.weights["weight"] = w.to(DEV)
    x, r = _rand((9, 120), 2).to(dtype), _rand((9, 120), 3).to(dtype)
    rd = None if dt == "float32" else "bfloat16"
    assert _err(part.forward(x.to(DEV)), plain.rms_norm(x.float(), w.float(), 3e-5, rd)) < TOL[dt]
    y, res = part.forward_add(x.to(DEV), r.to(DEV).clone())
    wy, wr = plain.add_rms_norm(x.float(), r.float(), w.float(), 3e-5, rd)
    assert _err(y, wy) < TOL[dt] and _err(res, wr) < TOL[dt]


def test_position_encoding_part():
    part = make_part("position_encoding", PartSpec("rotary_neox", {"head_dim": 48, "theta": 5e5, "max_position": 300}),
                     _ctx(torch.float32))
    t = part.rotary_table().cpu()
    ang = plain.rope_angles(48, torch.arange(300), 5e5)
    assert t.shape == (300, 48)
    assert float((t[:, :24] - ang.cos()).abs().max()) < 2e-6 and float((t[:, 24:] - ang.sin()).abs().max()) < 2e-6
    none = make_part("position_encoding", PartSpec("none"), _ctx(torch.float32))
    assert none.rotary_table() is None
    # fewer rotated channels than the head has: a narrower table, with the angles of a head of that size
    part = make_part("position_encoding", PartSpec("rotary_neox", {"head_dim": 48, "rotary_dim": 20, "theta": 5e5,
                                                                   "max_position": 300}), _ctx(torch.float32))
    t = part.rotary_table().cpu()
    ang = plain.rope_angles(20, torch.arange(300), 5e5)
    assert t.shape == (300, 20)
    assert float((t[:, :10] - ang.cos()).abs().max()) < 2e-6 and float((t[:, 10:] - ang.sin()).abs().max()) < 2e-6
    for bad in (0, 21, 50):
        with pytest.raises(ValueError, match="rotated channels"):
            make_part("position_encoding", PartSpec("rotary_neox", {"head_dim": 48, "rotary_dim": bad, "theta": 5e5}),
                      _ctx(torch.float32))


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_feed_forward_part(dt):
    dtype = DTYPES[dt]
    part = make_part("feed_forward", PartSpec("swiglu", {"hidden_size": 96, "intermediate_size": 200}), _ctx(dtype))
    decls = part.param_decls()
    assert decls["gate_up_proj.weight"].shape == (400, 96)
    assert [s.name for s in decls["gate_up_proj.weight"].sources] == ["gate_proj.weight", "up_proj.weight"]
    g, u, d = (_rand(s, i, 0.2).to(dtype) for i, s in enumerate([(200, 96), (200, 96), (96, 200)]))
    part.weights["gate_up_proj.weight"] = torch.cat([g, u]).to(DEV)
    part.weights["down_proj.weight"] = d.to(DEV)
    x = _rand((11, 96), 7).to(dtype)
    want = plain.feed_forward(x.float(), g.float(), u.float(), d.float(), None if dt == "float32" else "bfloat16")
    assert _err(part.forward(x.to(DEV)), want) < TOL[dt]


def _attention_setup(dtype, window=None, qk_norm=True, heads=6, kv_heads=3, D=32, hidden=96, page=8, pages=12):
    ctx = _ctx(dtype, hidden)
    ctx.position_encodings["rope"] = make_part("position_encoding", PartSpec(
        "rotary_neox", {"head_dim": D, "theta": 1e4, "max_position": 256}), ctx)
    part = make_part("mixer", PartSpec("attention", {
        "hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": D, "qk_norm": qk_norm,
        "eps": 1e-6, "position_encoding": "rope", "window": window}), ctx)
    w = {"q_proj.weight": _rand((heads * D, hidden), 1, 0.2), "k_proj.weight": _rand((kv_heads * D, hidden), 2, 0.2),
         "v_proj.weight": _rand((kv_heads * D, hidden), 3, 0.2), "o_proj.weight": _rand((hidden, heads * D), 4, 0.2),
         "q_norm.weight": 1 + _rand((D,), 5, 0.1), "k_norm.weight": 1 + _rand((D,), 6, 0.1)}
    w = {k: v.to(dtype) for k, v in w.items()}
    part.weights["qkv_proj.weight"] = torch.cat([w["q_proj.weight"], w["k_proj.weight"], w["v_proj.weight"]]).to(DEV)
    part.weights["o_proj.weight"] = w["o_proj.weight"].to(DEV)
    if qk_norm:
        part.weights["q_norm.weight"] = w["q_norm.weight"].to(DEV)
        part.weights["k_norm.weight"] = w["k_norm.weight"].to(DEV)
    need = part.cache_need()
    cache = CacheManager([CacheGroup(window, (0,))], page, pages, enable_prefix_caching=False)
    from torch_kernels import new_caches
    kc, vc = new_caches(pages, need.num_kv_heads, need.head_dim, page, dtype, DEV)
    lc = LayerCache(group=0, k=kc, v=vc)
    pcfg = plain.PlainConfig(vocab_size=10, hidden_size=hidden, num_layers=1, num_heads=heads, num_kv_heads=kv_heads,
                             head_dim=D, intermediate_size=1, rms_norm_eps=1e-6, rope_theta=1e4, max_position=256,
                             tie_word_embeddings=False, attention_bias=False)
    return part, cache, lc, {f"a.{k}": v.float() for k, v in w.items()}, pcfg


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [None, 10])
def test_attention_part_in_portions(dt, window):
    dtype = DTYPES[dt]
    part, cache, lc, w, pcfg = _attention_setup(dtype, window)
    assert part.cache_need().window == window
    T = 60
    x = _rand((T, 96), 9).to(dtype)
    rd = None if dt == "float32" else "bfloat16"
    want = plain.self_attention(x.float(), torch.arange(T), w, "a", pcfg, window, rd)
    cache.admit("r")
    got, pos = [], 0
    for n in (13, 1, 1, 20, 2, 23):
        cache.reserve("r", pos + n, first_query=pos)
        batch = build_batch([StepEntry("r", [0] * n, pos, [])], cache, 8, 10, DEV)
        got.append(part.forward(x[pos:pos + n].to(DEV), batch, lc))
        pos += n
        cache.check()
    assert _err(torch.cat(got), want) < TOL[dt]
    if window:
        assert cache.table("r", 0)[0] == -1                  # the window has passed the first pages
    part.kernels.check_faults()


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("rot", [12, 32])
def test_attention_part_with_a_rotation_of_fewer_channels(dt, rot):
    """The attention part with a position encoding that rotates the first `rot` of 32 channels,
    through the fused kernel, in portions and single tokens, against a computation in double on
    the whole sequence.  rot = 32 is the package's ordinary case, by the same computation."""
    dtype = DTYPES[dt]
    heads, kv_heads, D, hidden, T = 6, 3, 32, 96, 90
    ctx = _ctx(dtype, hidden)
    ctx.position_encodings["rope"] = make_part("position_encoding", PartSpec(
        "rotary_neox", {"head_dim": D, "rotary_dim": rot, "theta": 1e4, "max_position": 256}), ctx)
    part = make_part("mixer", PartSpec("attention", {
        "hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": D, "qk_norm": True,
        "eps": 1e-6, "position_encoding": "rope", "window": None}), ctx)
    w = {"q": _rand((heads * D, hidden), 1, 0.2), "k": _rand((kv_heads * D, hidden), 2, 0.2),
         "v": _rand((kv_heads * D, hidden), 3, 0.2), "o": _rand((hidden, heads * D), 4, 0.2),
         "qn": 1 + _rand((D,), 5, 0.1), "kn": 1 + _rand((D,), 6, 0.1)}
    w = {k: v.to(dtype) for k, v in w.items()}
    part.weights["qkv_proj.weight"] = torch.cat([w["q"], w["k"], w["v"]]).to(DEV)
    part.weights["o_proj.weight"] = w["o"].to(DEV)
    part.weights["q_norm.weight"], part.weights["k_norm.weight"] = w["qn"].to(DEV), w["kn"].to(DEV)
    x = _rand((T, hidden), 9).to(dtype)

    f = {k: v.double() for k, v in w.items()}
    xd = x.double()
    norm = lambda v, g: v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-6) * g
    ang = torch.arange(T, dtype=torch.float64)[:, None] / (1e4 ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot))[None, :]
    c, s_ = ang.cos()[:, None, :], ang.sin()[:, None, :]

    def rotate(v):                                                  # [T, heads, D]: pairs (i, i + rot/2) of the first rot
        a, b = v[..., : rot // 2], v[..., rot // 2: rot]
        return torch.cat((a * c - b * s_, b * c + a * s_, v[..., rot:]), dim=-1)

    q = rotate(norm((xd @ f["q"].T).reshape(T, heads, D), f["qn"]))
    k = rotate(norm((xd @ f["k"].T).reshape(T, kv_heads, D), f["kn"])).repeat_interleave(heads // kv_heads, 1)
    v = (xd @ f["v"].T).reshape(T, kv_heads, D).repeat_interleave(heads // kv_heads, 1)
    sc = torch.einsum("thd,shd->hts", q, k) * D ** -0.5
    sc = sc.masked_fill(torch.ones(T, T).triu(1).bool(), float("-inf"))
    want = (torch.einsum("hts,shd->thd", torch.softmax(sc, -1), v).reshape(T, heads * D) @ f["o"].T).float()

    need = part.cache_need()
    cache = CacheManager([CacheGroup(None, (0,))], 8, 14, enable_prefix_caching=False)
    from torch_kernels import new_caches
    kc, vc = new_caches(14, need.num_kv_heads, need.head_dim, 8, dtype, DEV)
    lc = LayerCache(group=0, k=kc, v=vc)
    cache.admit("r")
    got, pos = [], 0
    for n in (13, 1, 1, 66, 2, 7):                                  # 66: as many tokens as take the tiled kernel where it serves
        cache.reserve("r", pos + n, first_query=pos)
        batch = build_batch([StepEntry("r", [0] * n, pos, [])], cache, 8, 10, DEV)
        y = part.forward(x[pos:pos + n].to(DEV), batch, lc)
        got.append(y.tensor() if hasattr(y, "tensor") else y)
        pos += n
    assert _err(torch.cat(got), want) < (1e-5 if dt == "float32" else 2.0 ** -5)
    part.kernels.check_faults()


def test_attention_part_without_qk_norm_and_with_bias_declares_its_tensors():
    ctx = _ctx(torch.float32)
    part = make_part("mixer", PartSpec("attention", {"hidden_size": 96, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                                     "qk_norm": False, "bias": True, "position_encoding": None}), ctx)
    decls = part.param_decls()
    assert set(decls) == {"qkv_proj.weight", "qkv_proj.bias", "o_proj.weight"}
    assert [(s.name, s.row, s.rows) for s in decls["qkv_proj.bias"].sources] == [
        ("q_proj.bias", 0, 64), ("k_proj.bias", 64, 32), ("v_proj.bias", 96, 32)]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_block_part(dt):
    """The pre-norm residual block: first without, then with an incoming residual."""
    dtype = DTYPES[dt]
    name = "b"
    folder = H.model_folder(name, dt)
    r = H.make_runner(folder, dt, 8, 16)
    cfg, w = plain.read_folder(folder)
    rd = None if dt == "float32" else "bfloat16"
    T = 20
    toks = H.random_tokens(cfg.vocab_size, T, 3)
    r.cache.admit("x")
    r.cache.reserve("x", T)
    batch = build_batch([StepEntry("x", toks, 0, [])], r.cache, 8, cfg.vocab_size, DEV)
    h0 = w["model.embed_tokens.weight"][torch.tensor(toks)]
    pos = torch.arange(T)

    def plain_layer(i, h, res):
        p = f"model.layers.{i}"
        if res is None:
            x, res = plain.rms_norm(h, w[f"{p}.input_layernorm.weight"], cfg.rms_norm_eps, rd), h
        else:
            x, res = plain.add_rms_norm(h, res, w[f"{p}.input_layernorm.weight"], cfg.rms_norm_eps, rd)
        a = plain.self_attention(x, pos, w, f"{p}.self_attn", cfg, None, rd)
        y, res = plain.add_rms_norm(a, res, w[f"{p}.post_attention_layernorm.weight"], cfg.rms_norm_eps, rd)
        return plain.feed_forward(y, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                                  w[f"{p}.mlp.down_proj.weight"], rd), res

    h = h0.to(dtype).to(DEV)
    m1, r1 = r.model.blocks[0].forward(h, None, batch, r.layer_caches[0])
    wm1, wr1 = plain_layer(0, h0, None)
    assert _err(m1, wm1) < 4 * TOL[dt] and _err(r1, wr1) < TOL[dt]
    m2, r2 = r.model.blocks[1].forward(m1, r1, batch, r.layer_caches[1])
    wm2, wr2 = plain_layer(1, wm1, wr1)
    assert _err(m2, wm2) < 8 * TOL[dt] and _err(r2, wr2) < 4 * TOL[dt]


# ------------------------------------------------------------------------------ a toy mixer with state
class ToyDecayMixer(Part):
    """s_t = decay * s_{t-1} + x_t per request, kept in a state slot; out_t = s_t W^T.
    Written with torch operations: a mixer need not use the package's kernels."""

    def __init__(self, params, build):
        super().__init__(params, build)
        self.hidden = params["hidden_size"]
        self.decay = params["decay"]

    def param_decls(self):
        return {"mix.weight": ParamDecl((self.hidden, self.hidden))}

    def cache_need(self):
        return FixedState({"s": ((self.hidden,), "float32")})

    def forward(self, x, batch, cache):
        out = torch.empty_like(x)
        state = cache.state["s"]
        slots = batch.state_slots.tolist()
        t = 0
        for s, (n, start) in enumerate(zip(batch.q_lens, batch.starts)):
            cur = torch.zeros(self.hidden, device=x.device) if start == 0 else state[slots[s]].clone()
            for i in range(n):
                cur = self.decay * cur + x[t + i].float()
                out[t + i] = (self.weights["mix.weight"].float() @ cur).to(x.dtype)
            state[slots[s]] = cur
            t += n
        return out


def _toy_spec(cfg: dict) -> ModelSpec:
    H_, V = cfg["hidden_size"], cfg["vocab_size"]
    norm = PartSpec("rms_norm", {"dim": H_, "eps": cfg["eps"]})
    ffn = PartSpec("swiglu", {"hidden_size": H_, "intermediate_size": cfg["inner"]})
    attn = PartSpec("attention", {"hidden_size": H_, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16, "qk_norm": True,
                                  "eps": cfg["eps"], "position_encoding": "rope", "window": None})
    toy = PartSpec("toy_decay", {"hidden_size": H_, "decay": cfg["decay"]})
    names = {"mixer_norm": "norm1", "mixer": "mixer", "feed_forward_norm": "norm2", "feed_forward": "ffn"}
    layers = tuple(LayerSpec(PartSpec("pre_norm_residual"), {"mixer_norm": norm, "mixer": m, "feed_forward_norm": norm,
                                                              "feed_forward": ffn}, f"layers.{i}", names)
                   for i, m in enumerate([toy, attn]))
    return ModelSpec(architecture="ToyStateLM", hidden_size=H_, vocab_size=V, max_position=128, dtype="float32",
                     embedding=PartSpec("token_embedding", {"name": "embed"}), layers=layers,
                     order=(LayerRun(0), LayerRun(1), LayerRun(0)),          # the toy layer runs twice
                     final_norm=PartSpec("rms_norm", {"dim": H_, "eps": cfg["eps"], "name": "norm"}),
                     head=PartSpec("output_head", {"name": "head", "tied": True}),
                     position_encodings={"rope": PartSpec("rotary_neox", {"head_dim": 16, "theta": 1e4, "max_position": 128})})


def test_a_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    register_part("mixer", "toy_decay", ToyDecayMixer, replace=True)
    register_architecture("ToyStateLM", lambda d: d, _toy_spec, replace=True)
    cfg = {"architectures": ["ToyStateLM"], "hidden_size": 64, "vocab_size": 99, "inner": 72, "eps": 1e-5, "decay": 0.5,
           "torch_dtype": "float32"}
    folder = write_random_model(str(tmp_path / "toy"), cfg, seed=5, std=0.1)
    r = ModelRunner.from_folder(folder, dtype="float32", page_size=8, num_pages=16, max_requests=3, quiet=True)
    assert len(r.groups) == 1 and r.state_runs == [0, 2] and r.cache.slots.num_slots == 3
    assert not r.cache.prefix_caching
    assert "layers.0.mixer.mix.weight" in r.model.params
    reqs = {k: H.random_tokens(99, n, i) for i, (k, n) in enumerate({"a": 30, "b": 17, "c": 41}.items())}

    def drive(plan):
        pos = {k: 0 for k in reqs}
        got = {k: [] for k in reqs}
        for k in reqs:
            r.cache.admit(k)
        for step in plan:
            entries = []
            for k, n in step:
                r.cache.reserve(k, pos[k] + n)
                entries.append(StepEntry(k, reqs[k][pos[k]:pos[k] + n], pos[k], list(range(n))))
                pos[k] += n
            out = r.step(entries)
            row = 0
            for e in entries:
                got[e.request].append(out[row:row + len(e.tokens)].cpu())
                row += len(e.tokens)
        for k in reqs:
            r.cache.release(k)
        r.cache.check()
        return {k: torch.cat(v) for k, v in got.items()}

    whole = drive([[("a", 30)], [("b", 17)], [("c", 41)]])
    cut = drive([[("a", 7), ("b", 1)], [("c", 20), ("a", 1), ("b", 10)], [("a", 22), ("c", 1)], [("b", 6), ("c", 20)]])
    for k in reqs:
        assert H.rel_err(cut[k], whole[k]) < 2e-5, k
    # the state does its work: a request cut in two without its state differs from the whole
    r.cache.admit("a")
    r.cache.reserve("a", 30)
    r.step([StepEntry("a", reqs["a"][:10], 0, [])])
    for lc in r.layer_caches:
        if lc.state is not None:
            lc.state["s"].zero_()
    lost = r.step([StepEntry("a", reqs["a"][10:], 10, list(range(20)))]).cpu()
    r.cache.release("a")
    assert H.rel_err(lost, whole["a"][10:]) > 1e-3


class ToyDecayMixerOnDevice(ToyDecayMixer):
    """The same mixer with its single-token steps written on the device only: the state rows are
    gathered by batch.state_slots, reset where batch.seq_starts is 0, advanced and scattered back,
    with no value of the batch read on the host.  Such a step can be captured and replayed."""
    replays_state_steps = True

    def forward(self, x, batch, cache):
        if batch.num_decode != batch.num_seqs:
            return super().forward(x, batch, cache)
        state = cache.state["s"]
        rows = batch.state_slots.long()
        old = state.index_select(0, rows) * (batch.seq_starts != 0).float()[:, None]
        new = self.decay * old + x.float()
        state.index_copy_(0, rows, new)
        return (new @ self.weights["mix.weight"].float().T).to(x.dtype)


def test_single_token_steps_of_a_mixer_with_state_on_the_device_are_captured_and_replayed(tmp_path):
    """A model with per-request state decodes through captured steps when its mixer says that it
    handles the state on the device: every replay equals the eager step, with a batch size that is
    captured at its first occurrence (whose set-up runs must not advance the state), rows of
    padding, eager portions of another request between the replays, and bursts on the device."""
    from nano_vllm_amd.sampling.sampler import Sampler
    register_part("mixer", "toy_decay", ToyDecayMixerOnDevice, replace=True)
    register_architecture("ToyStateLM", lambda d: d, _toy_spec, replace=True)
    cfg = {"architectures": ["ToyStateLM"], "hidden_size": 64, "vocab_size": 99, "inner": 72, "eps": 1e-5, "decay": 0.5,
           "torch_dtype": "float32"}
    folder = write_random_model(str(tmp_path / "toy"), cfg, seed=5, std=0.1)
    eager = ModelRunner.from_folder(folder, dtype="float32", page_size=8, num_pages=32, max_requests=5, quiet=True)
    graphed = ModelRunner.from_folder(folder, dtype="float32", page_size=8, num_pages=32, max_requests=5, quiet=True)
    graphed.enable_decode_graphs(max_batch=4, max_len=128)
    assert graphed._graph_max_batch == 4 and graphed.state_runs == [0, 2]
    assert graphed.layer_caches[0].state["s"].shape[0] == 5 + 1           # the last row: the padding rows' slot
    reqs = {f"r{i}": H.random_tokens(99, n, 40 + i) for i, n in enumerate((60, 50, 45))}
    extra = H.random_tokens(99, 23, 77)
    for r in (eager, graphed):
        for rid, toks in reqs.items():
            r.cache.admit(rid)
            r.cache.reserve(rid, 12)
            r.step([StepEntry(rid, toks[:12], 0, [])])
    pos = {rid: 12 for rid in reqs}
    live = list(reqs)
    for step in range(16):
        if step == 6:
            live = live[:2]
        if step == 11:
            live = list(reqs)
        outs = []
        for r in (eager, graphed):
            entries = []
            for rid in live:
                r.cache.reserve(rid, pos[rid] + 1)
                entries.append(StepEntry(rid, [reqs[rid][pos[rid]]], pos[rid], [0]))
            outs.append(r.step(entries).clone())
            if step % 3 == 1:
                r.cache.admit("x")
                r.cache.reserve("x", len(extra))
                r.step([StepEntry("x", extra, 0, [len(extra) - 1])])
                r.cache.release("x")
            torch.cuda.synchronize()
        for rid in live:
            pos[rid] += 1
        assert torch.equal(outs[0], outs[1]), f"replay {step} differs from the eager step"
    assert sorted(graphed._graphs) == [2, 4]
    # bursts: sampled tokens fed back on the device, the state advanced by the replays
    sampler_e, sampler_g = Sampler(eager.kernels, eager.device), Sampler(graphed.kernels, graphed.device)
    temps, seeds, ids = [0.0, 0.9, 0.0], [3, 3, 3], [0, 1, 2]
    last = {rid: reqs[rid][pos[rid]] for rid in reqs}
    toks_e = {rid: [last[rid]] for rid in reqs}
    for _ in range(9):
        entries = []
        for rid in reqs:
            n = pos[rid] + len(toks_e[rid])
            eager.cache.reserve(rid, n)
            entries.append(StepEntry(rid, [toks_e[rid][-1]], n - 1, [0]))
        out = sampler_e.sample(eager.step(entries), temps, seeds, ids, [pos[rid] + len(toks_e[rid]) for rid in reqs])
        for rid, tok in zip(reqs, out):
            toks_e[rid].append(tok)
    toks_g = {rid: [last[rid]] for rid in reqs}
    for n in (4, 5):
        entries = []
        for rid in reqs:
            m = pos[rid] + len(toks_g[rid])
            graphed.cache.reserve(rid, m + n - 1)
            entries.append(StepEntry(rid, [toks_g[rid][-1]], m - 1, [0]))
        for row in graphed.decode_burst(entries, n, sampler_g, temps, seeds, ids):
            for rid, tok in zip(reqs, row):
                toks_g[rid].append(tok)
    assert toks_e == toks_g
    # a mixer that handles its state on the host keeps the runner eager
    register_part("mixer", "toy_decay", ToyDecayMixer, replace=True)
    host = ModelRunner.from_folder(folder, dtype="float32", page_size=8, num_pages=16, max_requests=3, quiet=True)
    host.enable_decode_graphs(max_batch=4, max_len=128)
    assert host._graph_max_batch == 0


# ------------------------------------------------------------------------------ toy feed-forward with routing,
# ------------------------------------------------------------------------------ toy position encoding
class ToyRoutedFeedForward(Part):
    """Each token goes to its top_k of E small experts (up -> silu -> down), mixed with the softmax
    of the chosen router logits.  The router runs in float32.  Products on the chosen rows go through
    the package's own linear kernel; the routing is plain torch."""

    def __init__(self, params, build):
        super().__init__(params, build)
        self.hidden, self.inner = params["hidden_size"], params["inner"]
        self.experts, self.top_k = params["experts"], params["top_k"]

    def param_decls(self):
        d = {"router.weight": ParamDecl((self.experts, self.hidden), dtype="float32")}
        for e in range(self.experts):
            d[f"experts.{e}.up.weight"] = ParamDecl((self.inner, self.hidden))
            d[f"experts.{e}.down.weight"] = ParamDecl((self.hidden, self.inner))
        return d

    def forward(self, x, batch=None):
        w = self.weights
        scores = x.float() @ w["router.weight"].float().T
        top, chosen = scores.topk(self.top_k, dim=-1)
        mix = torch.softmax(top, dim=-1)
        out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
        for e in range(self.experts):
            rows, slot = (chosen == e).nonzero(as_tuple=True)
            if rows.numel() == 0:
                continue
            h = self.kernels.linear(x[rows].contiguous(), w[f"experts.{e}.up.weight"])
            h = (h.float() * torch.sigmoid(h.float())).to(x.dtype)
            y = self.kernels.linear(h, w[f"experts.{e}.down.weight"])
            out.index_add_(0, rows, y.float() * mix[rows, slot, None])
        return out.to(x.dtype)


class ToyInterleavedRotary(Part):
    """Rotation of the pairs (2i, 2i+1) (the package's own encoding pairs i with i + D/2): no
    table, so the mixer calls apply()."""

    def __init__(self, params, build):
        super().__init__(params, build)
        self.head_dim, self.theta = params["head_dim"], params["theta"]

    def rotary_table(self):
        return None

    def apply(self, q, k, positions, num_heads, num_kv_heads, head_dim):
        inv = 1.0 / (self.theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32, device=q.device) / head_dim))
        ang = positions.float()[:, None] * inv[None, :]
        cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
        for x, heads in ((q, num_heads), (k, num_kv_heads)):
            if heads == 0:
                continue
            v = x.float().reshape(x.shape[0], heads, head_dim // 2, 2)
            a, b = v[..., 0], v[..., 1]
            x.copy_(torch.stack((a * cos - b * sin, b * cos + a * sin), dim=-1).reshape(x.shape[0], -1).to(x.dtype))


def _routed_spec(cfg: dict) -> ModelSpec:
    H_, V, D = cfg["hidden_size"], cfg["vocab_size"], cfg["head_dim"]
    norm = PartSpec("rms_norm", {"dim": H_, "eps": cfg["eps"]})
    dense = PartSpec("swiglu", {"hidden_size": H_, "intermediate_size": cfg["inner"]})
    routed = PartSpec("toy_routed", {"hidden_size": H_, "inner": cfg["expert_inner"], "experts": cfg["experts"],
                                     "top_k": cfg["top_k"]})
    attn = PartSpec("attention", {"hidden_size": H_, "num_heads": cfg["heads"], "num_kv_heads": cfg["kv_heads"],
                                  "head_dim": D, "qk_norm": True, "eps": cfg["eps"], "position_encoding": "pairs",
                                  "window": None})
    names = {"mixer_norm": "norm1", "mixer": "attn", "feed_forward_norm": "norm2", "feed_forward": "ffn"}
    layers = tuple(LayerSpec(PartSpec("pre_norm_residual"), {"mixer_norm": norm, "mixer": attn, "feed_forward_norm": norm,
                                                              "feed_forward": f}, f"layers.{i}", names)
                   for i, f in enumerate([routed, dense, routed]))
    return ModelSpec(architecture="ToyRoutedLM", hidden_size=H_, vocab_size=V, max_position=256, dtype="float32",
                     embedding=PartSpec("token_embedding", {"name": "embed"}), layers=layers,
                     order=tuple(LayerRun(i) for i in range(3)),
                     final_norm=PartSpec("rms_norm", {"dim": H_, "eps": cfg["eps"], "name": "norm"}),
                     head=PartSpec("output_head", {"name": "head", "tied": False}),
                     position_encodings={"pairs": PartSpec("toy_pairs_rotary", {"head_dim": D, "theta": cfg["theta"]})})


def _routed_plain(w, cfg, tokens, first_position=0):
    """The toy model on a whole sequence, in double, written without the package."""
    f = lambda name: w[name].double()
    H_, D, hq, hkv = cfg["hidden_size"], cfg["head_dim"], cfg["heads"], cfg["kv_heads"]
    eps = cfg["eps"]
    norm = lambda x, name: x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * f(name)
    T = len(tokens)
    pos = torch.arange(first_position, first_position + T, dtype=torch.float64)
    inv = 1.0 / (cfg["theta"] ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    ang = pos[:, None] * inv[None, :]

    def rotate(x):                                                  # [T, heads, D], pairs (2i, 2i+1)
        v = x.reshape(T, -1, D // 2, 2)
        a, b = v[..., 0], v[..., 1]
        c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
        return torch.stack((a * c - b * s, b * c + a * s), dim=-1).reshape(T, -1, D)

    x = f("embed.weight")[torch.tensor(tokens)]
    for i in range(3):
        p = f"layers.{i}"
        h = norm(x, f"{p}.norm1.weight")
        q = (h @ f(f"{p}.attn.q_proj.weight").T).reshape(T, hq, D)
        k = (h @ f(f"{p}.attn.k_proj.weight").T).reshape(T, hkv, D)
        v = (h @ f(f"{p}.attn.v_proj.weight").T).reshape(T, hkv, D)
        q = rotate(norm(q, f"{p}.attn.q_norm.weight"))
        k = rotate(norm(k, f"{p}.attn.k_norm.weight"))
        k, v = k.repeat_interleave(hq // hkv, 1), v.repeat_interleave(hq // hkv, 1)
        s = torch.einsum("thd,shd->hts", q, k) * D ** -0.5
        s = s.masked_fill(torch.ones(T, T).triu(1).bool(), float("-inf"))
        o = torch.einsum("hts,shd->thd", torch.softmax(s, -1), v).reshape(T, hq * D)
        x = x + o @ f(f"{p}.attn.o_proj.weight").T
        h = norm(x, f"{p}.norm2.weight")
        if i == 1:
            g = h @ f(f"{p}.ffn.gate_proj.weight").T
            y = (g * torch.sigmoid(g) * (h @ f(f"{p}.ffn.up_proj.weight").T)) @ f(f"{p}.ffn.down_proj.weight").T
        else:
            top, chosen = (h @ f(f"{p}.ffn.router.weight").T).topk(cfg["top_k"], dim=-1)
            mix = torch.softmax(top, -1)
            y = torch.zeros_like(h)
            for t in range(T):
                for j in range(cfg["top_k"]):
                    e = int(chosen[t, j])
                    u = f(f"{p}.ffn.experts.{e}.up.weight") @ h[t]
                    y[t] += mix[t, j] * (f(f"{p}.ffn.experts.{e}.down.weight") @ (u * torch.sigmoid(u)))
        x = x + y
    return (norm(x, "norm.weight") @ f("head.weight").T).float()


def test_a_toy_feed_forward_with_routing_and_another_position_encoding(tmp_path):
    """Both are defined above, registered here and run through loader, step function and cache
    like the package's own parts; the result is checked against a computation in double that
    shares nothing with the package."""
    from safetensors.torch import load_file
    register_part("feed_forward", "toy_routed", ToyRoutedFeedForward, replace=True)
    register_part("position_encoding", "toy_pairs_rotary", ToyInterleavedRotary, replace=True)
    register_architecture("ToyRoutedLM", lambda d: d, _routed_spec, replace=True)
    cfg = {"architectures": ["ToyRoutedLM"], "hidden_size": 72, "vocab_size": 131, "inner": 88, "expert_inner": 40,
           "experts": 5, "top_k": 2, "heads": 6, "kv_heads": 2, "head_dim": 16, "eps": 1e-5, "theta": 5e3,
           "torch_dtype": "float32"}
    folder = write_random_model(str(tmp_path / "routed"), cfg, seed=8, std=0.15)
    r = ModelRunner.from_folder(folder, dtype="float32", page_size=8, num_pages=24, max_requests=3, quiet=True)
    w = load_file(os.path.join(folder, "model.safetensors"))
    assert w["layers.0.ffn.router.weight"].dtype == torch.float32 and "layers.2.ffn.experts.4.down.weight" in w
    reqs = {k: H.random_tokens(131, n, 20 + i) for i, (k, n) in enumerate({"a": 45, "b": 70, "c": 23}.items())}
    want = {k: _routed_plain(w, cfg, v) for k, v in reqs.items()}
    got = H.run_portions(r, "a", reqs["a"], [45])
    assert H.rel_err(got, want["a"]) < 2e-5
    got = H.run_portions(r, "b", reqs["b"], H.changing_portions(70, 4))
    assert H.rel_err(got, want["b"]) < 2e-5
    mixed = H.run_mixed(r, reqs, seed=3)
    for k in reqs:
        assert H.rel_err(mixed[k], want[k]) < 2e-5, k
    # only distances count: all positions shifted by 40 give the same logits
    shifted = _routed_plain(w, cfg, reqs["c"], first_position=40)
    assert H.rel_err(shifted, want["c"]) < 1e-9
    r.kernels.check_faults()
