"""Pins of the plain implementation (tests/plain_qwen3.py) by what fixes it beside the
reference's text: library routines it must reduce to, and invariants, each chosen so that
a plausible mistake fails it.  The reference holds no test vectors of its own."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as plain

torch.manual_seed(0)


def _cfg(**kw):
    d = dict(vocab_size=50, hidden_size=24, num_layers=2, num_heads=4, num_kv_heads=2, head_dim=8,
             intermediate_size=40, rms_norm_eps=1e-5, rope_theta=10000.0, max_position=64,
             tie_word_embeddings=False, attention_bias=False)
    d.update(kw)
    return plain.PlainConfig(**d)


def _weights(cfg, seed=0, dtype=torch.float64, std=0.3):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: (std * torch.randn(*s, generator=g)).to(dtype)
    n = lambda *s: (1 + 0.2 * torch.randn(*s, generator=g)).to(dtype)
    w = {"model.embed_tokens.weight": r(cfg.vocab_size, cfg.hidden_size), "model.norm.weight": n(cfg.hidden_size)}
    if not cfg.tie_word_embeddings:
        w["lm_head.weight"] = r(cfg.vocab_size, cfg.hidden_size)
    for i in range(cfg.num_layers):
        p = f"model.layers.{i}"
        w[f"{p}.input_layernorm.weight"] = n(cfg.hidden_size)
        w[f"{p}.post_attention_layernorm.weight"] = n(cfg.hidden_size)
        w[f"{p}.self_attn.q_proj.weight"] = r(cfg.num_heads * cfg.head_dim, cfg.hidden_size)
        w[f"{p}.self_attn.k_proj.weight"] = r(cfg.num_kv_heads * cfg.head_dim, cfg.hidden_size)
        w[f"{p}.self_attn.v_proj.weight"] = r(cfg.num_kv_heads * cfg.head_dim, cfg.hidden_size)
        w[f"{p}.self_attn.o_proj.weight"] = r(cfg.hidden_size, cfg.num_heads * cfg.head_dim)
        w[f"{p}.self_attn.q_norm.weight"] = n(cfg.head_dim)
        w[f"{p}.self_attn.k_norm.weight"] = n(cfg.head_dim)
        w[f"{p}.mlp.gate_proj.weight"] = r(cfg.intermediate_size, cfg.hidden_size)
        w[f"{p}.mlp.up_proj.weight"] = r(cfg.intermediate_size, cfg.hidden_size)
        w[f"{p}.mlp.down_proj.weight"] = r(cfg.hidden_size, cfg.intermediate_size)
    return w


# ------------------------------------------------------------------------------ norms
def test_rms_norm_is_the_library_routine():
    x, w = torch.randn(5, 24, dtype=torch.float64), torch.randn(24, dtype=torch.float64)
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (24,), w, 1e-5), atol=1e-12)


def test_rms_norm_unit_weight_has_unit_mean_square():
    x = 3.0 * torch.randn(7, 32, dtype=torch.float64)
    y = plain.rms_norm(x, torch.ones(32, dtype=torch.float64), 0.0)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(7, dtype=torch.float64), atol=1e-12)


def test_add_rms_norm_is_norm_of_the_sum_and_returns_the_sum():
    x, r = torch.randn(4, 16, dtype=torch.float64), torch.randn(4, 16, dtype=torch.float64)
    w = torch.randn(16, dtype=torch.float64)
    y, s = plain.add_rms_norm(x, r, w, 1e-6)
    assert torch.equal(s, x + r)
    assert torch.allclose(y, plain.rms_norm(x + r, w, 1e-6), atol=1e-12)


def test_bfloat16_rounding_casts_before_the_weight():
    # layernorm.py:25: cast(x * rsqrt) * w - the normalised value is rounded first
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    w = torch.tensor([1.003, 0.997, 1.5, 0.75])
    y = plain.rms_norm(x, w, 1e-6, rounding="bfloat16")
    n = (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16).float()
    assert torch.equal(y, (n * w).to(torch.bfloat16).float())


# ------------------------------------------------------------------------------ rotary
def test_rope_position_zero_is_the_identity():
    x = torch.randn(1, 3, 16, dtype=torch.float64)
    ang = plain.rope_angles(16, torch.tensor([0]), 10000.0).double()
    assert torch.equal(plain.apply_rope(x, ang), x)


def test_rope_is_complex_multiplication_of_half_split_pairs():
    # pair (i, i + D/2) taken as x1 + i*x2 is multiplied by exp(+i * p * inv_freq_i):
    # an interleaved pairing, or a turn the other way, fails this
    D, p = 16, 7
    x = torch.randn(D, dtype=torch.float64)
    ang = plain.rope_angles(D, torch.tensor([p]), 10000.0).double()
    y = plain.apply_rope(x.view(1, 1, D), ang).view(D)
    inv_freq = torch.tensor([10000.0 ** (-2.0 * i / D) for i in range(D // 2)], dtype=torch.float64)
    z = torch.complex(x[: D // 2], x[D // 2:]) * torch.polar(torch.ones(D // 2, dtype=torch.float64), p * inv_freq)
    assert torch.allclose(y[: D // 2], z.real, atol=1e-5) and torch.allclose(y[D // 2:], z.imag, atol=1e-5)


def test_rope_of_a_vector_worked_by_hand():
    # head_dim 4, theta 10000: the two frequencies are 1 and 10000^(-2/4) = 0.01 (an exponent of
    # i/D would give 0.1, one of 2i/(D/2) would give 0.0001); position 3: angles 3 and 0.03.
    # Pairs (0, 2) and (1, 3) of x = [1, 2, 3, 4]:
    #   y0 = 1 cos 3 - 3 sin 3      y2 = 3 cos 3 + 1 sin 3      cos 3 = -0.98999250, sin 3 = 0.14112001
    #   y1 = 2 cos .03 - 4 sin .03  y3 = 4 cos .03 + 2 sin .03  cos .03 = 0.99955003, sin .03 = 0.02999550
    ang = plain.rope_angles(4, torch.tensor([3]), 10000.0)
    assert torch.allclose(ang, torch.tensor([[3.0, 0.03]]), rtol=1e-6)
    y = plain.apply_rope(torch.tensor([[[1.0, 2.0, 3.0, 4.0]]], dtype=torch.float64), ang.double())
    want = torch.tensor([-1.41335252, 1.87911807, -2.82885748, 4.05819114], dtype=torch.float64)
    assert torch.allclose(y.view(4), want, atol=1e-6)


def test_rope_scores_depend_on_distance_only():
    D = 32
    q, k = torch.randn(1, 1, D, dtype=torch.float64), torch.randn(1, 1, D, dtype=torch.float64)

    def score(m, n):
        a = plain.rope_angles(D, torch.tensor([m]), 1e6).double()
        b = plain.rope_angles(D, torch.tensor([n]), 1e6).double()
        return (plain.apply_rope(q, a) * plain.apply_rope(k, b)).sum()

    assert abs(score(9, 4) - score(25, 20)) < 1e-4           # float32 angles
    assert abs(score(9, 4) - score(9, 5)) > 1e-3


def test_rope_keeps_pair_norms():
    D = 16
    x = torch.randn(1, 2, D, dtype=torch.float64)
    y = plain.apply_rope(x, plain.rope_angles(D, torch.tensor([11]), 10000.0).double())
    n = lambda t: t[..., : D // 2] ** 2 + t[..., D // 2:] ** 2
    assert torch.allclose(n(x), n(y), atol=1e-12)


# ------------------------------------------------------------------------------ attention
@pytest.mark.parametrize("hq,hkv", [(4, 4), (4, 2), (6, 1), (1, 1)])
def test_attention_is_the_library_routine(hq, hkv):
    T, D = 9, 8
    q = torch.randn(T, hq, D, dtype=torch.float64)
    k, v = torch.randn(T, hkv, D, dtype=torch.float64), torch.randn(T, hkv, D, dtype=torch.float64)
    got = plain.causal_attention(q, k, v, D ** -0.5)
    kk, vv = k.repeat_interleave(hq // hkv, 1), v.repeat_interleave(hq // hkv, 1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1),
                                          is_causal=True, scale=D ** -0.5).transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-10)


def test_attention_first_token_returns_its_own_value_and_is_causal():
    T, D = 6, 8
    q, k, v = (torch.randn(T, 2, D, dtype=torch.float64) for _ in range(3))
    o = plain.causal_attention(q, k, v, 0.3)
    assert torch.allclose(o[0], v[0], atol=1e-12)
    k2, v2 = k.clone(), v.clone()
    k2[4:], v2[4:] = 0.0, 5.0                                 # later tokens change
    assert torch.allclose(plain.causal_attention(q, k2, v2, 0.3)[:4], o[:4], atol=1e-12)


def test_attention_window_masks_old_keys():
    T, D, W = 10, 4, 3
    q, k, v = (torch.randn(T, 1, D, dtype=torch.float64) for _ in range(3))
    o = plain.causal_attention(q, k, v, 0.5, window=W)
    for i in range(T):
        lo = max(0, i - W + 1)
        s = (k[lo:i + 1, 0] @ q[i, 0]) * 0.5
        want = torch.softmax(s, 0) @ v[lo:i + 1, 0]
        assert torch.allclose(o[i, 0], want, atol=1e-12)


# ------------------------------------------------------------------------------ feed-forward
def test_swiglu_is_silu_times_up():
    g, u = torch.randn(3, 10, dtype=torch.float64), torch.randn(3, 10, dtype=torch.float64)
    assert torch.allclose(plain.silu_mul(g, u), F.silu(g) * u, atol=1e-12)
    assert torch.count_nonzero(plain.silu_mul(torch.zeros(3, 10), u.float())) == 0


# ------------------------------------------------------------------------------ whole model
def _textbook(w, cfg, ids):
    """x += Attn(norm(x)); x += MLP(norm(x)); norm(x) - the residual written the usual way."""
    ids = torch.as_tensor(ids)
    pos = torch.arange(len(ids))
    x = w["model.embed_tokens.weight"][ids]
    for i in range(cfg.num_layers):
        p = f"model.layers.{i}"
        x = x + plain.self_attention(plain.rms_norm(x, w[f"{p}.input_layernorm.weight"], cfg.rms_norm_eps), pos, w,
                                     f"{p}.self_attn", cfg)
        y = plain.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], cfg.rms_norm_eps)
        x = x + plain.feed_forward(y, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                                   w[f"{p}.mlp.down_proj.weight"])
    return plain.rms_norm(x, w["model.norm.weight"], cfg.rms_norm_eps) @ w["lm_head.weight"].T


def test_deferred_residual_is_the_textbook_pre_norm_net():
    cfg = _cfg()
    w = _weights(cfg)
    ids = [3, 1, 4, 1, 5, 9, 2, 6]
    assert torch.allclose(plain.logits(w, cfg, ids), _textbook(w, cfg, ids), atol=1e-9)


def test_zero_output_projections_leave_the_normalised_embedding():
    cfg = _cfg()
    w = _weights(cfg)
    for i in range(cfg.num_layers):
        w[f"model.layers.{i}.self_attn.o_proj.weight"].zero_()
        w[f"model.layers.{i}.mlp.down_proj.weight"].zero_()
    ids = [7, 7, 2]
    h0 = w["model.embed_tokens.weight"][torch.tensor(ids)]
    want = plain.rms_norm(h0, w["model.norm.weight"], cfg.rms_norm_eps) @ w["lm_head.weight"].T
    assert torch.allclose(plain.logits(w, cfg, ids), want, atol=1e-12)


def _library_model(w, cfg, ids):
    """The whole decoder put together from library routines only: F.embedding, F.rms_norm,
    F.linear, torch.polar (the rotation as a complex product), F.scaled_dot_product_attention
    with is_causal (kv heads repeated for their query heads), F.silu, and the residual written
    the usual way.  Nothing of tests/plain_qwen3.py is called."""
    T, D, Hq, Hkv = len(ids), cfg.head_dim, cfg.num_heads, cfg.num_kv_heads
    x = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    pos = torch.arange(T, dtype=torch.float64)
    freq = torch.tensor([cfg.rope_theta ** (-2.0 * i / D) for i in range(D // 2)], dtype=torch.float64)
    turn = torch.polar(torch.ones(T, D // 2, dtype=torch.float64), pos[:, None] * freq[None, :])     # [T, D/2]

    def rotate(t):                                               # t [T, heads, D]
        z = torch.complex(t[..., : D // 2], t[..., D // 2:]) * turn[:, None, :]
        return torch.cat((z.real, z.imag), dim=-1)

    for i in range(cfg.num_layers):
        p = f"model.layers.{i}"
        a = f"{p}.self_attn"
        y = F.rms_norm(x, (cfg.hidden_size,), w[f"{p}.input_layernorm.weight"], cfg.rms_norm_eps)
        bias = (lambda n: w[f"{a}.{n}.bias"]) if cfg.attention_bias else (lambda n: None)
        q = F.linear(y, w[f"{a}.q_proj.weight"], bias("q_proj")).view(T, Hq, D)
        k = F.linear(y, w[f"{a}.k_proj.weight"], bias("k_proj")).view(T, Hkv, D)
        v = F.linear(y, w[f"{a}.v_proj.weight"], bias("v_proj")).view(T, Hkv, D)
        if not cfg.attention_bias:
            q = F.rms_norm(q, (D,), w[f"{a}.q_norm.weight"], cfg.rms_norm_eps)
            k = F.rms_norm(k, (D,), w[f"{a}.k_norm.weight"], cfg.rms_norm_eps)
        q, k = rotate(q), rotate(k)
        k, v = (t.repeat_interleave(Hq // Hkv, dim=1) for t in (k, v))
        o = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
        x = x + F.linear(o.transpose(0, 1).reshape(T, Hq * D), w[f"{a}.o_proj.weight"])
        y = F.rms_norm(x, (cfg.hidden_size,), w[f"{p}.post_attention_layernorm.weight"], cfg.rms_norm_eps)
        m = F.silu(F.linear(y, w[f"{p}.mlp.gate_proj.weight"])) * F.linear(y, w[f"{p}.mlp.up_proj.weight"])
        x = x + F.linear(m, w[f"{p}.mlp.down_proj.weight"])
    x = F.rms_norm(x, (cfg.hidden_size,), w["model.norm.weight"], cfg.rms_norm_eps)
    return F.linear(x, w["model.embed_tokens.weight"] if cfg.tie_word_embeddings else w["lm_head.weight"])


@pytest.mark.parametrize("kw", [
    dict(),                                                                        # grouped heads, untied
    dict(tie_word_embeddings=True, num_heads=6, num_kv_heads=6, head_dim=4, rope_theta=1e6, rms_norm_eps=1e-6),
    dict(attention_bias=True, num_kv_heads=1, num_layers=3),                       # bias, no q/k norm
    dict(num_heads=8, num_kv_heads=2, head_dim=16, hidden_size=40, intermediate_size=56, vocab_size=97),
])
def test_whole_model_is_the_composition_of_library_routines(kw):
    """The plain model as a whole against a second one that is made of library routines: a
    norm in the wrong place, a wrong pairing or direction of the rotation, a wrong head
    grouping, a missing bias or a q/k norm where there is a bias all fail this.  (The one
    formula both type is the frequency theta^(-2i/D), which the vector worked by hand pins.)"""
    cfg = _cfg(**kw)
    w = _weights(cfg, seed=5)
    if cfg.attention_bias:
        g = torch.Generator().manual_seed(9)
        for i in range(cfg.num_layers):
            for n, rows in (("q_proj", cfg.num_heads), ("k_proj", cfg.num_kv_heads), ("v_proj", cfg.num_kv_heads)):
                w[f"model.layers.{i}.self_attn.{n}.bias"] = torch.randn(rows * cfg.head_dim, generator=g).double()
    ids = torch.randint(0, cfg.vocab_size, (19,), generator=torch.Generator().manual_seed(2)).tolist()
    got = plain.logits(w, cfg, ids)
    want = _library_model(w, cfg, ids)
    # the angles of the plain model are float32, as the reference's table is
    assert torch.allclose(got, want, atol=1e-5 * float(want.abs().max())), float((got - want).abs().max())
    if cfg.attention_bias:
        for i in range(cfg.num_layers):          # the q/k norm weights are there but must not be read
            w[f"model.layers.{i}.self_attn.q_norm.weight"] *= 3.0
        assert torch.equal(plain.logits(w, cfg, ids), got)


def test_shift_of_all_positions_changes_nothing():
    # only distances count; float32 angles limit the agreement
    cfg = _cfg()
    w = _weights(cfg)
    ids = [5, 4, 3, 2, 1, 0, 9]
    a, b = plain.logits(w, cfg, ids), plain.logits(w, cfg, ids, first_position=13)
    assert float((a - b).abs().max()) < 1e-4 * float(a.abs().max())


def test_q_norm_comes_before_the_rotation_and_not_on_values():
    cfg = _cfg(num_layers=1)
    w = _weights(cfg)
    ids = [1, 2, 3, 4]
    base = plain.logits(w, cfg, ids)
    # scaling q_proj leaves the model unchanged up to eps: the norm follows the projection
    w2 = dict(w)
    w2["model.layers.0.self_attn.q_proj.weight"] = 4.0 * w["model.layers.0.self_attn.q_proj.weight"]
    assert torch.allclose(plain.logits(w2, cfg, ids), base, atol=1e-3)
    # scaling v_proj does change it: values are not normalised
    w3 = dict(w)
    w3["model.layers.0.self_attn.v_proj.weight"] = 4.0 * w["model.layers.0.self_attn.v_proj.weight"]
    assert not torch.allclose(plain.logits(w3, cfg, ids), base, atol=1e-3)


def test_tied_head_uses_the_embedding():
    cfg = _cfg(tie_word_embeddings=True)
    w = _weights(cfg)
    h = plain.hidden_states(w, cfg, [1, 2, 3])
    assert torch.allclose(plain.logits(w, cfg, [1, 2, 3]), h @ w["model.embed_tokens.weight"].T)


def test_single_token_attention_is_the_projected_value():
    # one token sees only itself: its output is o_proj(v) with v neither normalised nor turned,
    # each query head taking the value of kv head h // G
    cfg = _cfg(num_layers=1)
    w = _weights(cfg)
    x = torch.randn(1, cfg.hidden_size, dtype=torch.float64)
    got = plain.self_attention(x, torch.tensor([17]), w, "model.layers.0.self_attn", cfg)
    v = (x @ w["model.layers.0.self_attn.v_proj.weight"].T).view(cfg.num_kv_heads, cfg.head_dim)
    o = v.repeat_interleave(cfg.num_heads // cfg.num_kv_heads, 0).reshape(1, -1)
    assert torch.allclose(got, o @ w["model.layers.0.self_attn.o_proj.weight"].T, atol=1e-12)


# ------------------------------------------------------------------------------ sampling
def test_sampling_temperature_zero_is_argmax_lowest_index_on_ties():
    l = torch.tensor([0.5, 2.0, 2.0, -1.0])
    assert plain.sample(l, 0.0) == 1


def test_sampling_small_temperature_is_argmax():
    l = torch.randn(40)
    assert plain.sample(l, 1e-4, seed=3, request=1, position=2) == int(torch.argmax(l))


def test_sampling_frequencies_follow_the_softmax():
    l = torch.tensor([1.0, 0.0, -1.0, 0.5, -2.0])
    T, n = 0.7, 3000
    counts = torch.zeros(5)
    for i in range(n):
        counts[plain.sample(l, T, seed=5, request=0, position=i)] += 1
    p = torch.softmax(l.double() / T, 0)
    chi2 = float(((counts - n * p) ** 2 / (n * p)).sum())
    assert chi2 < 20.0            # 4 degrees of freedom: 18.5 is the 0.1 % point


def test_noise_is_a_pure_function_of_its_key():
    a = plain.exponential_noise(1, 2, 3, 16)
    assert torch.equal(a, plain.exponential_noise(1, 2, 3, 16))
    assert not torch.equal(a, plain.exponential_noise(1, 2, 4, 16))
    assert float(a.min()) > 0
