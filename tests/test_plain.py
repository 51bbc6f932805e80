"""Pins the plain implementation by what fixes it beside the reference's text: special cases that
reduce to a library routine, invariants, and the constants the reference's files hold.  Each test
is chosen so that a plausible mistake (wrong pairing or sign in the rotation, a norm in the wrong
place, a forgotten scale) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_minicpm4 as P

DT = P.DT


def test_linear_is_library_linear_times_alpha():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 7, generator=g, dtype=DT)
    w = torch.randn(3, 7, generator=g, dtype=DT)
    b = torch.randn(3, generator=g, dtype=DT)
    assert torch.allclose(P.plain_linear(x, w, b, 0.25), 0.25 * F.linear(x, w, b))
    # fused qkv == separate projections concatenated (fused_linear.cpp:62-71)
    w2 = torch.randn(4, 7, generator=g, dtype=DT)
    fused = P.plain_linear(x, torch.cat([w, w2]))
    assert torch.allclose(fused[:, :3], P.plain_linear(x, w), atol=1e-13)
    assert torch.allclose(fused[:, 3:], P.plain_linear(x, w2), atol=1e-13)


def test_rmsnorm_library_and_invariance():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(4, 96, generator=g, dtype=DT)
    w = torch.randn(96, generator=g, dtype=DT)
    assert torch.allclose(P.plain_rmsnorm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5), atol=1e-13)
    # scale invariance when eps -> 0
    assert torch.allclose(P.plain_rmsnorm(3.7 * x, w, 0.0), P.plain_rmsnorm(x, w, 0.0), atol=1e-12)
    # eps sits inside the root, next to the mean (not the sum)
    one = torch.ones(1, 96, dtype=DT)
    assert torch.allclose(P.plain_rmsnorm(one, torch.ones(96, dtype=DT), 3.0), one / 2.0)


def _cfg_plain_rope(d=16, theta=10000.0, max_pos=64):
    return {"hidden_size": d, "num_attention_heads": 1, "rope_theta": theta,
            "max_position_embeddings": max_pos}


def test_rope_is_complex_multiplication_on_half_split_pairs():
    cfg = _cfg_plain_rope()
    cos, sin = P.plain_rope_tables(cfg)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(9, 2, 16, generator=g, dtype=DT)
    pos = torch.tensor([0, 1, 2, 5, 9, 17, 33, 62, 63])
    y = P.plain_apply_rope(x, pos, cos, sin, 16)
    # pairs are (i, i + d/2): build complex numbers from the two halves
    z = torch.complex(x[..., :8], x[..., 8:])
    inv = 1.0 / (10000.0 ** (torch.arange(8, dtype=DT) * 2 / 16))
    rot = torch.polar(torch.ones(9, 8, dtype=DT), pos.to(DT)[:, None] * inv[None, :])
    zz = z * rot[:, None, :]
    assert torch.allclose(y[..., :8], zz.real, atol=1e-12)
    assert torch.allclose(y[..., 8:], zz.imag, atol=1e-12)
    # position 0 is the identity
    assert torch.equal(y[0], x[0])
    # an interleaved (GPT-J) pairing would give something else
    zi = torch.complex(x[..., 0::2], x[..., 1::2]) * rot[:, None, :]
    assert not torch.allclose(y[..., :8], zi.real, atol=1e-3)


def test_rope_scores_depend_on_distance_only():
    cfg = P.tiny_config_b()
    cos, sin = P.plain_rope_tables(cfg)
    g = torch.Generator().manual_seed(3)
    q = torch.randn(1, 1, 32, generator=g, dtype=DT)
    k = torch.randn(1, 1, 32, generator=g, dtype=DT)
    def score(pq, pk):
        a = P.plain_apply_rope(q, torch.tensor([pq]), cos, sin, 32)
        b = P.plain_apply_rope(k, torch.tensor([pk]), cos, sin, 32)
        return (a * b).sum()
    assert torch.allclose(score(10, 3), score(107, 100), atol=1e-10)
    assert not torch.allclose(score(10, 3), score(10, 4), atol=1e-6)


def test_longrope_factor_choice_and_magnitude():
    cfg = P.tiny_config_b()  # max 256 > original 64 -> long factors, m = sqrt(1 + ln4/ln64)
    cos, sin = P.plain_rope_tables(cfg)
    m = math.sqrt(1 + math.log(4) / math.log(64))
    assert abs(m - 1.1547005) < 1e-6
    assert torch.allclose(cos[0], torch.full((16,), m, dtype=DT))
    assert torch.allclose(cos * cos + sin * sin, torch.full_like(cos, m * m))
    lf = torch.tensor(cfg["rope_scaling"]["long_factor"], dtype=DT)
    inv = 1.0 / (lf * 50000.0 ** (torch.arange(16, dtype=DT) * 2 / 32))
    assert torch.allclose(sin[1], m * torch.sin(inv))
    # at or below the original length: short factors, no magnitude change
    cfg2 = dict(cfg, max_position_embeddings=64)
    cos2, sin2 = P.plain_rope_tables(cfg2)
    sf = torch.tensor(cfg["rope_scaling"]["short_factor"], dtype=DT)
    inv2 = 1.0 / (sf * 50000.0 ** (torch.arange(16, dtype=DT) * 2 / 32))
    assert torch.allclose(sin2[1], torch.sin(inv2))
    # all factors 1 and no extension -> plain rotation
    cfg3 = dict(cfg2, rope_scaling={"type": "longrope", "short_factor": [1.0] * 16,
                                    "long_factor": [1.0] * 16,
                                    "original_max_position_embeddings": 64})
    cfg4 = dict(cfg2, rope_scaling=None)
    assert torch.equal(P.plain_rope_tables(cfg3)[1], P.plain_rope_tables(cfg4)[1])
    # `factor` given replaces the ratio of lengths
    cfg5 = dict(cfg)
    cfg5["rope_scaling"] = dict(cfg["rope_scaling"], factor=16.0)
    c5, _ = P.plain_rope_tables(cfg5)
    assert torch.allclose(c5[0], torch.full((16,), math.sqrt(1 + math.log(16) / math.log(64)), dtype=DT))
    with pytest.raises(ValueError):
        P.plain_rope_tables(dict(cfg, rope_scaling={"type": "bogus"}))
    with pytest.raises(KeyError):
        P.plain_rope_tables(dict(cfg, rope_scaling={"type": "longrope", "short_factor": [1.0] * 16}))


def test_llama3_and_yarn_frequency_maps():
    """What fixes the two maps beside their stated definitions (the reference holds no arithmetic or vector
    for them: parity unpinned): factor 1 leaves every pair alone; the fastest pair is kept and the slowest is
    divided by the factor; the map never raises a frequency and keeps their order; the band edges fall where
    a pair's turns within the original length cross the given numbers."""
    rd, theta, orig = 64, 10000.0, 256
    inv = [1.0 / theta ** (2.0 * i / rd) for i in range(rd // 2)]
    l3 = {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_max_position_embeddings": orig}
    new = P.plain_llama3_frequencies(inv, l3)
    turns = [orig * w / (2 * math.pi) for w in inv]
    for w, n, t in zip(inv, new, turns):
        if t > 4.0:
            assert n == w
        elif t < 1.0:
            assert n == w / 8.0
        else:
            assert w / 8.0 < n < w
    assert any(1.0 <= t <= 4.0 for t in turns) and new == sorted(new, reverse=True)
    assert P.plain_llama3_frequencies(inv, dict(l3, factor=1.0)) == pytest.approx(inv, rel=1e-15)
    # a pair exactly on an edge belongs to both descriptions: the blend is continuous there
    edge = 2 * math.pi * 4.0 / orig
    assert P.plain_llama3_frequencies([edge * (1 + 1e-12)], l3)[0] == pytest.approx(P.plain_llama3_frequencies([edge * (1 - 1e-12)], l3)[0], rel=1e-9)

    yn = {"factor": 4.0, "original_max_position_embeddings": orig}
    new, m = P.plain_yarn_frequencies(inv, yn, rd, theta)
    assert new[0] == inv[0] and new[-1] == pytest.approx(inv[-1] / 4.0) and new == sorted(new, reverse=True)
    assert all(n <= w for n, w in zip(new, inv))
    assert m == pytest.approx(0.1 * math.log(4.0) + 1.0)           # mscale 1 over mscale_all_dim 0
    first = math.floor(rd * math.log(orig / (2 * math.pi * 32)) / (2 * math.log(theta)))
    assert all(new[i] == inv[i] for i in range(max(first, 0) + 1)) and new[max(first, 0) + 1] < inv[max(first, 0) + 1]
    same, one = P.plain_yarn_frequencies(inv, dict(yn, factor=1.0), rd, theta)
    assert same == pytest.approx(inv, rel=1e-15) and one == 1.0
    _, both = P.plain_yarn_frequencies(inv, dict(yn, mscale=0.7, mscale_all_dim=0.7), rd, theta)
    assert both == pytest.approx(1.0)
    # through the tables: the scaled configurations' scores still depend on distances only, and the yarn
    # magnitude multiplies cos and sin alike
    for cfg in (P.tiny_config_d(), P.tiny_config_e()):
        cos, sin = P.plain_rope_tables(cfg)
        mag = float(cos[0, 0])
        assert torch.allclose(cos * cos + sin * sin, torch.full_like(cos, mag * mag))
        assert (mag == 1.0) == (cfg["rope_scaling"].get("rope_type") == "llama3")
        assert not torch.allclose(sin[1], P.plain_rope_tables(dict(cfg, rope_scaling=None))[1][1])


def test_partial_rotary_dim():
    base = {"hidden_size": 64, "num_attention_heads": 2}
    assert P.plain_rotary_dim(base) == 32
    assert P.plain_rotary_dim(dict(base, partial_rotary_factor=0.5)) == 16
    assert P.plain_rotary_dim(dict(base, partial_rotary_factor=1.0)) == 32
    assert P.plain_rotary_dim(dict(base, partial_rotary_factor=0.3)) == 10  # round(9.6)=10
    assert P.plain_rotary_dim(dict(base, partial_rotary_factor=0.28)) == 8  # 9 -> even


def test_attention_is_library_sdpa_with_repeated_kv():
    g = torch.Generator().manual_seed(4)
    T, nh, nkv, d = 11, 6, 2, 16
    q = torch.randn(T, nh, d, generator=g, dtype=DT)
    k = torch.randn(T, nkv, d, generator=g, dtype=DT)
    v = torch.randn(T, nkv, d, generator=g, dtype=DT)
    out = P.plain_attention(q, k, v, 1 / math.sqrt(d))
    kk = k.repeat_interleave(nh // nkv, dim=1)  # head h -> kv head h // g (contiguous groups)
    vv = v.repeat_interleave(nh // nkv, dim=1)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1),
                                         is_causal=True, scale=1 / math.sqrt(d)).transpose(0, 1)
    assert torch.allclose(out, ref, atol=1e-12)
    # a later token does not change earlier outputs
    out2 = P.plain_attention(q[:7], k[:7], v[:7], 1 / math.sqrt(d))
    assert torch.allclose(out[:7], out2, atol=1e-12)
    # one query row, one head: softmax(q k^T) v
    o1 = P.plain_attention(q[:1, :1], k[:1, :1], v[:1, :1], 0.3)
    assert torch.allclose(o1, v[:1, :1])
    # window of 3 keys
    ow = P.plain_attention(q, k, v, 0.25, window=3)
    s = (q[10, 0] @ k[8:11, 0].T) * 0.25
    assert torch.allclose(ow[10, 0], torch.softmax(s, 0) @ v[8:11, 0], atol=1e-12)


def test_swiglu_special_cases():
    g = torch.Generator().manual_seed(5)
    a = torch.randn(4, 10, generator=g, dtype=DT)
    b = torch.randn(4, 10, generator=g, dtype=DT)
    assert torch.allclose(P.plain_swiglu(a, b), F.silu(a) * b, atol=1e-14)
    assert torch.allclose(P.plain_swiglu(a, torch.ones_like(a)), F.silu(a), atol=1e-14)
    assert torch.equal(P.plain_swiglu(torch.zeros_like(a), b), torch.zeros_like(a))
    # gate is the first argument: silu is applied to it, not to `up`
    assert not torch.allclose(P.plain_swiglu(a, b), P.plain_swiglu(b, a))


@pytest.mark.parametrize("make", [P.tiny_config_a, P.tiny_config_b, P.tiny_config_c])
def test_scale_depth_zero_makes_layers_vanish(make):
    cfg = dict(make(), scale_depth=0.0)
    W = P.plain_random_weights(cfg, 3)
    ids = [3, 1, 4, 1, 5]
    logits = P.plain_forward(cfg, W, ids)
    E = W["model.embed_tokens.weight"].to(DT)
    head = W.get("lm_head.weight", W["model.embed_tokens.weight"]).to(DT)
    x = E[torch.tensor(ids)] * cfg["scale_emb"]
    h = F.rms_norm(x, (cfg["hidden_size"],), W["model.norm.weight"].to(DT), cfg["rms_norm_eps"])
    a = cfg["dim_model_base"] / cfg["hidden_size"] if "dim_model_base" in cfg else 1.0
    assert torch.allclose(logits, a * (h @ head.T), atol=1e-10)


def test_logits_linear_in_dim_model_base_and_tied_head_is_unscaled():
    cfg = P.tiny_config_a()
    W = P.plain_random_weights(cfg, 5)
    ids = list(range(7))
    l1 = P.plain_forward(cfg, W, ids)
    l2 = P.plain_forward(dict(cfg, dim_model_base=64), W, ids)
    assert torch.allclose(2 * l1, l2, atol=1e-10)
    # an explicit lm_head equal to the unscaled table gives the same logits as the tied model
    W2 = dict(W)
    W2["lm_head.weight"] = W["model.embed_tokens.weight"].clone()
    assert torch.equal(P.plain_forward(cfg, W2, ids), l1)
    # without dim_model_base there is no logit scale
    cfg3 = {k: v for k, v in cfg.items() if k != "dim_model_base"}
    assert torch.allclose(P.plain_forward(cfg3, W, ids), l1 * (64 / 32), atol=1e-10)


def test_mup_constants_off_is_a_plain_prenorm_decoder():
    cfg = P.tiny_config_a()
    L = cfg["num_hidden_layers"]
    cfg = dict(cfg, scale_depth=math.sqrt(L), scale_emb=1.0)
    del cfg["dim_model_base"]
    assert abs(P.plain_residual_scale(cfg) - 1.0) < 1e-15
    W = {k: v.to(DT) for k, v in P.plain_random_weights(cfg, 9).items()}
    ids = torch.tensor([5, 9, 200, 17, 3, 3])
    T = len(ids)
    x = F.embedding(ids, W["model.embed_tokens.weight"])
    d = 16
    pos = torch.arange(T, dtype=DT)
    inv = 1.0 / (10000.0 ** (torch.arange(8, dtype=DT) * 2 / 16))
    rot = torch.polar(torch.ones(T, 8, dtype=DT), pos[:, None] * inv[None, :])[:, None, :]
    def rope(t):
        z = torch.complex(t[..., :8], t[..., 8:]) * rot
        return torch.cat([z.real, z.imag], -1)
    for l in range(L):
        p = f"model.layers.{l}."
        h = F.rms_norm(x, (64,), W[p + "input_layernorm.weight"], 1e-6)
        q = rope(F.linear(h, W[p + "self_attn.q_proj.weight"]).view(T, 4, d))
        k = rope(F.linear(h, W[p + "self_attn.k_proj.weight"]).view(T, 2, d))
        v = F.linear(h, W[p + "self_attn.v_proj.weight"]).view(T, 2, d)
        o = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                           is_causal=True, enable_gqa=True).transpose(0, 1)
        x = x + F.linear(o.reshape(T, 64), W[p + "self_attn.o_proj.weight"])
        h = F.rms_norm(x, (64,), W[p + "post_attention_layernorm.weight"], 1e-6)
        x = x + F.linear(F.silu(F.linear(h, W[p + "mlp.gate_proj.weight"]))
                         * F.linear(h, W[p + "mlp.up_proj.weight"]), W[p + "mlp.down_proj.weight"])
    ref = F.linear(F.rms_norm(x, (64,), W["model.norm.weight"], 1e-6), W["model.embed_tokens.weight"])
    out = P.plain_forward(cfg, W, ids.tolist())
    assert torch.allclose(out, ref, atol=1e-9)


@pytest.mark.parametrize("make", [P.tiny_config_a, P.tiny_config_b])
def test_shift_of_all_positions_changes_nothing(make):
    cfg = make()
    W = P.plain_random_weights(cfg, 11)
    ids = [7, 8, 9, 10, 11, 12, 13]
    a = P.plain_forward(cfg, W, ids)
    b = P.plain_forward(cfg, W, ids, first_position=40)
    assert torch.allclose(a, b, atol=1e-9)
    # and the model is causal
    c = P.plain_forward(cfg, W, ids[:4])
    assert torch.allclose(a[:4], c, atol=1e-10)
    # sharp weights: the position of a token matters (the rotation is not a no-op)
    d = P.plain_forward(cfg, W, [7, 9, 8, 10])
    assert (d[3] - c[3]).abs().max() > 1e-3


def test_residual_scale_and_weight_names():
    cfg = P.tiny_config_a()
    assert abs(P.plain_residual_scale(cfg) - 1.4 / math.sqrt(2)) < 1e-15
    assert abs(P.plain_residual_scale({"num_hidden_layers": 9}) - 1 / 3) < 1e-15
    names = P.plain_weight_shapes(P.tiny_config_b())
    assert names["model.layers.2.self_attn.k_proj.weight"] == (32, 96)
    assert names["model.layers.0.mlp.down_proj.weight"] == (96, 200)
    assert "lm_head.weight" in names and "lm_head.weight" not in P.plain_weight_shapes(cfg)


def test_sampling_distribution_and_inverse_cdf():
    l = torch.tensor([2.0, 1.0, 0.5, 3.0, -1.0, 3.0])
    p = P.plain_sample_distribution(l, 1.0, 1, 1.0)
    assert p.tolist() == [0, 0, 0, 1, 0, 0]  # first index on ties
    assert P.plain_sample(l, 0.0, 0, 1.0, 0.99) == 3
    p = P.plain_sample_distribution(l, 0.7, 0, 1.0)
    assert torch.allclose(p, torch.softmax(l.to(DT) / 0.7, 0))
    p = P.plain_sample_distribution(l, 1.0, 3, 1.0)
    assert (p > 0).tolist() == [True, False, False, True, False, True]
    assert abs(p.sum() - 1) < 1e-12
    p = P.plain_sample_distribution(l, 1.0, 0, 0.5)  # the two 3.0 hold > 0.5 of the mass together
    assert (p > 0).tolist() == [False, False, False, True, False, True]
    # inverse CDF in vocabulary order
    assert P.plain_sample(l, 1.0, 0, 0.5, 0.0) == 3
    assert P.plain_sample(l, 1.0, 0, 0.5, 0.49) == 3
    assert P.plain_sample(l, 1.0, 0, 0.5, 0.51) == 5
    assert P.plain_sample(l, 1.0, 0, 0.5, 0.999999) == 5
