"""The plain implementation pinned by what fixes it beside the reference's text:
vectors the reference's own selftest holds, special cases that reduce to a
library routine, and invariants, each chosen so that a plausible mistake fails."""
import math

import numpy as np
import pytest

from helpers import CONFIGS, random_tokens
from plain import qwen3_plain as plain


def rng(seed):
    return np.random.default_rng(seed)


# -------------------------------------------------------------------- RMSNorm
def test_rmsnorm_reference_vector():
    """n=1024, rows=3, U(-1,1), eps 1e-6 against the selftest's own loop
    (/root/reference/src/selftest.cpp:74-100): 1/sqrt(ss/n + eps) * w."""
    r = rng(2)
    x, w = r.uniform(-1, 1, (3, 1024)), r.uniform(-1, 1, 1024)
    want = np.stack([x[i] * (1.0 / math.sqrt(float((x[i] ** 2).sum()) / 1024 + 1e-6)) * w for i in range(3)])
    assert np.abs(plain.rms_norm(x, w, 1e-6) - want).max() < 1e-12


def test_rmsnorm_invariants():
    x = rng(0).normal(size=(4, 50))
    one = np.ones(50)
    y = plain.rms_norm(x, one, 1e-6)
    assert np.allclose(np.sqrt((y ** 2).mean(-1)), 1.0, atol=1e-5)        # unit RMS out
    assert np.allclose(plain.rms_norm(7.0 * x, one, 1e-12), plain.rms_norm(x, one, 1e-12), atol=1e-9)
    tiny = np.full((1, 8), 1e-4)                                          # eps sits inside the root
    assert np.allclose(plain.rms_norm(tiny, np.ones(8), 1e-6), 1e-4 / math.sqrt(1e-8 + 1e-6))
    w = rng(1).normal(size=50)                                            # the weight multiplies, no 1 + w
    assert np.allclose(plain.rms_norm(x, w, 1e-6), y * w)
    assert np.allclose(plain.rms_norm(x, np.zeros(50), 1e-6), 0.0)


# ----------------------------------------------------------------------- rope
def test_rope_reference_vector():
    """rows=2, heads=4, hd=128, theta=1e6, positions {0,5} against the selftest's
    loop (/root/reference/src/selftest.cpp:102-134): pairs (k, k + hd/2)."""
    r = rng(3)
    x = r.uniform(-1, 1, (2, 4, 128))
    want = np.zeros_like(x)
    for m, pos in enumerate((0, 5)):
        for h in range(4):
            for k in range(64):
                a = pos * 1e6 ** (-2.0 * k / 128)
                c, s = math.cos(a), math.sin(a)
                want[m, h, k] = x[m, h, k] * c - x[m, h, k + 64] * s
                want[m, h, k + 64] = x[m, h, k] * s + x[m, h, k + 64] * c
    assert np.abs(plain.rope_neox(x, [0, 5], 1e6) - want).max() < 1e-12


def test_rope_with_angles_in_32_bit():
    """The reference has the angle in 32-bit (src/cuda/rope.cu:20): five tokens in that changes nothing one could
    see, 5,000 tokens in the angle is up to 5000 * 2^-23 = 6e-4 off, and so are the rotated values."""
    r = rng(6)
    x = r.normal(size=(1, 2, 64))
    rounded = plain.float32_angles()
    assert np.abs(plain.rope_neox(x, [5], 1e4, rounded) - plain.rope_neox(x, [5], 1e4)).max() < 2e-6
    far = np.abs(plain.rope_neox(x, [5000], 1e4, rounded) - plain.rope_neox(x, [5000], 1e4)).max()
    assert 1e-6 < far < 6e-4 * np.abs(x).max() * 2
    # it leaves the other sites to the rounder it wraps
    seen = []
    both = plain.float32_angles(lambda site, a: (seen.append(site), a)[1])
    both("gemm_in", x)
    both("rope_angle", x)
    assert seen == ["gemm_in"]


def test_rope_invariants():
    r = rng(4)
    q, k = r.normal(size=(1, 1, 32)), r.normal(size=(1, 1, 32))
    assert np.array_equal(plain.rope_neox(q, [0], 1e4), q)                # position 0: identity
    assert np.allclose(np.linalg.norm(plain.rope_neox(q, [9], 1e4)), np.linalg.norm(q))
    # <R_m q, R_n k> depends on m - n only
    d1 = (plain.rope_neox(q, [12], 1e4) * plain.rope_neox(k, [5], 1e4)).sum()
    d2 = (plain.rope_neox(q, [107], 1e4) * plain.rope_neox(k, [100], 1e4)).sum()
    assert abs(d1 - d2) < 1e-9
    # and on its sign: the transposed rotation would give the same for n - m
    d3 = (plain.rope_neox(q, [5], 1e4) * plain.rope_neox(k, [12], 1e4)).sum()
    assert abs(d1 - d3) > 1e-3
    # half-split pairing: a one-hot at dim 1 spreads to dims 1 and 1 + hd/2 (not to dim 0 or 2)
    e = np.zeros((1, 1, 32))
    e[0, 0, 1] = 1
    assert set(np.nonzero(np.abs(plain.rope_neox(e, [3], 1e4)[0, 0]) > 1e-12)[0]) == {1, 17}
    # pair 0 turns by exactly `pos` radians, whatever theta is
    e = np.zeros((1, 1, 32))
    e[0, 0, 0] = 1
    y = plain.rope_neox(e, [2], 123.0)[0, 0]
    assert np.allclose([y[0], y[16]], [math.cos(2), math.sin(2)])
    # a huge theta leaves every other pair still
    y = plain.rope_neox(r.normal(size=(1, 1, 32)), [1], 1e300)
    assert np.abs(np.delete(y - plain.rope_neox(y, [0], 1e300), [0, 16])).max() == 0


# ------------------------------------------------------------------ attention
def softmax_attention(q, k, v):
    """numpy softmax(Q K^T / sqrt(d) + causal) V for plain multi-head attention."""
    T, nh, hd = q.shape
    out = np.zeros_like(q)
    mask = np.triu(np.full((T, T), -np.inf), 1)
    for h in range(nh):
        s = q[:, h] @ k[:, h].T / math.sqrt(hd) + mask
        p = np.exp(s - s.max(-1, keepdims=True))
        out[:, h] = (p / p.sum(-1, keepdims=True)) @ v[:, h]
    return out


def test_attention_reduces_to_plain_softmax_attention():
    r = rng(5)
    q, k, v = (r.normal(size=(9, 3, 8)) for _ in range(3))
    assert np.abs(plain.attention(q, k, v) - softmax_attention(q, k, v)).max() < 1e-12


def test_attention_special_cases_and_invariants():
    r = rng(6)
    q, k, v = r.normal(size=(7, 4, 8)), r.normal(size=(7, 2, 8)), r.normal(size=(7, 2, 8))
    out = plain.attention(q, k, v)
    assert np.array_equal(out[0, 0], v[0, 0]) and np.array_equal(out[0, 3], v[0, 1])   # one key: its value
    zero = plain.attention(np.zeros_like(q), k, v)
    assert np.allclose(zero[4, 1], v[:5, 0].mean(0))                     # q = 0: the mean of the prefix
    # head h reads kv head h // G: heads 0, 1 -> 0 and heads 2, 3 -> 1
    k2, v2 = k.copy(), v.copy()
    k2[:, 1] += 1.0
    v2[:, 1] -= 2.0
    out2 = plain.attention(q, k2, v2)
    assert np.array_equal(out2[:, :2], out[:, :2]) and not np.allclose(out2[:, 2:], out[:, 2:])
    # causal: later tokens do not change earlier rows
    k3, v3 = k.copy(), v.copy()
    k3[5:], v3[5:] = 9.0, -9.0
    assert np.array_equal(plain.attention(q, k3, v3)[:5], out[:5])
    # the scale is 1/sqrt(hd): doubling q equals the unscaled scores of hd/4
    big = plain.attention(np.sqrt(8.0) * q, k, v)
    s = np.einsum("d,td->t", q[6, 0], k[:, 0])
    p = np.exp(s - s.max())
    assert np.allclose(big[6, 0], (p / p.sum()) @ v[:, 0])


def test_attention_window():
    r = rng(7)
    q, k, v = (r.normal(size=(12, 2, 8)) for _ in range(3))
    assert np.array_equal(plain.attention(q, k, v, window=12), plain.attention(q, k, v))
    w1 = plain.attention(q, k, v, window=1)
    assert np.array_equal(w1, v)                                          # only itself
    w3 = plain.attention(q, k, v, window=3)
    assert np.allclose(w3[7], plain.attention(q[5:8], k[5:8], v[5:8])[2])  # keys 5, 6, 7 and no others


# ----------------------------------------------------------------- feed-forward
def test_swiglu():
    g = np.array([0.0, 50.0, -50.0, 1.0])
    u = np.array([3.0, 2.0, 2.0, -1.0])
    y = plain.swiglu(g, u)
    assert y[0] == 0.0 and abs(y[1] - 100.0) < 1e-9 and abs(y[2]) < 1e-18
    assert abs(y[3] + 1.0 / (1.0 + math.exp(-1.0))) < 1e-15
    assert not np.allclose(plain.swiglu(g, u), plain.swiglu(u, g))        # the gate is the first operand


def test_linear_is_x_wt():
    r = rng(8)
    x, w = r.normal(size=(3, 5)), r.normal(size=(4, 5))
    assert np.array_equal(plain.linear(x, w), x @ w.T)
    assert np.array_equal(plain.linear(x, np.eye(5)), x)


def test_round_bf16_matches_torch():
    import torch
    x = rng(9).normal(size=1000).astype(np.float32) * 3
    x[:4] = [1.00390625, 1.01171875, -1.00390625, 3.0e38]                 # ties go to even
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float64).numpy()
    assert np.array_equal(plain.round_bf16(x), want)


# ---------------------------------------------------------------- whole model
@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    import tinyinfer_amd  # noqa: F401
    from helpers import read_folder
    from tinyinfer_amd.weights import write_model_folder
    d = str(tmp_path_factory.mktemp("plain_b"))
    write_model_folder(d, CONFIGS["B"], seed=11)
    return read_folder(d)


def test_model_is_causal_and_shift_invariant(model_b):
    cfg, w = model_b
    toks = random_tokens(20, cfg["vocab_size"], 1)
    full = plain.forward(w, cfg, toks)
    assert full.shape == (20, cfg["vocab_size"])
    assert np.abs(plain.forward(w, cfg, toks[:11]) - full[:11]).max() < 1e-12   # a prefix gives the same rows
    # only distances count: shifting every position changes nothing
    assert np.abs(plain.forward(w, cfg, toks, first_position=1000) - full).max() < 1e-9


def test_every_weight_matters_where_it_should(model_b):
    """A norm in the wrong place or a forgotten weight changes the logits: scaling
    one tensor changes them, except where the math says it cannot."""
    cfg, w = model_b
    toks = random_tokens(12, cfg["vocab_size"], 2)
    base = plain.forward(w, cfg, toks)
    for name in ("model.layers.1.input_layernorm.weight", "model.layers.0.post_attention_layernorm.weight",
                 "model.layers.2.self_attn.q_norm.weight", "model.layers.2.self_attn.k_norm.weight",
                 "model.norm.weight", "lm_head.weight", "model.layers.1.mlp.up_proj.weight"):
        w2 = dict(w)
        w2[name] = w[name] * 1.5
        assert np.abs(plain.forward(w2, cfg, toks) - base).max() > 1e-4, name
    # q and k are normed per head after the projection: scaling q_proj or k_proj changes (almost) nothing
    for name in ("model.layers.0.self_attn.q_proj.weight", "model.layers.0.self_attn.k_proj.weight"):
        w2 = dict(w)
        w2[name] = w[name] * 1.5
        assert np.abs(plain.forward(w2, cfg, toks) - base).max() < 1e-4, name
    # v is not normed
    w2 = dict(w)
    w2["model.layers.0.self_attn.v_proj.weight"] = w["model.layers.0.self_attn.v_proj.weight"] * 1.5
    assert np.abs(plain.forward(w2, cfg, toks) - base).max() > 1e-4
    # untied: the head is its own matrix; tied would read the embedding
    tied = dict(cfg, tie_word_embeddings=True)
    assert np.abs(plain.forward(w, tied, toks) - base).max() > 1e-3


def test_one_layer_one_head_by_hand():
    """A one-layer, one-head model written out with numpy routines only."""
    r = rng(12)
    H, hd, F, V, T = 8, 8, 12, 20, 5
    cfg = dict(num_hidden_layers=1, num_attention_heads=1, num_key_value_heads=1, head_dim=hd,
               rms_norm_eps=1e-6, rope_theta=100.0, tie_word_embeddings=True)
    p = "model.layers.0."
    w = {"model.embed_tokens.weight": r.normal(size=(V, H)), "model.norm.weight": 1 + 0.1 * r.normal(size=H),
         p + "input_layernorm.weight": 1 + 0.1 * r.normal(size=H),
         p + "post_attention_layernorm.weight": 1 + 0.1 * r.normal(size=H),
         p + "self_attn.q_proj.weight": r.normal(size=(hd, H)), p + "self_attn.k_proj.weight": r.normal(size=(hd, H)),
         p + "self_attn.v_proj.weight": r.normal(size=(hd, H)), p + "self_attn.o_proj.weight": r.normal(size=(H, hd)),
         p + "self_attn.q_norm.weight": 1 + 0.1 * r.normal(size=hd),
         p + "self_attn.k_norm.weight": 1 + 0.1 * r.normal(size=hd),
         p + "mlp.gate_proj.weight": r.normal(size=(F, H)), p + "mlp.up_proj.weight": r.normal(size=(F, H)),
         p + "mlp.down_proj.weight": r.normal(size=(H, F))}
    toks = [3, 7, 7, 0, 19]

    def norm(x, g):
        return x / np.sqrt((x ** 2).mean(-1, keepdims=True) + 1e-6) * g

    def rot(x):
        out = np.zeros_like(x)
        for t in range(T):
            for k in range(hd // 2):
                a = t * 100.0 ** (-2.0 * k / hd)
                out[t, k] = x[t, k] * math.cos(a) - x[t, k + hd // 2] * math.sin(a)
                out[t, k + hd // 2] = x[t, k] * math.sin(a) + x[t, k + hd // 2] * math.cos(a)
        return out

    x = w["model.embed_tokens.weight"][toks]
    h = norm(x, w[p + "input_layernorm.weight"])
    q = rot(norm(h @ w[p + "self_attn.q_proj.weight"].T, w[p + "self_attn.q_norm.weight"]))
    k = rot(norm(h @ w[p + "self_attn.k_proj.weight"].T, w[p + "self_attn.k_norm.weight"]))
    v = h @ w[p + "self_attn.v_proj.weight"].T
    s = q @ k.T / math.sqrt(hd) + np.triu(np.full((T, T), -np.inf), 1)
    a = np.exp(s - s.max(-1, keepdims=True))
    x = x + (a / a.sum(-1, keepdims=True)) @ v @ w[p + "self_attn.o_proj.weight"].T
    h = norm(x, w[p + "post_attention_layernorm.weight"])
    g = h @ w[p + "mlp.gate_proj.weight"].T
    x = x + (g / (1 + np.exp(-g)) * (h @ w[p + "mlp.up_proj.weight"].T)) @ w[p + "mlp.down_proj.weight"].T
    want = norm(x, w["model.norm.weight"]) @ w["model.embed_tokens.weight"].T
    assert np.abs(plain.forward(w, cfg, toks) - want).max() < 1e-10


# ------------------------------------------------------------------- sampling
def test_sampling_distribution():
    l = np.array([1.0, 3.0, 3.0, -2.0, 0.5])
    assert plain.argmax_lowest(l) == 1                                    # ties: the lowest index
    p = plain.sample_distribution(l, 1.0)
    want = np.exp(l - 3.0)
    assert np.allclose(p, want / want.sum())
    assert np.allclose(plain.sample_distribution(l, 0.5), np.exp(2 * (l - 3)) / np.exp(2 * (l - 3)).sum())
    assert plain.sample_distribution(l, 1.0, top_k=1).tolist() == [0, 0.5, 0.5, 0, 0]     # equals stay together
    p3 = plain.sample_distribution(l, 1.0, top_k=3)
    assert p3[3] == 0 and p3[4] == 0 and p3[0] > 0
    pp = plain.sample_distribution(l, 1.0, top_p=0.5)
    assert set(np.nonzero(pp)[0]) == {1, 2}
    assert plain.draw(np.array([0.25, 0.25, 0.5]), 0.0) == 0
    assert plain.draw(np.array([0.25, 0.25, 0.5]), 0.26) == 1
    assert plain.draw(np.array([0.25, 0.25, 0.5]), 0.999) == 2
    assert plain.draw(np.array([0.0, 1.0, 0.0]), 0.0) == 1
