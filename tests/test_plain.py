"""Pins for the plain implementation: what fixes each formula beside the
reference's text.  Vectors marked (ref) are held by the reference's own tests
(tests/test_modal_orchestrator.py, tests/test_orchestrator.py)."""
import math

import numpy as np
import pytest

from conftest import TINY_A, TINY_B, random_tokens
from plain import gemma2_plain as P

F = np.float64
rng = np.random.default_rng(5)


def tiny_weights(cfg, seed, std=0.08, gstd=0.2):
    c = P.read_config(cfg)
    r = np.random.default_rng(seed)
    w = {"embed_tokens.weight": r.normal(0, std, (c["V"], c["H"]))}
    for l in range(c["L"]):
        p = f"layers.{l}."
        w[p + "self_attn.q_proj.weight"] = r.normal(0, std, (c["nh"] * c["hd"], c["H"]))
        w[p + "self_attn.k_proj.weight"] = r.normal(0, std, (c["nkv"] * c["hd"], c["H"]))
        w[p + "self_attn.v_proj.weight"] = r.normal(0, std, (c["nkv"] * c["hd"], c["H"]))
        w[p + "self_attn.o_proj.weight"] = r.normal(0, std, (c["H"], c["nh"] * c["hd"]))
        w[p + "mlp.gate_proj.weight"] = r.normal(0, std, (c["I"], c["H"]))
        w[p + "mlp.up_proj.weight"] = r.normal(0, std, (c["I"], c["H"]))
        w[p + "mlp.down_proj.weight"] = r.normal(0, std, (c["H"], c["I"]))
        for n in ("input_layernorm", "post_attention_layernorm", "pre_feedforward_layernorm",
                  "post_feedforward_layernorm"):
            w[p + n + ".weight"] = r.normal(0, gstd, c["H"])
    w["norm.weight"] = r.normal(0, gstd, c["H"])
    return w


# ------------------------------------------------------------------ norm
def test_rmsnorm_reduces_to_numpy_and_ref_vector():
    x = rng.normal(size=(3, 10))
    y = P.rmsnorm(x, np.zeros(10), 1e-6, F)
    assert np.allclose(y, x / np.sqrt((x * x).mean(-1, keepdims=True) + 1e-6))
    ones = P.rmsnorm(np.ones((2, 8)), np.zeros(8), 1e-6, F)       # (ref) all ones, unit gain -> 1
    assert np.allclose(ones, 1.0, atol=1e-5)


def test_rmsnorm_gain_is_one_plus_w():
    x = rng.normal(size=(2, 6))
    base = P.rmsnorm(x, np.zeros(6), 1e-6, F)
    assert np.allclose(P.rmsnorm(x, np.ones(6), 1e-6, F), 2 * base)       # not w, not w alone
    assert np.allclose(P.rmsnorm(x, -np.ones(6), 1e-6, F), 0.0)
    assert np.allclose(P.rmsnorm(x, np.ones(6), 1e-6, F, unit_offset=False), base)


def test_rmsnorm_eps_sits_inside_the_root_and_rows_are_independent():
    x = np.full((1, 4), 1e-3)
    y = P.rmsnorm(x, np.zeros(4), 1e-2, F)
    assert np.allclose(y, 1e-3 / math.sqrt(1e-6 + 1e-2))
    a = rng.normal(size=(4, 5))
    assert np.allclose(P.rmsnorm(a, np.zeros(5), 1e-6, F)[2], P.rmsnorm(a[2:3], np.zeros(5), 1e-6, F)[0])
    assert np.allclose(P.rmsnorm(7 * a, np.zeros(5), 1e-12, F), P.rmsnorm(a, np.zeros(5), 1e-12, F))


# ------------------------------------------------------------------ rope
def test_rope_explicit_vector_pairs_i_with_i_plus_half():
    # hd 4, theta 100: pair (0,2) turns by pos*1, pair (1,3) by pos*100^(-2/4) = pos/10
    x = np.array([[[1.0, 2.0, 0.0, 0.0]]])
    y = P.rope(x, np.array([3]), 100.0, F)[0, 0]
    assert np.allclose(y, [math.cos(3), 2 * math.cos(0.3), math.sin(3), 2 * math.sin(0.3)])
    z = P.rope(np.array([[[0.0, 0.0, 1.0, 0.0]]]), np.array([3]), 100.0, F)[0, 0]
    assert np.allclose(z, [-math.sin(3), 0, math.cos(3), 0])                 # sign of the rotation


def test_rope_identity_norm_and_relative_property():
    q, k = rng.normal(size=(1, 1, 16)), rng.normal(size=(1, 1, 16))
    assert np.allclose(P.rope(q, np.array([0]), 1e4, F), q)
    r = P.rope(q, np.array([37]), 1e4, F)
    assert np.allclose(np.linalg.norm(r), np.linalg.norm(q))
    dot = lambda p, p2: float((P.rope(q, np.array([p]), 1e4, F) * P.rope(k, np.array([p2]), 1e4, F)).sum())
    assert np.isclose(dot(5, 2), dot(105, 102)) and not np.isclose(dot(5, 2), dot(5, 3))


# ------------------------------------------------------------------ softcap
def test_softcap():
    x = np.linspace(-200, 200, 41)
    assert P.softcap(x, None, F) is x
    y = P.softcap(x, 30.0, F)
    assert np.allclose(y, 30 * np.tanh(x / 30)) and np.all(np.abs(y) < 30) and np.allclose(y, -y[::-1])
    assert np.allclose(P.softcap(np.array([0.01]), 50.0, F), 0.01, rtol=1e-6)
    assert np.all(np.diff(P.softcap(np.linspace(-100, 100, 200), 50.0, F)) > 0)


# ------------------------------------------------------------------ attention
def sdpa(q, k, v):
    T, hd = q.shape
    s = q @ k.T / math.sqrt(hd)
    s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
    p = np.exp(s - s.max(-1, keepdims=True))
    return (p / p.sum(-1, keepdims=True)) @ v


def test_attention_reduces_to_textbook_causal_sdpa():
    T, nh, hd = 9, 3, 8
    q, k, v = (rng.normal(size=(T, nh, hd)) for _ in range(3))
    o = P.attention(q, k, v, np.arange(T), hd ** -0.5, None, None, F)
    for h in range(nh):
        assert np.allclose(o[:, h], sdpa(q[:, h], k[:, h], v[:, h]))
    assert np.allclose(P.attention(q, k, v, np.arange(T), hd ** -0.5, None, T, F), o)    # W >= T
    assert np.allclose(P.attention(q, k, v, np.arange(T), hd ** -0.5, 1e9, None, F), o, atol=1e-9)


def test_attention_ref_vectors_and_window_of_one():
    T, hd = 2, 4
    q = rng.normal(size=(T, 1, hd))
    o = P.attention(q, np.ones((T, 1, hd)), np.full((T, 1, hd), 0.5), np.arange(T), 0.5, None, None, F)
    assert np.allclose(o, 0.5)                                        # (ref) K=1, V=0.5 -> 0.5
    k, v = rng.normal(size=(6, 1, hd)), rng.normal(size=(6, 1, hd))
    q = rng.normal(size=(6, 1, hd))
    assert np.allclose(P.attention(q, k, v, np.arange(6), 1.0, None, 1, F), v)   # sees itself only


def test_gqa_equals_mha_with_repeated_kv_heads():
    T, nh, nkv, hd = 7, 6, 2, 8
    q = rng.normal(size=(T, nh, hd))
    k, v = rng.normal(size=(T, nkv, hd)), rng.normal(size=(T, nkv, hd))
    a = P.attention(q, k, v, np.arange(T), 0.3, 20.0, 4, F)
    b = P.attention(q, np.repeat(k, 3, axis=1), np.repeat(v, 3, axis=1), np.arange(T), 0.3, 20.0, 4, F)
    assert np.allclose(a, b)                    # head h reads kv head h // 3, not h % 2


def test_window_edge_is_i_minus_j_less_than_w():
    # one key stands out: the query sees it at distance W-1 and not at distance W
    T, hd, W = 12, 4, 5
    k = np.zeros((T, 1, hd)); v = np.zeros((T, 1, hd)); q = np.zeros((T, 1, hd))
    k[3, 0, 0] = 10.0; v[3, 0, :] = 1.0; q[:, 0, 0] = 10.0
    o = P.attention(q, k, v, np.arange(T), 1.0, None, W, F)
    assert o[3 + W - 1, 0, 0] > 0.99 and o[3 + W, 0, 0] == 0.0
    assert o[2, 0, 0] == 0.0                                          # causal: not before it exists


def cap_order_vectors(hd=16):
    """Two tokens, one head, chosen so that each wrong order of scale, cap and mask shows.
    q1.k0 = 1e4, q1.k1 = 0, q0.k0 = -1e4; v0 = 1, v1 = 0; scale 0.01, cap 50.
      right (scale, cap, mask): o1 = 1 / (1 + exp(-50 tanh 2)) = 1.000, o0 = 1 (sees key 0 only)
      cap before scale:         o1 = 1 / (1 + exp(-0.5)) = 0.622
      no cap:                   o1 = 1.000 too, but then o0's case below differs
      mask before cap:          the hidden key 1 gets cap * tanh(-inf) = -50 beside key 0's
                                -50 tanh 2 = -48.2:  o0 = 1 / (1 + exp(-1.8)) = 0.858"""
    q = np.zeros((2, 1, hd)); k = np.zeros((2, 1, hd)); v = np.zeros((2, 1, hd))
    q[0, 0, 0], q[1, 0, 0], k[0, 0, 0] = -100.0, 100.0, 100.0
    v[0, 0, :] = 1.0
    return q, k, v, 0.01, 50.0


def test_scale_then_cap_then_mask_inside_attention():
    q, k, v, scale, cap = cap_order_vectors()
    o = P.attention(q, k, v, np.arange(2), scale, cap, None, F)
    assert abs(o[1, 0, 0] - 1.0) < 1e-6          # 0.622 if the cap came before the scale
    assert abs(o[0, 0, 0] - 1.0) < 1e-12         # 0.858 if the mask came before the cap
    # and the cap is there at all: without it the same vectors give another o for a softer case
    q2 = q / 10                                   # q1.k0 = 1e3 -> scaled 10, capped 9.87
    o_cap = P.attention(q2, np.stack([k[0], k[0] * 0.9]), np.stack([v[0], v[1]]), np.arange(2), scale, 5.0, None, F)
    # scores 10 and 9 scaled; capped at 5: 5 tanh 2 = 4.820 and 5 tanh 1.8 = 4.734: nearly a tie
    assert abs(o_cap[1, 0, 0] - 1 / (1 + math.exp(5 * math.tanh(1.8) - 5 * math.tanh(2.0)))) < 1e-9
    assert P.visible(np.array([4]), np.arange(6), 3).tolist() == [[False, False, True, True, True, False]]


# ------------------------------------------------------------------ feed-forward
def test_gelu_and_geglu():
    z = np.array([-5.0, -1.0, 0.0, 0.5, 2.0, 8.0])
    want = [0.5 * t * (1 + math.tanh(0.7978845608028654 * (t + 0.044715 * t ** 3))) for t in z]
    g = P.gelu_tanh(z, F)
    assert np.allclose(g, want) and g[2] == 0 and abs(g[-1] - 8.0) < 1e-9 and abs(g[0]) < 1e-5
    x = rng.normal(size=(3, 4)); wg = rng.normal(size=(5, 4)); wd = rng.normal(size=(4, 5))
    ones_up = np.zeros((5, 4))
    # up = 1 everywhere (through a bias-free trick: x has a constant column)
    x[:, 0] = 1.0; ones_up[:, 0] = 1.0
    assert np.allclose(P.geglu_ffn(x, wg, ones_up, wd, F), P.gelu_tanh(x @ wg.T, F) @ wd.T)
    assert np.allclose(np.ones((2, 3)) @ np.full((4, 3), 0.5).T, 1.5)        # (ref) ones x 0.5 = K * 0.5


# ------------------------------------------------------------------ whole model
@pytest.mark.parametrize("cfg,seed", [(TINY_A, 0), (TINY_B, 1)])
def test_prefix_property_and_position_shift(cfg, seed):
    w = tiny_weights(cfg, seed)
    toks = random_tokens(cfg["vocab_size"], 30, seed)
    z = P.forward(cfg, w, toks, F)
    z_short = P.forward(cfg, w, toks[:17], F)
    assert np.allclose(z[:17], z_short, atol=1e-10)                   # later tokens change nothing
    z_shift = P.forward(cfg, w, toks, F, positions=np.arange(30) + 1000)
    assert np.allclose(z, z_shift, atol=1e-8)                         # only distances count
    assert np.all(np.abs(z) < cfg["final_logit_softcapping"])


def test_embedding_scale_and_tied_unscaled_head():
    cfg = TINY_A
    w = tiny_weights(cfg, 2)
    toks = [3, 9, 27]
    E = w["embed_tokens.weight"]
    assert np.allclose(P.embed(toks, E, math.sqrt(64), F), E[toks] * 8.0)
    x = P.forward(cfg, w, toks, F, return_hidden=True)
    z = P.forward(cfg, w, toks, F)
    assert np.allclose(z, 30 * np.tanh((x @ E.T) / 30))              # the head is E itself, unscaled


def test_post_norms_act_on_the_sublayer_output_not_on_the_sum():
    cfg = TINY_B
    w = tiny_weights(cfg, 3)
    toks = random_tokens(cfg["vocab_size"], 12, 3)
    for l in range(cfg["num_hidden_layers"]):
        w[f"layers.{l}.post_attention_layernorm.weight"][:] = -1.0       # gain 0
        w[f"layers.{l}.post_feedforward_layernorm.weight"][:] = -1.0
    x = P.forward(cfg, w, toks, F, return_hidden=True)
    E = w["embed_tokens.weight"]
    h0 = E[toks] * math.sqrt(cfg["hidden_size"])
    assert np.allclose(x, P.rmsnorm(h0, w["norm.weight"], cfg["rms_norm_eps"], F))


def test_sliding_layers_alternate_from_layer_zero():
    c = P.read_config(TINY_B)
    assert c["sliding"] == [True, False, True]
    assert P.read_config(dict(TINY_B, sliding_window=None))["sliding"] == [False] * 3
    assert P.read_config(dict(TINY_B, layer_types=["full_attention"] * 3))["sliding"] == [False] * 3
    # the window matters: with prompts longer than W, sliding != global
    w = tiny_weights(TINY_B, 4)
    toks = random_tokens(1000, 40, 4)
    a = P.forward(TINY_B, w, toks, F)
    b = P.forward(dict(TINY_B, sliding_window=None), w, toks, F)
    assert np.allclose(a[:16], b[:16]) and not np.allclose(a[20:], b[20:])


def test_float32_agrees_with_float64():
    w = tiny_weights(TINY_A, 6)
    toks = random_tokens(512, 25, 6)
    a = P.forward(TINY_A, {k: v.astype(np.float32) for k, v in w.items()}, toks, np.float32)
    b = P.forward(TINY_A, {k: v.astype(np.float32) for k, v in w.items()}, toks, np.float64)
    assert a.dtype == np.float32 and np.abs(a - b).max() < 2e-5
