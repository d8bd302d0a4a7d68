"""A plain, slow Gemma 2 forward pass over whole sequences (NumPy, no cache).

Test-only oracle.  One function per part; nothing here is shared with the
engine's product path: it reads config.json keys itself and looks weights up
by their checkpoint names.  Formulas are taken from the reference's files,
cited as ``path:line`` relative to ``/root/reference/zse-engine/zse_engine``.
Where the reference has no Gemma 2 code (it lists the architecture but runs
it through its Llama path) the formula is the one its Gemma-family kernels and
its adapter's docstring name, and the citation says so.

Every function takes ``dt`` (``np.float32`` or ``np.float64``): all arithmetic
is carried out in that type.
"""
from __future__ import annotations

import math

import numpy as np

GELU_K = 0.7978845608028654  # sqrt(2/pi), orchestrator/kernels.py:1691
GELU_C = 0.044715            # orchestrator/kernels.py:1692


def read_config(cfg: dict) -> dict:
    """config.json keys and defaults as the adapter reads them
    (format/arch/gemma2.py:26-48), plus the Gemma 2 knobs its docstring names
    (format/arch/gemma2.py:3-12) and format/config.py:63-64 holds as fields."""
    nh = cfg["num_attention_heads"]
    out = dict(
        L=cfg["num_hidden_layers"],
        H=cfg["hidden_size"],
        nh=nh,
        nkv=cfg.get("num_key_value_heads", nh),
        hd=cfg.get("head_dim", cfg["hidden_size"] // nh),
        I=cfg["intermediate_size"],
        V=cfg["vocab_size"],
        theta=float(cfg.get("rope_theta", 10000.0)),
        eps=float(cfg.get("rms_norm_eps", 1e-6)),
        window=cfg.get("sliding_window"),
        tied=cfg.get("tie_word_embeddings", True),
        attn_cap=cfg.get("attn_logit_softcapping"),
        final_cap=cfg.get("final_logit_softcapping"),
    )
    out["qpas"] = cfg.get("query_pre_attn_scalar", out["hd"])
    types = cfg.get("layer_types")
    if types is None:
        # layer 0 sliding, layer 1 global, alternating; no window => all global
        types = ["sliding_attention" if (l % 2 == 0 and out["window"]) else "full_attention"
                 for l in range(out["L"])]
    out["sliding"] = [t == "sliding_attention" for t in types]
    return out


def rmsnorm(x, w, eps, dt, unit_offset=True):
    """x * rsqrt(mean(x^2) + eps) * (1 + w).

    rsqrt(sum_sq / H + eps) placement: orchestrator/kernels.py:1435-1465 (:1457);
    the (1 + w) gain of Gemma 2: comment at orchestrator/kernels.py:1476-1478."""
    x = x.astype(dt)
    ms = np.mean(x * x, axis=-1, keepdims=True)
    g = (1.0 + w.astype(dt)) if unit_offset else w.astype(dt)
    return x / np.sqrt(ms + dt(eps)) * g


def rope(x, positions, theta, dt):
    """Rotate-half RoPE over the full head: pair (i, i + hd/2), frequency
    theta^(-2i/hd) (orchestrator/kernels.py:264-297).

    x: [T, heads, hd]; positions: [T]."""
    T, _, hd = x.shape
    half = hd // 2
    i = np.arange(half, dtype=dt)
    freq = dt(1.0) / np.power(dt(theta), (dt(2.0) * i) / dt(hd))
    ang = positions.astype(dt)[:, None] * freq[None, :]            # [T, half]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    x = x.astype(dt)
    a, b = x[..., :half], x[..., half:]
    return np.concatenate([a * c - b * s, b * c + a * s], axis=-1)


def softcap(x, cap, dt):
    """cap * tanh(x / cap) (orchestrator/kernels.py:1714-1727); None = identity."""
    if cap is None:
        return x
    return dt(cap) * np.tanh(x / dt(cap))


def visible(positions_q, positions_k, window):
    """Key j visible to query i iff j <= i (orchestrator/kernels.py:883) and, on
    a sliding layer, i - j < window: the reference keeps the last ``window``
    tokens including the new one (cache/cache_manager.py:409-415)."""
    d = positions_q[:, None] - positions_k[None, :]
    m = d >= 0
    if window is not None:
        m &= d < window
    return m


def attention(q, k, v, positions, scale, cap, window, dt):
    """Grouped-query attention over a whole sequence.

    q: [T, nh, hd], k/v: [T, nkv, hd].  Query head h reads KV head h // (nh/nkv)
    (orchestrator/kernels.py:548, 875).  Scores are scaled, soft-capped, masked,
    then softmax with max subtraction and the weighted sum of values
    (three passes, orchestrator/kernels.py:886-956)."""
    T, nh, hd = q.shape
    nkv = k.shape[1]
    g = nh // nkv
    mask = visible(positions, positions, window)
    out = np.zeros((T, nh, hd), dtype=dt)
    for h in range(nh):
        kh = k[:, h // g, :].astype(dt)
        vh = v[:, h // g, :].astype(dt)
        s = (q[:, h, :].astype(dt) @ kh.T) * dt(scale)
        s = softcap(s, cap, dt)
        s = np.where(mask, s, -np.inf)
        s = s - np.max(s, axis=-1, keepdims=True)
        p = np.exp(s)
        p = p / np.sum(p, axis=-1, keepdims=True)
        out[:, h, :] = p @ vh
    return out


def gelu_tanh(z, dt):
    """0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))) (orchestrator/kernels.py:1690-1693)."""
    z = z.astype(dt)
    return dt(0.5) * z * (dt(1.0) + np.tanh(dt(GELU_K) * (z + dt(GELU_C) * z * z * z)))


def geglu_ffn(x, wg, wu, wd, dt):
    """(gelu_tanh(x Wg^T) * (x Wu^T)) Wd^T; wiring orchestrator/model_runner.py:518-530;
    weights are [out, in] applied as x W^T (orchestrator/kernels.py:1080)."""
    g = x.astype(dt) @ wg.astype(dt).T
    u = x.astype(dt) @ wu.astype(dt).T
    return (gelu_tanh(g, dt) * u) @ wd.astype(dt).T


def embed(tokens, table, scale, dt):
    """Gather rows (orchestrator/kernels.py:1789-1806) times sqrt(hidden)
    (orchestrator/model_runner.py:153-158, 332-339)."""
    return table[np.asarray(tokens)].astype(dt) * dt(scale)


def get_weight(weights, name):
    """Names appear with or without the ``model.`` prefix (format/arch/gemma2.py:50-55)."""
    if name in weights:
        return weights[name]
    return weights["model." + name]


def forward(cfg: dict, weights: dict, tokens, dt=np.float32, embed_scale=None,
            positions=None, return_hidden=False):
    """Logits [T, V] of one whole sequence.

    Layer order (sandwich of four norms): orchestrator/model_runner.py:425-439, 450-537;
    tensor names: format/arch/gemma2.py:57-85; tied head uses the unscaled
    embedding matrix (orchestrator/model_runner.py:566-572); final softcap
    orchestrator/model_runner.py:573-576."""
    c = read_config(cfg)
    T = len(tokens)
    pos = np.arange(T) if positions is None else np.asarray(positions)
    E = get_weight(weights, "embed_tokens.weight")
    if embed_scale is None:
        embed_scale = dt(math.sqrt(c["H"]))
    h = embed(tokens, E, embed_scale, dt)
    scale = dt(c["qpas"]) ** dt(-0.5)
    for l in range(c["L"]):
        p = f"layers.{l}."
        W = lambda n: get_weight(weights, p + n)
        r = h
        x = rmsnorm(h, W("input_layernorm.weight"), c["eps"], dt)
        q = (x @ W("self_attn.q_proj.weight").astype(dt).T).reshape(T, c["nh"], c["hd"])
        k = (x @ W("self_attn.k_proj.weight").astype(dt).T).reshape(T, c["nkv"], c["hd"])
        v = (x @ W("self_attn.v_proj.weight").astype(dt).T).reshape(T, c["nkv"], c["hd"])
        q = rope(q, pos, c["theta"], dt)
        k = rope(k, pos, c["theta"], dt)
        window = c["window"] if c["sliding"][l] else None
        o = attention(q, k, v, pos, scale, c["attn_cap"], window, dt)
        a = o.reshape(T, c["nh"] * c["hd"]) @ W("self_attn.o_proj.weight").astype(dt).T
        a = rmsnorm(a, W("post_attention_layernorm.weight"), c["eps"], dt)
        h = r + a
        r = h
        x = rmsnorm(h, W("pre_feedforward_layernorm.weight"), c["eps"], dt)
        m = geglu_ffn(x, W("mlp.gate_proj.weight"), W("mlp.up_proj.weight"),
                      W("mlp.down_proj.weight"), dt)
        m = rmsnorm(m, W("post_feedforward_layernorm.weight"), c["eps"], dt)
        h = r + m
    x = rmsnorm(h, get_weight(weights, "norm.weight"), c["eps"], dt)
    if return_hidden:
        return x
    head = E if c["tied"] else weights["lm_head.weight"]
    z = x @ head.astype(dt).T
    return softcap(z, c["final_cap"], dt)


# ---------------------------------------------------------------- sampling

def softmax(z, dt=np.float64):
    """Max-subtracted softmax (orchestrator/sampler.py:168-173)."""
    z = np.asarray(z, dtype=dt)
    e = np.exp(z - np.max(z))
    return e / np.sum(e)


def greedy(logits):
    """First index of the maximum (strict ``>`` scan, orchestrator/sampler.py:135-143)."""
    return int(np.argmax(np.asarray(logits)))


def apply_repetition_penalty(logits, counts: dict, penalty):
    """logit / p if positive else logit * p, with p scaled by frequency as
    penalty^(1 + log2(count)) (orchestrator/sampler.py:64-74)."""
    z = np.array(logits, dtype=np.float64)
    for tid, cnt in counts.items():
        if 0 <= tid < len(z):
            s = penalty ** (1.0 + math.log2(cnt)) if cnt > 1 else penalty
            z[tid] = z[tid] / s if z[tid] > 0 else z[tid] * s
    return z


def top_k_filter(z, k):
    """Keep values >= the k-th largest; ties at the threshold stay
    (orchestrator/sampler.py:146-156)."""
    z = np.array(z, dtype=np.float64)
    if k <= 0 or k >= len(z):
        return z
    thr = np.sort(z)[::-1][k - 1]
    z[z < thr] = -np.inf
    return z


def top_p_filter(z, p):
    """Smallest set, by descending probability, whose cumulative probability
    reaches p (orchestrator/sampler.py:186-203)."""
    z = np.array(z, dtype=np.float64)
    if p >= 1.0:
        return z
    pr = softmax(z)
    order = np.argsort(-pr, kind="stable")
    cum = np.cumsum(pr[order])
    n_keep = int(np.searchsorted(cum, p, side="left")) + 1
    keep = np.zeros(len(z), dtype=bool)
    keep[order[:n_keep]] = True
    z[~keep] = -np.inf
    return z


def categorical(probs, u):
    """First index whose running sum exceeds u; last index as fallback
    (orchestrator/sampler.py:205-213)."""
    cum = np.cumsum(np.asarray(probs, dtype=np.float64))
    idx = int(np.searchsorted(cum, u, side="right"))
    return min(idx, len(cum) - 1)


def sample(logits, u, temperature=1.0, top_k=0, top_p=1.0, repetition_penalty=1.0, counts=None):
    """Order of operations of orchestrator/sampler.py:33-98: penalty, greedy
    test, temperature, top-k, top-p, softmax, inverse CDF with the uniform u."""
    z = np.array(logits, dtype=np.float64)
    if repetition_penalty != 1.0 and counts:
        z = apply_repetition_penalty(z, counts, repetition_penalty)
    if temperature <= 0 or temperature < 1e-6:
        return greedy(z)
    z = z * (1.0 / temperature)
    z = top_k_filter(z, top_k)
    z = top_p_filter(z, top_p)
    return categorical(softmax(z), u)
