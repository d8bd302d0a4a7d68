"""The window and the contexts of the real models: a window of 4,096 keys, contexts of 4,095 to
8,320 tokens, heads of 256 and 128 channels, pages of 16 tokens.  The attention kernels alone
against NumPy at a handful of rows (decoded tokens in both cuts of their keys with the grid
that starts at the window, portions of 512 rows behind 7,680 tokens on every portion kernel),
and a two-layer slice at Gemma 2 2B's widths fed 4,090 tokens in portions of 512 and then one
by one across the window's edge, on pools so small that the sliding layer's pages are given
back and used again.

In every kernel case the key that a query's window begins with carries most of the weight,
and the key just before it (outside the window by one) would carry as much and has a value of
50: a window that is off by one key in either direction shows as an error of order 1."""
import numpy as np
import pytest

from gpu_util import assert_close, make_runner
from plain import gemma2_plain as P
from test_gpu_kernels import bf16, np_attention, up

pytestmark = pytest.mark.gpu

W = 4096
BS = 16
GEOMETRIES = [(4, 2, 256), (4, 2, 128)]         # heads, KV heads, head_dim: two heads a KV head
SCALE, CAP = 0.0625, 50.0


@pytest.fixture(scope="module")
def rt():
    from zse_amd.runtime.device import Runtime
    return Runtime.get()


def marked_request(rng, ctx, n, nh, nkv, hd, window, rows, dtype):
    """Keys, values [ctx, nkv, hd] and queries [n, nh, hd] for a request whose last ``n`` tokens
    are new.  For each of ``rows`` (indices among the new tokens) channel c (its number in
    ``rows``) is the row's own: the query has 16 there and next to nothing elsewhere, the first
    key of its window has 8 there, and so has the key before it, whose value is 50."""
    kk, vv = rng.normal(size=(ctx, nkv, hd)), rng.normal(size=(ctx, nkv, hd))
    qq = rng.normal(size=(n, nh, hd))
    kk[:, :, :len(rows)] = 0.0
    for c, i in enumerate(rows):
        pos = ctx - n + i
        first = max(0, pos - window + 1) if window else 0
        qq[i] *= 0.125
        qq[i, :, :len(rows)] = 0.0
        qq[i, :, c] = 16.0
        kk[first, :, c] = 8.0
        if first > 0:
            kk[first - 1, :, c] = 8.0
            vv[first - 1] = 50.0
    if dtype == "bfloat16":
        kk, vv, qq = (bf16(a).astype(np.float64) for a in (kk, vv, qq))
    return kk, vv, qq


def lay_out(kk, vv, table_row, free, vt, kc, vc, holes_before=0):
    """Scatter a request's keys and values into pages; pages that lie wholly before
    ``holes_before`` are not stored at all and stay holes (-1) in the table, as pages that the
    window has passed are."""
    ctx = kk.shape[0]
    for j in range(-(-ctx // BS)):
        if (j + 1) * BS <= holes_before:
            continue
        pg = free.pop()
        table_row[j] = pg
        bk, bv = kk[j * BS:(j + 1) * BS], vv[j * BS:(j + 1) * BS]
        kc[pg, :, :len(bk)] = bk.transpose(1, 0, 2)
        if vt:
            vc[pg, :, :, :len(bv)] = bv.transpose(1, 2, 0)
        else:
            vc[pg, :, :len(bv)] = bv.transpose(1, 0, 2)


@pytest.mark.parametrize("nh,nkv,hd", GEOMETRIES)
@pytest.mark.parametrize("kernel", ["plain_f32", "mfma"])
def test_decoded_tokens_at_the_real_window(rt, kernel, nh, nkv, hd):
    dtype = "float32" if kernel == "plain_f32" else "bfloat16"
    k = rt.kernels(dtype)
    vt = kernel == "mfma"
    rng = np.random.default_rng(hd)
    ctxs = [4095, 4096, 4097, 8191, 8320, 4112, 300]
    R = len(ctxs)
    max_ctx = 8320
    max_blocks = max_ctx // BS
    pages = sum(-(-c // BS) for c in ctxs) + 1
    # stale values in every place that is not written below, page 0 (which table holes read) included
    kc = rng.normal(size=(pages, nkv, BS, hd)).astype(np.float32)
    vc = rng.normal(size=(pages, nkv, hd, BS) if vt else (pages, nkv, BS, hd)).astype(np.float32)
    free = list(range(pages - 1, 0, -1))
    table = np.full((R, max_blocks), -1, np.int32)
    want, q_rows, leaks = [], [], []
    for r, ctx in enumerate(ctxs):
        kk, vv, qq = marked_request(rng, ctx, 1, nh, nkv, hd, W, [0], dtype)
        want.append(np_attention(qq, kk, vv, [ctx - 1], SCALE, CAP, W))
        if ctx > W:
            leaks += [np.abs(np_attention(qq, kk, vv, [ctx - 1], SCALE, CAP, w) - want[-1]).max() for w in (W - 1, W + 1)]
        # the pages the window had passed before this token came are gone, for the longer requests
        lay_out(kk, vv, table[r], free, vt, kc, vc, holes_before=max(0, ctx - 1 - W + 1) if r >= 3 else 0)
        q_rows.append(qq.reshape(1, nh * hd))
    assert (table[4, :(8320 - W) // BS] == -1).all() and table[4, (8320 - W) // BS] >= 0
    want = np.concatenate(want)
    Q, KC, VC, TBL = up(rt, np.concatenate(q_rows), dtype), up(rt, kc, dtype), up(rt, vc, dtype), rt.upload(table)
    QS, CL = rt.upload(np.arange(R + 1, dtype=np.int32)), rt.upload(np.array(ctxs, np.int32))
    POS, REQ = rt.upload(np.array(ctxs, np.int32) - 1), rt.upload(np.arange(R, dtype=np.int32))
    for chunk in ((64, 32) if kernel == "mfma" else (0,)):
        OUT = rt.zeros((R, nh * hd), dtype)
        if kernel == "mfma":
            ws = rt.zeros((k.zk_attention_bf16_workspace(R, nh, hd, max_ctx) // 4 + 1,), "float32")
            k.zk_attention_bf16(Q.ptr, nh * hd, KC.ptr, VC.ptr, TBL.ptr, max_blocks, QS.ptr, CL.ptr, OUT.ptr, R, 0, 1,
                                max_ctx, nh, nkv, hd, BS, SCALE, CAP, W, chunk, ws.ptr, ws.nbytes, rt.stream)
        else:
            k.zk_attention_plain(Q.ptr, nh * hd, KC.ptr, VC.ptr, TBL.ptr, max_blocks, REQ.ptr, POS.ptr, OUT.ptr, R,
                                 nh, nkv, hd, BS, SCALE, CAP, W, 0, rt.stream)
        got = rt.download_f32(OUT).reshape(R, nh, hd)
        err = np.abs(got - want).max(axis=(1, 2))
        tol = 2e-5 if dtype == "float32" else 0.02
        assert (err < tol).all(), f"chunk {chunk}: errors per context {dict(zip(ctxs, err))}"
    # the edge decides: a window one key longer or shorter gives another result altogether
    assert min(leaks) > 0.5, leaks


@pytest.mark.parametrize("window", [W, 0])
@pytest.mark.parametrize("nh,nkv,hd", GEOMETRIES)
@pytest.mark.parametrize("kernel", ["plain_f32", "mfma"])
def test_a_portion_of_512_rows_behind_7680_tokens(rt, kernel, nh, nkv, hd, window):
    dtype = "float32" if kernel == "plain_f32" else "bfloat16"
    k = rt.kernels(dtype)
    vt = kernel == "mfma"
    rng = np.random.default_rng(hd + window)
    past, n = 7680, 512
    ctx = past + n
    rows = [0, 31, 33, 255, 300, 511]
    kk, vv, qq = marked_request(rng, ctx, n, nh, nkv, hd, window, rows, dtype)
    want = np_attention(qq[rows], kk, vv, [past + i for i in rows], SCALE, CAP, window)
    max_blocks = ctx // BS + 2
    pages = ctx // BS + 2
    kc = rng.normal(size=(pages, nkv, BS, hd)).astype(np.float32)
    vc = rng.normal(size=(pages, nkv, hd, BS) if vt else (pages, nkv, BS, hd)).astype(np.float32)
    table = np.full((1, max_blocks), -1, np.int32)
    # what the window had passed before the portion came is gone
    lay_out(kk, vv, table[0], list(rng.permutation(np.arange(1, pages))), vt, kc, vc,
            holes_before=max(0, past - window + 1) if window else 0)
    Q, KC, VC, TBL = up(rt, qq.reshape(n, nh * hd), dtype), up(rt, kc, dtype), up(rt, vc, dtype), rt.upload(table)
    QS, CL = rt.upload(np.array([0, n], np.int32)), rt.upload(np.array([ctx], np.int32))
    POS, REQ = rt.upload(np.arange(past, ctx, dtype=np.int32)), rt.upload(np.zeros(n, np.int32))
    modes = [0] if kernel == "plain_f32" else [0, 1, 4, 5] + ([8] if hd <= 128 else [])
    for mode in modes:
        OUT = rt.zeros((n, nh * hd), dtype)
        if kernel == "mfma":
            need = k.zk_attention_bf16_portion_workspace(n + 128, nh, nkv, hd) + 4096
            ws = rt.zeros((need // 4,), "float32")
            k.zk_attention_bf16_portion_kernel(mode)
            try:
                k.zk_attention_bf16(Q.ptr, nh * hd, KC.ptr, VC.ptr, TBL.ptr, max_blocks, QS.ptr, CL.ptr, OUT.ptr, 1, 1,
                                    n, ctx, nh, nkv, hd, BS, SCALE, CAP, window, 64, ws.ptr, ws.nbytes, rt.stream)
            finally:
                k.zk_attention_bf16_portion_kernel(0)
        else:
            k.zk_attention_plain(Q.ptr, nh * hd, KC.ptr, VC.ptr, TBL.ptr, max_blocks, REQ.ptr, POS.ptr, OUT.ptr, n,
                                 nh, nkv, hd, BS, SCALE, CAP, window, 0, rt.stream)
        got = rt.download_f32(OUT).reshape(n, nh, hd)
        assert np.isfinite(got).all()
        err = np.abs(got[rows] - want).max(axis=(1, 2))
        tol = 2e-5 if dtype == "float32" else 0.02
        assert (err < tol).all(), f"portion kernel {mode}: errors per row {dict(zip(rows, err))}"


# ------------------------------------------------------------------ a slice of the 2B model across the window
# hidden width, head size and grouping of Gemma 2 2B; a narrow feed-forward and a small
# vocabulary, which the window does not care about, keep the float64 oracle at half a minute
SLICE = dict(architectures=["Gemma2ForCausalLM"], model_type="gemma2", num_hidden_layers=2, hidden_size=2304,
             num_attention_heads=8, num_key_value_heads=4, head_dim=256, query_pre_attn_scalar=256,
             intermediate_size=2304, vocab_size=2048, rope_theta=10000.0, sliding_window=W,
             attn_logit_softcapping=50.0, final_logit_softcapping=30.0, rms_norm_eps=1e-6,
             max_position_embeddings=8192)
PROMPT, DECODED, LAST = 4090, 70, 24
# float32 against the float64 oracle at positions 4,136 to 4,159: 2.2e-4 was measured, against
# 3e-6 at the first few hundred positions.  All of it is the rotation angle: the engine, like the
# reference (orchestrator/kernels.py:270-271), multiplies position and frequency in 32-bit, and
# at position 4,100 half a unit in the last place of the angle is 1.2e-4 rad (the frequency's own
# rounding adds as much), where the oracle's angle is exact.  Against an oracle that rounds
# frequency and angle to 32-bit and is float64 otherwise, the engine stays within the 5e-5 of
# short sequences; that is what the test asserts, beside a bound on the angles' share.
F32_ANGLE_SHARE = 1e-3


def rope_with_32_bit_angles(x, positions, theta, dt):
    """``P.rope`` with the frequency and the angle rounded to float32 before sine and cosine."""
    hd = x.shape[-1]
    half = hd // 2
    freq = (1.0 / np.power(np.float64(theta), 2.0 * np.arange(half) / hd)).astype(np.float32)
    ang = (positions.astype(np.float32)[:, None] * freq[None, :]).astype(np.float64)
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    x = x.astype(dt)
    a, b = x[..., :half], x[..., half:]
    return np.concatenate([a * c - b * s, b * c + a * s], axis=-1)


@pytest.fixture(scope="module")
def slice_folders(tmp_path_factory):
    """{dtype: folder}: one draw of weights (NumPy's generator: the engine's own random-weights
    function takes a minute on the host for a model of this size), stored as float32 and as
    bfloat16."""
    import json
    import os
    import zse_amd.models  # noqa: F401
    from zse_amd.config.base import resolve_architecture
    from zse_amd.engine.model import Model
    from zse_amd.parts.base import ROLE_GAIN
    from zse_amd.weights import safetensors as st
    from zse_amd.weights.loader import merge_reqs
    arch = resolve_architecture(SLICE)
    rng = np.random.default_rng(9)
    tensors = {}
    for r in merge_reqs(Model(arch.plan(arch.config_from_dict(SLICE))).tensor_reqs()).values():
        # attention weights wide enough that the softmax over 4,096 keys is far from uniform
        std = 0.1 if r.role == ROLE_GAIN else 0.03 if ("q_proj" in r.name or "k_proj" in r.name) else \
            0.01 if "embed_tokens" in r.name else 0.02
        tensors[r.name] = (rng.standard_normal(r.shape, dtype=np.float32) * np.float32(std))
    out = {}
    for dtype in ("float32", "bfloat16"):
        d = str(tmp_path_factory.mktemp(f"slice_{dtype}"))
        with open(os.path.join(d, "config.json"), "w") as f:
            json.dump(SLICE, f)
        packed = {n: ("F32", a) if dtype == "float32" else ("BF16", st.f32_to_bf16_bits(a)) for n, a in tensors.items()}
        st.write_file(os.path.join(d, "model.safetensors"), packed)
        out[dtype] = d
    return out


def run_slice(folder, dtype, toks):
    from zse_amd.engine.runner import StepEntry
    page = 16
    # the sliding layer's pool: the window, the page that is leaving it, one step's tokens and
    # the page they end in, nothing more (the engine's own rule for a single request); the
    # other layer's pool holds every key
    full = -(-len(toks) // page)
    windowed = min(-(-(W + 512) // page) + 2, full - 1)
    runner = make_runner(folder, dtype, page_size=page, num_pages=[windowed, full], max_seqs=1,
                         max_batch_tokens=512, max_model_len=8192)
    m = runner.manager
    assert [g.window for g in m.groups] == [W, None]
    at, rows, used, handed_on = 0, [], 0, 0
    seen, prev = set(), set()
    while at < len(toks):
        n = min(512, PROMPT - at) if at < PROMPT else 1
        want = [i for i in range(n) if at + i >= len(toks) - LAST]
        z = runner.step([StepEntry("a", toks[at:at + n], want)])
        rows += [r.copy() for r in z]
        at += n
        table = {p for p in m.table("a", 0) if p >= 0}
        handed_on += len((table & seen) - prev)          # held once, given back, and held again
        prev = table
        seen |= table
        used = max(used, m.pools[0].used_pages)
    assert m.table("a", 0)[0] < 0, "the window passed the first page and it is still held"
    assert handed_on > 0, "no page that the window released was used again"
    assert used <= windowed
    runner.finish("a")
    runner.close()
    return np.stack(rows)


def test_a_2b_width_slice_across_the_window(slice_folders, monkeypatch):
    from conftest import random_tokens, read_weights
    from gpu_util import F32_ATOL
    toks = random_tokens(SLICE["vocab_size"], PROMPT + DECODED, 17)
    got32 = run_slice(slice_folders["float32"], "float32", toks)
    got16 = run_slice(slice_folders["bfloat16"], "bfloat16", toks)
    assert got32.shape == got16.shape == (LAST, SLICE["vocab_size"])
    w = read_weights(slice_folders["float32"])

    def oracle(window):
        scale = np.float64(np.float32(np.sqrt(float(SLICE["hidden_size"]))))
        x = P.forward(dict(SLICE, sliding_window=window), w, toks, np.float64, embed_scale=scale,
                      return_hidden=True)[-LAST:]
        return P.softcap(x @ P.get_weight(w, "embed_tokens.weight").astype(np.float64).T,
                         SLICE["final_logit_softcapping"], np.float64)

    exact = oracle(W)
    with monkeypatch.context() as mp:
        mp.setattr(P, "rope", rope_with_32_bit_angles)
        want = oracle(W)
        # a window one key shorter moves the logits by far more than the tolerance: the comparison can fail
        off_by_one = np.abs(oracle(W - 1) - want).max()
    err, err_exact = np.abs(got32 - want).max(), np.abs(got32 - exact).max()
    print(f"float32 at positions {len(toks) - LAST} to {len(toks) - 1}: {err:.3e} against the oracle with 32-bit "
          f"angles, {err_exact:.3e} against the exact one; a window of {W - 1} keys moves the logits by {off_by_one:.3e}")
    assert err < F32_ATOL, f"float32 against the oracle with 32-bit angles: {err:.3e}"
    assert err_exact < F32_ANGLE_SHARE, f"float32 against the exact oracle: {err_exact:.3e}"
    assert off_by_one > 20 * F32_ATOL, off_by_one
    # bfloat16 against the 32-bit path (the file's weights rounded to bfloat16, the same otherwise)
    assert_close(got16, got32, "bfloat16", "bfloat16 slice against the 32-bit path")
