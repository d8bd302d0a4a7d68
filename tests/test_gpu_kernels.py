"""Each kernel alone against plain NumPy, at other sizes than the engine's tests use."""
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt():
    from zse_amd.runtime.device import Runtime
    return Runtime.get()


def bf16(x):
    from zse_amd.weights.safetensors import bf16_bits_to_f32, f32_to_bf16_bits
    return bf16_bits_to_f32(f32_to_bf16_bits(np.asarray(x, np.float32)))


def up(rt, x, dtype):
    """Host float array -> device tensor of the library's activation type."""
    from zse_amd.weights.safetensors import f32_to_bf16_bits
    x = np.ascontiguousarray(x, np.float32)
    return rt.upload(f32_to_bf16_bits(x), "bfloat16") if dtype == "bfloat16" else rt.upload(x, "float32")


def gelu(z):
    return 0.5 * z * (1 + np.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------ matrix products
GEMM_SHAPES = [(1, 1000, 96), (7, 320, 320), (8, 2304, 2048), (16, 50, 64), (33, 1000, 328),
               (64, 513, 1024), (65, 300, 96), (200, 1000, 320), (300, 257, 2304), (128, 128, 64)]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gemm_plain(rt, dtype, M, N, K):
    k = rt.kernels(dtype)
    rng = np.random.default_rng(M * 1000 + N)
    a, w = rng.normal(size=(M, K)), rng.normal(size=(N, K))
    if dtype == "bfloat16":
        a, w = bf16(a), bf16(w)
    A, W = up(rt, a, dtype), up(rt, w, dtype)
    C = rt.empty((M, N), "float32")
    k.zk_gemm_plain(A.ptr, K, W.ptr, C.ptr, N, 1, M, N, K, rt.stream)
    want = a.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(rt.download(C) - want).max() < 1e-4 * math.sqrt(K)


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_bf16_matrix_cores(rt, M, N, K):
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(M * 1000 + N + 1)
    a, w = bf16(rng.normal(size=(M, K))), bf16(rng.normal(size=(N, K)))
    A, W = up(rt, a, "bfloat16"), up(rt, w, "bfloat16")
    want = a.astype(np.float64) @ w.astype(np.float64).T
    C = rt.empty((M, N), "float32")
    k.zk_gemm_bf16(A.ptr, K, W.ptr, C.ptr, N, 1, M, N, K, 0, 0.0, rt.stream)
    assert np.abs(rt.download(C) - want).max() < 1e-4 * math.sqrt(K)      # float accumulation
    Cb = rt.empty((M, N), "bfloat16")
    k.zk_gemm_bf16(A.ptr, K, W.ptr, Cb.ptr, N, 0, M, N, K, 0, 0.0, rt.stream)
    got = rt.download_f32(Cb)
    assert np.abs(got - want).max() <= np.abs(want).max() * 2.0 ** -8 + 1e-4 * math.sqrt(K)
    k.zk_gemm_bf16(A.ptr, K, W.ptr, C.ptr, N, 1, M, N, K, 1, 7.5, rt.stream)
    assert np.abs(rt.download(C) - 7.5 * np.tanh(want / 7.5)).max() < 1e-4 * math.sqrt(K)


@pytest.mark.parametrize("M,I,K,act", [(1, 320, 96, "gelu_tanh"), (8, 1000, 64, "silu"), (40, 176, 320, "gelu_tanh"),
                                       (130, 330, 96, "gelu_tanh"), (257, 64, 128, "silu")])
def test_gemm_bf16_gated_epilogue(rt, M, I, K, act):
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(M + I)
    a, w = bf16(rng.normal(size=(M, K))), bf16(rng.normal(size=(2 * I, K)) * 0.3)
    A, W = up(rt, a, "bfloat16"), up(rt, w, "bfloat16")
    C = rt.empty((M, I), "float32")
    k.zk_gemm_bf16(A.ptr, K, W.ptr, C.ptr, I, 1, M, I, K, 2 if act == "gelu_tanh" else 3, 0.0, rt.stream)
    g = a.astype(np.float64) @ w[:I].astype(np.float64).T
    u = a.astype(np.float64) @ w[I:].astype(np.float64).T
    want = (gelu(g) if act == "gelu_tanh" else g / (1 + np.exp(-g))) * u
    assert np.abs(rt.download(C) - want).max() < 2e-4 * math.sqrt(K) * max(1.0, np.abs(u).max())


def test_gemm_reference_vector(rt):
    # ones times 0.5 gives K * 0.5 (reference tests/test_modal_orchestrator.py:271-302)
    for dtype in ("float32", "bfloat16"):
        k = rt.kernels(dtype)
        A, W = up(rt, np.ones((4, 64)), dtype), up(rt, np.full((8, 64), 0.5), dtype)
        C = rt.empty((4, 8), "float32")
        k.zk_gemm_plain(A.ptr, 64, W.ptr, C.ptr, 8, 1, 4, 8, 64, rt.stream)
        assert np.all(rt.download(C) == 32.0)


def test_gemm_refuses_what_it_cannot_do(rt):
    from zse_amd.runtime.device import DeviceError
    k = rt.kernels("bfloat16")
    A, W, C = rt.empty((4, 100), "bfloat16"), rt.empty((8, 100), "bfloat16"), rt.empty((4, 8), "float32")
    with pytest.raises(DeviceError, match="multiples of 8"):
        k.zk_gemm_bf16(A.ptr, 100, W.ptr, C.ptr, 8, 1, 4, 8, 100, 0, 0.0, rt.stream)


# ------------------------------------------------------------------ attention over the cache
def np_attention(q, k, v, pos_q, scale, cap, window):
    """q [n, nh, hd] at positions pos_q over keys/values [ctx, nkv, hd] (float64)."""
    n, nh, hd = q.shape
    g = nh // k.shape[1]
    out = np.zeros((n, nh, hd))
    for i in range(n):
        lo = max(0, pos_q[i] - window + 1) if window else 0
        for h in range(nh):
            s = (k[lo:pos_q[i] + 1, h // g] @ q[i, h]) * scale
            if cap:
                s = cap * np.tanh(s / cap)
            p = np.exp(s - s.max())
            out[i, h] = (p / p.sum()) @ v[lo:pos_q[i] + 1, h // g]
    return out


def paged(rt, dtype, kv, bs, pages, transposed, rng):
    """Scatter [ctx, nkv, hd] into a pool of pages in a random order; returns (tensor, table)."""
    ctx, nkv, hd = kv.shape
    nblk = -(-ctx // bs)
    ids = rng.permutation(pages)[:nblk]
    pool = rng.normal(size=(pages, nkv, bs, hd)).astype(np.float32)      # stale data in unused places
    for j in range(nblk):
        blk = kv[j * bs:(j + 1) * bs]
        pool[ids[j], :, :len(blk), :] = blk.transpose(1, 0, 2)
    if transposed:
        pool = np.ascontiguousarray(pool.transpose(0, 1, 3, 2))
    return up(rt, pool, dtype), ids


ATT_CASES = [
    # nh nkv hd  bs  ctxs (cached before) and new-token counts per request, window, cap
    dict(nh=4, nkv=2, hd=16, bs=4, reqs=[(0, 9), (13, 1), (30, 5)], window=8, cap=50.0),
    dict(nh=6, nkv=1, hd=32, bs=8, reqs=[(0, 40), (70, 1), (17, 1)], window=16, cap=20.0),
    dict(nh=8, nkv=4, hd=256, bs=16, reqs=[(0, 70), (300, 1), (129, 3), (511, 1)], window=0, cap=50.0),
    dict(nh=8, nkv=4, hd=256, bs=16, reqs=[(200, 45), (640, 1)], window=128, cap=0.0),
    dict(nh=32, nkv=16, hd=128, bs=32, reqs=[(5, 33), (255, 1), (256, 1)], window=100, cap=30.0),
    dict(nh=3, nkv=3, hd=64, bs=16, reqs=[(0, 2), (127, 1), (128, 2)], window=0, cap=0.0),
    dict(nh=10, nkv=2, hd=48, bs=16, reqs=[(3, 20), (60, 1)], window=24, cap=10.0),      # plain kernel only
]


@pytest.mark.parametrize("case", range(len(ATT_CASES)))
@pytest.mark.parametrize("kernel", ["plain_f32", "plain_bf16", "plain_bf16_vt", "mfma"])
def test_attention_over_pages(rt, kernel, case):
    c = ATT_CASES[case]
    dtype = "float32" if kernel == "plain_f32" else "bfloat16"
    k = rt.kernels(dtype)
    nh, nkv, hd, bs = c["nh"], c["nkv"], c["hd"], c["bs"]
    if kernel == "mfma" and not k.zk_attention_bf16_supports(nh, nkv, hd, bs):
        assert hd == 48
        pytest.skip("head_dim 48 is served by the plain kernel")
    vt = kernel in ("plain_bf16_vt", "mfma")
    rng = np.random.default_rng(case)
    reqs = sorted(c["reqs"], key=lambda x: x[1] == 1)              # several tokens first
    R = len(reqs)
    total = [a + b for a, b in reqs]
    pages = sum(-(-t // bs) for t in total) + 3
    max_blocks = max(-(-t // bs) for t in total) + 2
    scale = 0.31
    q_rows, tok_pos, tok_req, table = [], [], [], np.full((R, max_blocks), -1, np.int32)
    want = []
    kc = np.zeros((pages, nkv, bs, hd), np.float32)
    vc = np.zeros((pages, nkv, hd, bs) if vt else (pages, nkv, bs, hd), np.float32)
    free = list(rng.permutation(pages))
    for r, (past, n) in enumerate(reqs):
        ctx = past + n
        kk, vv = rng.normal(size=(ctx, nkv, hd)), rng.normal(size=(ctx, nkv, hd))
        qq = rng.normal(size=(n, nh, hd))
        # one far key stands out for the last query of the request
        far = max(0, ctx - 1 - (c["window"] - 1 if c["window"] else ctx - 1))
        kk[far, :, :] = 0
        kk[far, :, 0] = 6.0
        qq[-1, :, 0] = 6.0
        if dtype == "bfloat16":
            kk, vv, qq = bf16(kk).astype(np.float64), bf16(vv).astype(np.float64), bf16(qq).astype(np.float64)
        pos = np.arange(past, ctx)
        want.append(np_attention(qq, kk, vv, pos, scale, c["cap"], c["window"]))
        for j in range(-(-ctx // bs)):
            pg = free.pop()
            table[r, j] = pg
            blk_k, blk_v = kk[j * bs:(j + 1) * bs], vv[j * bs:(j + 1) * bs]
            kc[pg, :, :len(blk_k)] = blk_k.transpose(1, 0, 2)
            if vt:
                vc[pg, :, :, :len(blk_v)] = blk_v.transpose(1, 2, 0)
            else:
                vc[pg, :, :len(blk_v)] = blk_v.transpose(1, 0, 2)
        q_rows.append(qq.reshape(n, nh * hd))
        tok_pos += list(pos)
        tok_req += [r] * n
    want = np.concatenate(want)
    T = len(tok_pos)
    q = np.concatenate(q_rows)
    Q, KC, VC = up(rt, q, dtype), up(rt, kc, dtype), up(rt, vc, dtype)
    TBL = rt.upload(table)
    POS, REQ = rt.upload(np.array(tok_pos, np.int32)), rt.upload(np.array(tok_req, np.int32))
    qs = np.concatenate([[0], np.cumsum([n for _, n in reqs])]).astype(np.int32)
    QS, CL = rt.upload(qs), rt.upload(np.array(total, np.int32))
    OUT = rt.zeros((T, nh * hd), dtype)
    if kernel == "mfma":
        n_multi = sum(1 for _, n in reqs if n > 1)
        ws = rt.zeros((max(1, k.zk_attention_bf16_workspace(R, nh, hd, max(total)) // 4),), "float32")
        k.zk_attention_bf16(Q.ptr, nh * hd, KC.ptr, VC.ptr, TBL.ptr, max_blocks, QS.ptr, CL.ptr, OUT.ptr,
                            R, n_multi, max(n for _, n in reqs), max(total), nh, nkv, hd, bs, scale,
                            c["cap"], c["window"], ws.ptr, ws.nbytes, rt.stream)
    else:
        k.zk_attention_plain(Q.ptr, nh * hd, KC.ptr, VC.ptr, TBL.ptr, max_blocks, REQ.ptr, POS.ptr, OUT.ptr,
                             T, nh, nkv, hd, bs, scale, c["cap"], c["window"], 1 if vt else 0, rt.stream)
    got = rt.download_f32(OUT).reshape(T, nh, hd)
    tol = 2e-5 if dtype == "float32" else 0.02
    err = np.abs(got - want)
    assert err.max() < tol, f"max error {err.max()} at token {np.unravel_index(err.argmax(), err.shape)}"
