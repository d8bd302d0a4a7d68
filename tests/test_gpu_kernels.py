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


_ALIVE = []


@pytest.fixture(autouse=True)
def _drop_device_tensors():
    yield
    _ALIVE.clear()


_GEMM_WS = {}


def gemm_workspace(rt):
    """One workspace for the split products, as the engine keeps one."""
    if "ws" not in _GEMM_WS:
        _GEMM_WS["ws"] = rt.zeros((rt.kernels("bfloat16").zk_gemm_bf16_workspace() // 4,), "float32")
    return _GEMM_WS["ws"]


def ptr(t):
    """A tensor's device pointer; the tensor stays allocated until the test ends (a kernel
    that was only enqueued must not find its operand freed)."""
    _ALIVE.append(t)
    return t.ptr


def gelu(z):
    return 0.5 * z * (1 + np.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------ matrix products
GEMM_SHAPES = [(1, 1000, 96), (7, 320, 320), (8, 2304, 2048), (16, 50, 64), (33, 1000, 328),
               (64, 513, 1024), (65, 300, 96), (200, 1000, 320), (300, 257, 2304), (128, 128, 64),
               (100, 200, 2048), (70, 90, 4168)]      # few tiles and a long K: split over blocks


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
    k.zk_gemm_bf16(A.ptr, K, W.ptr, C.ptr, N, 1, M, N, K, 0, 0.0, 0, None, 0, None, rt.stream)
    assert np.abs(rt.download(C) - want).max() < 1e-4 * math.sqrt(K)      # float accumulation
    ws = gemm_workspace(rt)      # with a workspace a long K is split over blocks and joined
    C2 = rt.empty((M, N), "float32")
    k.zk_gemm_bf16(A.ptr, K, W.ptr, C2.ptr, N, 1, M, N, K, 0, 0.0, 0, ws.ptr, ws.nbytes, None, rt.stream)
    assert np.abs(rt.download(C2) - want).max() < 1e-4 * math.sqrt(K)
    Cb = rt.empty((M, N), "bfloat16")
    k.zk_gemm_bf16(A.ptr, K, W.ptr, Cb.ptr, N, 0, M, N, K, 0, 0.0, 0, None, 0, None, rt.stream)
    got = rt.download_f32(Cb)
    assert np.abs(got - want).max() <= np.abs(want).max() * 2.0 ** -8 + 1e-4 * math.sqrt(K)
    k.zk_gemm_bf16(A.ptr, K, W.ptr, C.ptr, N, 1, M, N, K, 1, 7.5, 0, None, 0, None, rt.stream)
    assert np.abs(rt.download(C) - 7.5 * np.tanh(want / 7.5)).max() < 1e-4 * math.sqrt(K)


@pytest.mark.parametrize("M,I,K,act", [(1, 320, 96, "gelu_tanh"), (8, 1000, 64, "silu"), (40, 176, 320, "gelu_tanh"),
                                       (130, 330, 96, "gelu_tanh"), (257, 64, 128, "silu")])
def test_gemm_bf16_gated_epilogue(rt, M, I, K, act):
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(M + I)
    a, w = bf16(rng.normal(size=(M, K))), bf16(rng.normal(size=(2 * I, K)) * 0.3)
    A, W = up(rt, a, "bfloat16"), up(rt, w, "bfloat16")
    C = rt.empty((M, I), "float32")
    k.zk_gemm_bf16(A.ptr, K, W.ptr, C.ptr, I, 1, M, I, K, 2 if act == "gelu_tanh" else 3, 0.0, 0, None, 0, None, rt.stream)
    g = a.astype(np.float64) @ w[:I].astype(np.float64).T
    u = a.astype(np.float64) @ w[I:].astype(np.float64).T
    want = (gelu(g) if act == "gelu_tanh" else g / (1 + np.exp(-g))) * u
    assert np.abs(rt.download(C) - want).max() < 2e-4 * math.sqrt(K) * max(1.0, np.abs(u).max())


@pytest.mark.parametrize("M,N,K,gated", [(1, 1000, 96, False), (8, 2304, 2048, False), (40, 50, 64, False),
                                          (64, 333, 320, False), (200, 1000, 320, False), (300, 257, 2304, False),
                                          (3, 176, 64, True), (16, 320, 96, True), (130, 336, 128, True),
                                          # 17..64 rows: activations shared in LDS, one to eight k chunks
                                          (17, 100, 64, False), (33, 2304, 2048, False), (48, 333, 544, False),
                                          (64, 1000, 512, False), (50, 72, 800, False), (20, 176, 288, True),
                                          (64, 320, 800, True), (40, 336, 256, True), (33, 48, 1056, True),
                                          # over 64 rows, few tiles, long K: k ranges over blocks, then a join
                                          (100, 200, 2048, False), (130, 336, 2048, True), (70, 90, 4128, False),
                                          (512, 2304, 9216, False),
                                          # 17..64 rows, more than 512 strips: three strips a block
                                          # (the last block not full, the last strip not whole)
                                          (40, 8224, 288, True), (64, 9216, 2304, True), (24, 8200, 320, False)])
def test_gemm_bf16_strip_layout(rt, M, N, K, gated):
    """The same products with the weights rearranged into strips of 16 rows by 32 columns, and
    an embedding gather out of that layout."""
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(M + N + K)
    rows = 2 * N if gated else N
    a, w = bf16(rng.normal(size=(M, K))), bf16(rng.normal(size=(rows, K)) * (0.3 if gated else 1.0))
    A, W = up(rt, a, "bfloat16"), up(rt, w, "bfloat16")
    WS = rt.empty(((rows + 15) // 16 * 16, K), "bfloat16")
    k.zk_strip_layout(W.ptr, WS.ptr, rows, K, rt.stream)
    C = rt.empty((M, N), "float32")
    ws = gemm_workspace(rt)
    if gated:
        k.zk_gemm_bf16(A.ptr, K, WS.ptr, C.ptr, N, 1, M, N, K, 2, 0.0, 1, ws.ptr, ws.nbytes, None, rt.stream)
        g = a.astype(np.float64) @ w[:N].astype(np.float64).T
        want = gelu(g) * (a.astype(np.float64) @ w[N:].astype(np.float64).T)
        tol = 2e-4 * math.sqrt(K) * max(1.0, np.abs(want).max())
    else:
        k.zk_gemm_bf16(A.ptr, K, WS.ptr, C.ptr, N, 1, M, N, K, 0, 0.0, 1, ws.ptr, ws.nbytes, None, rt.stream)
        want = a.astype(np.float64) @ w.astype(np.float64).T
        tol = 1e-4 * math.sqrt(K)
    got = rt.download(C)
    assert np.abs(got - want).max() < tol
    # a second launch, over the first one's leavings in the workspace, gives the same bits
    k.zk_gemm_bf16(A.ptr, K, WS.ptr, C.ptr, N, 1, M, N, K, 2 if gated else 0, 0.0, 1, ws.ptr, ws.nbytes, None, rt.stream)
    assert np.array_equal(rt.download(C), got)
    if 16 < M <= 64:   # without a workspace K is not split over blocks: same values beyond rounding
        k.zk_gemm_bf16(A.ptr, K, WS.ptr, C.ptr, N, 1, M, N, K, 2 if gated else 0, 0.0, 1, None, 0, None, rt.stream)
        assert np.abs(rt.download(C) - want).max() < tol
    if not gated and K % 32 == 0:
        toks = rng.integers(0, N, 5).astype(np.int32)
        toks[0] = N - 1
        out = rt.empty((5, K), "float32")
        k.zk_embed(WS.ptr, ptr(rt.upload(toks)), out.ptr, 2.0, 5, K, N, 1, rt.stream)
        assert np.array_equal(rt.download(out), w[toks] * np.float32(2.0))


@pytest.mark.parametrize("N,K,gated", [(2304, 9216, False), (4096, 2304, False), (9216, 2304, True), (4608, 4096, False)])
def test_gemm_bf16_layer_shapes_at_medium_rows(rt, N, K, gated):
    """Layer-size products with a hundred to a thousand rows, where the dispatch picks among four
    tile sizes and up to eight ranges of K by a model of their times: whatever it picks agrees
    with the plain product of the same library (same 16-bit inputs, float sums)."""
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(N + K)
    rows = 2 * N if gated else N
    w = bf16(rng.normal(size=(rows, K)) * (0.02 if gated else 0.05))
    W = up(rt, w, "bfloat16")
    WS = rt.empty((rows, K), "bfloat16")
    k.zk_strip_layout(W.ptr, WS.ptr, rows, K, rt.stream)
    ws = gemm_workspace(rt)
    # 4096 rows into N = 2304: 144 tiles of 256 x 256... or 288 of 128 x 256, a round of the CUs
    # and a tail of 32 tiles, which is launched apart with K in ranges
    for M in (96, 200, 384, 520, 1000) + ((4096,) if (N, K) == (2304, 9216) else ()):
        a = bf16(rng.normal(size=(M, K)))
        A = up(rt, a, "bfloat16")
        C, R = rt.empty((M, N), "float32"), rt.empty((M, rows), "float32")
        k.zk_gemm_bf16(A.ptr, K, WS.ptr, C.ptr, N, 1, M, N, K, 2 if gated else 0, 0.0, 1, ws.ptr, ws.nbytes,
                       None, rt.stream)
        k.zk_gemm_plain(A.ptr, K, W.ptr, R.ptr, rows, 1, M, rows, K, rt.stream)
        got, ref = rt.download(C), rt.download(R).astype(np.float64)
        want = gelu(ref[:, :N]) * ref[:, N:] if gated else ref
        tol = 2e-5 * math.sqrt(K) * max(1.0, np.abs(want).max())
        err = np.abs(got - want).max()
        assert err < tol, f"M={M}: {err} against {tol}"


@pytest.mark.parametrize("M,N,K,gated,cap", [(2048, 2304, 2048, False, 0.0), (1500, 8208, 2304, False, 0.0),
                                              (4000, 9216, 2304, True, 0.0), (700, 14336, 3584, True, 0.0),
                                              (2048, 4096, 2304, False, 30.0), (1027, 2320, 9216, False, 0.0),
                                              (3000, 1168, 2304, True, 0.0),
                                              # K of one and of two k tiles: fewer stages than LDS holds
                                              (2500, 2304, 64, False, 0.0), (2100, 1024, 128, True, 0.0)])
def test_gemm_bf16_wide_blocks_with_strip_weights(rt, M, N, K, gated, cap):
    """Thousands of rows against strip-layout weights with K a whole number of 64: the 128 x 256
    and 256 x 256 blocks that copy their operands straight into LDS.  Row counts that end inside
    a block, widths that end inside a block's columns (2320, 8208, gated 1168), a soft cap, K in
    ranges with a join (1027 x 2320 x 9216), into a 16-bit C (whole blocks leave through LDS)
    and into a 32-bit one, against the plain product of the same 16-bit inputs."""
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(M + N + K)
    rows = 2 * N if gated else N
    a, w = bf16(rng.normal(size=(M, K))), bf16(rng.normal(size=(rows, K)) * (0.02 if gated else 0.05))
    A, W = up(rt, a, "bfloat16"), up(rt, w, "bfloat16")
    WS = rt.empty(((rows + 15) // 16 * 16, K), "bfloat16")
    k.zk_strip_layout(W.ptr, WS.ptr, rows, K, rt.stream)
    ws = gemm_workspace(rt)
    R = rt.empty((M, rows), "float32")
    k.zk_gemm_plain(A.ptr, K, W.ptr, R.ptr, rows, 1, M, rows, K, rt.stream)
    ref = rt.download(R).astype(np.float64)
    want = gelu(ref[:, :N]) * ref[:, N:] if gated else (cap * np.tanh(ref / cap) if cap else ref)
    epi = 2 if gated else (1 if cap else 0)
    C32, C16 = rt.empty((M, N), "float32"), rt.empty((M, N), "bfloat16")
    k.zk_gemm_bf16(A.ptr, K, WS.ptr, C32.ptr, N, 1, M, N, K, epi, cap, 1, ws.ptr, ws.nbytes, None, rt.stream)
    k.zk_gemm_bf16(A.ptr, K, WS.ptr, C16.ptr, N, 0, M, N, K, epi, cap, 1, ws.ptr, ws.nbytes, None, rt.stream)
    got32, got16 = rt.download(C32), rt.download_f32(C16)
    tol = 2e-5 * math.sqrt(K) * max(1.0, np.abs(want).max())
    assert np.abs(got32 - want).max() < tol
    # the 16-bit C holds the 32-bit one's values, rounded once
    assert np.array_equal(got16, bf16(got32))


def test_gemm_bf16_random_shapes(rt):
    """Forty shapes drawn at random over the three kernels' ranges, both weight layouts, with
    and without the gated epilogue and the workspace: whatever the dispatch picks must agree
    with the product in float64."""
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(2024)
    ws = gemm_workspace(rt)
    for case in range(40):
        M = int(rng.choice([rng.integers(1, 17), rng.integers(17, 65), rng.integers(65, 400)]))
        strip = bool(rng.integers(0, 2))
        gated = bool(rng.integers(0, 2))
        K = int(rng.integers(1, 140)) * (32 if strip else 8)
        N = int(rng.integers(1, 45)) * 16 if (gated and strip) else int(rng.integers(1, 700))
        rows = 2 * N if gated else N
        a, w = bf16(rng.normal(size=(M, K))), bf16(rng.normal(size=(rows, K)) * (0.3 if gated else 1.0))
        A, W = up(rt, a, "bfloat16"), up(rt, w, "bfloat16")
        if strip:
            WS = rt.empty(((rows + 15) // 16 * 16, K), "bfloat16")
            k.zk_strip_layout(W.ptr, WS.ptr, rows, K, rt.stream)
            W = WS
        C = rt.empty((M, N), "float32")
        use_ws = bool(rng.integers(0, 2))
        k.zk_gemm_bf16(A.ptr, K, W.ptr, C.ptr, N, 1, M, N, K, 2 if gated else 0, 0.0, 1 if strip else 0,
                       ws.ptr if use_ws else None, ws.nbytes if use_ws else 0, None, rt.stream)
        if gated:
            g = a.astype(np.float64) @ w[:N].astype(np.float64).T
            want = gelu(g) * (a.astype(np.float64) @ w[N:].astype(np.float64).T)
            tol = 2e-4 * math.sqrt(K) * max(1.0, np.abs(want).max())
        else:
            want = a.astype(np.float64) @ w.astype(np.float64).T
            tol = 1e-4 * math.sqrt(K)
        err = np.abs(rt.download(C) - want).max()
        assert err < tol, f"case {case}: M={M} N={N} K={K} strip={strip} gated={gated} workspace={use_ws}: {err}"


@pytest.mark.parametrize("M,N,K", [(8, 2304, 2048), (1, 2304, 9216), (16, 1024, 4096), (40, 2304, 9216), (64, 4096, 2304),
                                   (17, 1536, 1024),
                                   # up to 16 rows and more strips than CUs, unevenly spread: K in ranges
                                   (8, 4608, 36864), (1, 4608, 4096), (16, 5120, 2048)])
def test_gemm_bf16_leaves_partial_sums_to_a_reader_that_asks(rt, M, N, K):
    """A caller that passes a place for the number of parts gets the split product's partial
    sums as planes of [M, N] floats; added in order and rounded they are the bits the product
    stores when it joins them itself.  A product that does not split K says 0 and fills C."""
    import ctypes
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(M + N)
    a = bf16(rng.normal(size=(M, K)).astype(np.float32))
    w = bf16(rng.normal(size=(N, K)).astype(np.float32) / math.sqrt(K))
    A, W = up(rt, a, "bfloat16"), up(rt, w, "bfloat16")
    WS = rt.empty((N, K), "bfloat16")
    k.zk_strip_layout(W.ptr, WS.ptr, N, K, rt.stream)
    ws = gemm_workspace(rt)
    C = rt.zeros((M, N), "bfloat16")
    k.zk_gemm_bf16(A.ptr, K, WS.ptr, C.ptr, N, 0, M, N, K, 0, 0.0, 1, ws.ptr, ws.nbytes, None, rt.stream)
    joined = rt.download_f32(C)
    want = a.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(joined - want).max() <= 2.0 ** -7 * max(1.0, np.abs(want).max())
    C2 = rt.zeros((M, N), "bfloat16")
    parts = ctypes.c_int(-1)
    k.zk_gemm_bf16(A.ptr, K, WS.ptr, C2.ptr, N, 0, M, N, K, 0, 0.0, 1, ws.ptr, ws.nbytes, ctypes.byref(parts), rt.stream)
    P = parts.value
    assert P >= 0
    if M <= 16 and N > 4096:
        assert P >= 2          # 288 and 320 strips over 256 CUs
    if P == 0:
        assert np.array_equal(rt.download_f32(C2), joined)
        return
    planes = rt.download(ws)[:P * M * N].reshape(P, M, N)
    total = planes[0].copy()
    for p in range(1, P):
        total = total + planes[p]
    if M > 16:
        assert np.array_equal(bf16(total), joined)             # the same split either way
    else:
        assert np.abs(bf16(total) - want).max() <= 2.0 ** -7 * max(1.0, np.abs(want).max())
    assert not rt.download_f32(C2).any()                       # C was left alone
    # a float result, an epilogue or rows longer than N are joined by the product itself
    C3 = rt.zeros((M, N), "float32")
    k.zk_gemm_bf16(A.ptr, K, WS.ptr, C3.ptr, N, 1, M, N, K, 0, 0.0, 1, ws.ptr, ws.nbytes, ctypes.byref(parts), rt.stream)
    assert parts.value == 0 and np.abs(rt.download(C3) - want).max() <= 1e-3 * max(1.0, np.abs(want).max())


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
        k.zk_gemm_bf16(A.ptr, 100, W.ptr, C.ptr, 8, 1, 4, 8, 100, 0, 0.0, 0, None, 0, None, rt.stream)


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
    # many decoded tokens over long contexts: 64 keys a wave (fewer waves: 32)
    dict(nh=8, nkv=4, hd=64, bs=16, reqs=[(1500, 1), (1499, 1), (1000, 1), (1343, 1), (1279, 1), (1280, 1)],
         window=0, cap=50.0),
    # a portion whose row groups number 280: two groups a block (144 blocks run at once)
    dict(nh=8, nkv=8, hd=16, bs=16, reqs=[(20, 1100)], window=300, cap=20.0),
    dict(nh=10, nkv=2, hd=48, bs=16, reqs=[(3, 20), (60, 1)], window=24, cap=10.0),      # plain kernel only
    # portions whose blocks number a multiple of 8: the blocks of a KV head are dealt to 8 / nkv
    # XCDs (4, 2 and 1 KV heads), two requests in one launch
    dict(nh=8, nkv=4, hd=64, bs=16, reqs=[(37, 128), (0, 100)], window=0, cap=50.0),
    dict(nh=4, nkv=2, hd=32, bs=16, reqs=[(11, 64), (70, 50)], window=40, cap=0.0),
    dict(nh=2, nkv=1, hd=128, bs=16, reqs=[(5, 256)], window=0, cap=30.0),
    # decoded tokens whose window is much shorter than the context the step allows: the grid
    # covers a window's blocks and counts them from the one each request's window begins in;
    # the far key that stands out is the window's first, at, before and after a block's edge
    dict(nh=8, nkv=4, hd=64, bs=16, reqs=[(254, 1), (255, 1), (298, 1), (299, 1), (554, 1), (555, 1), (810, 1),
                                          (811, 1), (1499, 1), (39, 1)], window=300, cap=50.0),
    dict(nh=4, nkv=2, hd=256, bs=16, reqs=[(1100, 1), (767, 1), (768, 1), (5, 1)], window=513, cap=0.0),
    # long portions (tiles shared by the groups of a block): a portion that starts inside a page
    # and ends inside a tile, a window that begins inside a tile, pages of 8, 16, 32 and 64 keys,
    # one, two, three and eight heads a KV head, a second request of another length in the launch
    dict(nh=8, nkv=4, hd=256, bs=16, reqs=[(37, 300), (5, 70)], window=0, cap=50.0, ranges_by_size=True),
    dict(nh=8, nkv=4, hd=128, bs=8, reqs=[(100, 333)], window=150, cap=30.0),
    dict(nh=6, nkv=2, hd=64, bs=32, reqs=[(3, 260), (200, 45)], window=0, cap=0.0),
    dict(nh=3, nkv=3, hd=32, bs=64, reqs=[(60, 500)], window=97, cap=20.0),
    dict(nh=16, nkv=2, hd=16, bs=16, reqs=[(11, 190)], window=0, cap=50.0),
    # so many groups (66 of 32 rows x 16 KV heads) that the choice by size takes the shared tiles
    dict(nh=16, nkv=16, hd=16, bs=16, reqs=[(20, 2100)], window=700, cap=20.0),
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
    tol = 2e-5 if dtype == "float32" else 0.02
    outs = []
    # both cuts of the decoded tokens' keys; and every kernel for the portions: a group of rows a
    # block (1), tiles shared by 4 or 8 groups (pages of 8 keys or more), shared tiles with the keys
    # in ranges and a join (5; long contexts, else as 4), the choice by size (0)
    turns = [(0, 0)]
    if kernel == "mfma":
        turns = [(64, 0), (32, 0), (64, 1)] + ([(64, 4), (32, 8), (64, 5)] if bs >= 8 else [])
    for chunk, portion_kernel in turns:
        OUT = rt.zeros((T, nh * hd), dtype)
        if kernel == "mfma":
            k.zk_attention_bf16_portion_kernel(portion_kernel)
            n_multi = sum(1 for _, n in reqs if n > 1)
            # more context allowed than any request has, as in a captured step: more chunks than keys
            max_ctx = max(total) + 200
            ws_bytes = (k.zk_attention_bf16_workspace(R, nh, hd, max_ctx) + 255) // 256 * 256
            ws_bytes += k.zk_attention_bf16_portion_workspace(max(1, n_multi) * (max(n for _, n in reqs) + 128), nh, nkv, hd)
            ws = rt.zeros((ws_bytes // 4 + 1,), "float32")
            try:
                k.zk_attention_bf16(Q.ptr, nh * hd, KC.ptr, VC.ptr, TBL.ptr, max_blocks, QS.ptr, CL.ptr, OUT.ptr,
                                    R, n_multi, max(n for _, n in reqs), max_ctx, nh, nkv, hd, bs, scale,
                                    c["cap"], c["window"], chunk, ws.ptr, ws.nbytes, rt.stream)
            finally:
                k.zk_attention_bf16_portion_kernel(0)
        else:
            k.zk_attention_plain(Q.ptr, nh * hd, KC.ptr, VC.ptr, TBL.ptr, max_blocks, REQ.ptr, POS.ptr, OUT.ptr,
                                 T, nh, nkv, hd, bs, scale, c["cap"], c["window"], 1 if vt else 0, rt.stream)
        got = rt.download_f32(OUT).reshape(T, nh, hd)
        err = np.abs(got - want)
        assert err.max() < tol, (f"chunk {chunk}, portion kernel {portion_kernel}: max error {err.max()} at token "
                                 f"{np.unravel_index(err.argmax(), err.shape)}")
        outs.append(got)
    if kernel == "mfma" and c.get("ranges_by_size"):
        # few blocks of rows, 17 tiles of keys: the choice by size cuts the keys into ranges
        assert np.array_equal(outs[0], outs[turns.index((64, 5))]) and not np.array_equal(outs[0], outs[turns.index((64, 4))])


@pytest.mark.parametrize("seed", range(24))
def test_portion_attention_kernels_agree_on_random_launches(rt, seed):
    """Random launches (one to three portions of 2 to 700 rows behind 0 to 1,500 tokens, up to two
    decoded tokens beside them, 1 to 16 heads a KV head, windows, caps, pages of 8 to 64 keys,
    pages in random order): the kernels with shared tiles (four waves, eight, with the keys in
    ranges, and the choice by size) against the kernel of one group a block, which the cases above
    hold against NumPy."""
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(1000 + seed)
    nkv, g = int(rng.choice([1, 2, 3, 4, 8])), int(rng.choice([1, 2, 3, 4, 5, 8, 16]))
    nh, hd, bs = nkv * g, int(rng.choice([16, 32, 64, 128, 256])), int(rng.choice([8, 16, 32, 64]))
    reqs = [(int(rng.integers(0, 1500)), int(rng.integers(2, 700))) for _ in range(int(rng.integers(1, 4)))]
    n_multi = len(reqs)
    reqs += [(int(rng.integers(1, 1200)), 1) for _ in range(int(rng.integers(0, 3)))]
    window, cap = int(rng.choice([0, 0, 40, 300, 1000])), float(rng.choice([0.0, 30.0, 50.0]))
    total = [a + b for a, b in reqs]
    max_blocks = max(-(-t // bs) for t in total) + 1
    pages = sum(-(-t // bs) for t in total) + 2
    KC, VC = rt.empty((pages, nkv, bs, hd), "bfloat16"), rt.empty((pages, nkv, hd, bs), "bfloat16")
    k.zk_fill_normal(KC.ptr, 1, KC.numel, 1, 3 * seed + 1, 0.0, 1.0, rt.stream)
    k.zk_fill_normal(VC.ptr, 1, VC.numel, 1, 3 * seed + 2, 0.0, 1.0, rt.stream)
    table, free = np.full((len(reqs), max_blocks), -1, np.int32), list(rng.permutation(pages))
    for r, t in enumerate(total):
        for j in range(-(-t // bs)):
            table[r, j] = free.pop()
    T = sum(n for _, n in reqs)
    qs = np.concatenate([[0], np.cumsum([n for _, n in reqs])]).astype(np.int32)
    TBL, QS, CL = rt.upload(table), rt.upload(qs), rt.upload(np.array(total, np.int32))
    Q = rt.empty((T, nh * hd), "bfloat16")
    k.zk_fill_normal(Q.ptr, 1, Q.numel, 1, 3 * seed + 3, 0.0, 1.0, rt.stream)
    max_q, max_ctx = max(n for _, n in reqs), -(-max(total) // 256) * 256
    ws_bytes = (k.zk_attention_bf16_workspace(len(reqs), nh, hd, max_ctx) + 255) // 256 * 256
    ws_bytes += k.zk_attention_bf16_portion_workspace(n_multi * (max_q + 128), nh, nkv, hd)
    ws = rt.zeros((ws_bytes // 4 + 16,), "float32")
    outs = {}
    for mode in (1, 4, 8, 5, 0):
        OUT = rt.zeros((T, nh * hd), "bfloat16")
        k.zk_attention_bf16_portion_kernel(mode)
        try:
            k.zk_attention_bf16(Q.ptr, nh * hd, KC.ptr, VC.ptr, TBL.ptr, max_blocks, QS.ptr, CL.ptr, OUT.ptr, len(reqs),
                                n_multi, max_q, max_ctx, nh, nkv, hd, bs, hd ** -0.5, cap, window, 64, ws.ptr,
                                ws.nbytes, rt.stream)
        finally:
            k.zk_attention_bf16_portion_kernel(0)
        outs[mode] = rt.download_f32(OUT)
    for mode in (4, 8, 5, 0):
        assert np.isfinite(outs[mode]).all()
        err = np.abs(outs[mode] - outs[1]).max()
        assert err <= 0.02 * max(1.0, np.abs(outs[1]).max()), f"kernel {mode}: {err}; {nh} heads, {nkv} KV heads of {hd}, {reqs}"


def run_attention(rt, kernel, q, kk, vv, past, nh, nkv, hd, bs, scale, cap, window, chunk=64, max_ctx=None):
    """One request holding ``past`` cached tokens brings the rest of ``kk``/``vv`` [ctx, nkv, hd]
    with queries ``q`` [n, nh, hd]; pages are laid out in order.  Returns [n, nh, hd]."""
    dtype = "float32" if kernel == "plain_f32" else "bfloat16"
    k = rt.kernels(dtype)
    vt = kernel == "mfma"
    ctx, n = kk.shape[0], q.shape[0]
    assert past + n == ctx
    nblk = -(-ctx // bs)
    kc = np.zeros((nblk, nkv, bs, hd), np.float32)
    vc = np.zeros((nblk, nkv, hd, bs) if vt else (nblk, nkv, bs, hd), np.float32)
    for j in range(nblk):
        bk, bv = kk[j * bs:(j + 1) * bs], vv[j * bs:(j + 1) * bs]
        kc[j, :, :len(bk)] = bk.transpose(1, 0, 2)
        if vt:
            vc[j, :, :, :len(bv)] = bv.transpose(1, 2, 0)
        else:
            vc[j, :, :len(bv)] = bv.transpose(1, 0, 2)
    Q, KC, VC = up(rt, q.reshape(n, nh * hd), dtype), up(rt, kc, dtype), up(rt, vc, dtype)
    TBL = rt.upload(np.arange(nblk, dtype=np.int32).reshape(1, nblk))
    QS, CL = rt.upload(np.array([0, n], np.int32)), rt.upload(np.array([ctx], np.int32))
    POS, REQ = rt.upload(np.arange(past, ctx, dtype=np.int32)), rt.upload(np.zeros(n, np.int32))
    OUT = rt.zeros((n, nh * hd), dtype)
    if kernel == "mfma":
        max_ctx = max_ctx or ctx
        ws = rt.zeros((max(1, k.zk_attention_bf16_workspace(1, nh, hd, max_ctx) // 4),), "float32")
        k.zk_attention_bf16(Q.ptr, nh * hd, KC.ptr, VC.ptr, TBL.ptr, nblk, QS.ptr, CL.ptr, OUT.ptr, 1,
                            1 if n > 1 else 0, n, max_ctx, nh, nkv, hd, bs, scale, cap or 0.0, window or 0,
                            chunk, ws.ptr, ws.nbytes, rt.stream)
    else:
        k.zk_attention_plain(Q.ptr, nh * hd, KC.ptr, VC.ptr, TBL.ptr, nblk, REQ.ptr, POS.ptr, OUT.ptr, n, nh,
                             nkv, hd, bs, scale, cap or 0.0, window or 0, 0, rt.stream)
    return rt.download_f32(OUT).reshape(n, nh, hd)


@pytest.mark.parametrize("kernel", ["plain_f32", "plain_bf16", "mfma"])
def test_attention_scales_then_caps_then_masks(rt, kernel):
    # q1.k0 = 1e4, q1.k1 = 0, q0.k0 = -1e4, v0 = 1, v1 = 0, scale 0.01, cap 50 (all exact in bf16):
    # right order o1 = 1.000 and o0 = 1; the cap before the scale gives o1 = 0.622; the mask
    # before the cap lets the hidden key 1 into o0 = 0.858
    from test_plain import cap_order_vectors
    q, kk, vv, scale, cap = cap_order_vectors(16)
    tol = 1e-5 if kernel == "plain_f32" else 4e-3
    # both tokens as one portion
    o = run_attention(rt, kernel, q, kk, vv, 0, 1, 1, 16, 4, scale, cap, None)
    assert abs(o[1, 0, 0] - 1.0) < tol and abs(o[0, 0, 0] - 1.0) < tol, o[:, 0, 0]
    # each as a decoded token: query 0 with key 1 lying in the cache past its context, query 1
    for chunk in (64, 32):
        o0 = run_attention(rt, kernel, q[:1], kk[:1], vv[:1], 0, 1, 1, 16, 4, scale, cap, None, chunk)
        o1 = run_attention(rt, kernel, q[1:], kk, vv, 1, 1, 1, 16, 4, scale, cap, None, chunk)
        assert abs(o0[0, 0, 0] - 1.0) < tol and abs(o1[0, 0, 0] - 1.0) < tol, (o0[0, 0, 0], o1[0, 0, 0])
    # a softer pair where the cap decides the weights: scores 10 and 9 capped at 5 are nearly a tie
    k2 = np.stack([kk[0], kk[0] * 0.9]); v2 = np.stack([vv[0], vv[1]])
    want = 1 / (1 + math.exp(5 * math.tanh(1.8) - 5 * math.tanh(2.0)))      # 0.5215; uncapped: 0.731
    o = run_attention(rt, kernel, q / 10, k2, v2, 0, 1, 1, 16, 4, scale, 5.0, None)
    assert abs(o[1, 0, 0] - want) < max(tol, 2e-3)


def test_decode_attention_at_a_large_models_limits(rt):
    """64 decoded tokens at the head geometry of the largest model (32 heads, 16 KV heads of 128)
    in a step that allows 8192 tokens of context while the requests hold few: the workspace is
    what the kernel says it needs for these limits (136 MB), and the result is the plain kernel's."""
    k = rt.kernels("bfloat16")
    nh, nkv, hd, bs, R, max_ctx = 32, 16, 128, 16, 64, 8192
    need = k.zk_attention_bf16_workspace(R, nh, hd, max_ctx)
    assert need == R * nh * (max_ctx // 64) * (hd + 2) * 4 == 136314880
    rng = np.random.default_rng(5)
    ctxs = rng.integers(1, 300, R)
    ctxs[0], ctxs[1], ctxs[2] = 1, 64, 257
    max_blocks = max_ctx // bs
    pages = int(sum(-(-c // bs) for c in ctxs)) + 1
    kc = bf16(rng.normal(size=(pages, nkv, bs, hd)))
    v = bf16(rng.normal(size=(pages, nkv, bs, hd)))
    vt = np.ascontiguousarray(v.transpose(0, 1, 3, 2))
    table = np.full((R, max_blocks), -1, np.int32)
    at = 1                                                  # page 0 belongs to nobody
    for r, c in enumerate(ctxs):
        nb = -(-int(c) // bs)
        table[r, :nb] = np.arange(at, at + nb)
        at += nb
    q = bf16(rng.normal(size=(R, nh * hd)))
    Q, KC, V, VT = up(rt, q, "bfloat16"), up(rt, kc, "bfloat16"), up(rt, v, "bfloat16"), up(rt, vt, "bfloat16")
    TBL = rt.upload(table)
    QS, CL = rt.upload(np.arange(R + 1, dtype=np.int32)), rt.upload(ctxs.astype(np.int32))
    POS, REQ = rt.upload((ctxs - 1).astype(np.int32)), rt.upload(np.arange(R, dtype=np.int32))
    want_t = rt.zeros((R, nh * hd), "bfloat16")
    k.zk_attention_plain(Q.ptr, nh * hd, KC.ptr, V.ptr, TBL.ptr, max_blocks, REQ.ptr, POS.ptr, want_t.ptr, R,
                         nh, nkv, hd, bs, 144 ** -0.5, 50.0, 0, 0, rt.stream)
    want = rt.download_f32(want_t)
    ws = rt.zeros((need // 4,), "float32")
    for chunk in (64, 32):
        out = rt.zeros((R, nh * hd), "bfloat16")
        k.zk_attention_bf16(Q.ptr, nh * hd, KC.ptr, VT.ptr, TBL.ptr, max_blocks, QS.ptr, CL.ptr, out.ptr, R, 0,
                            1, max_ctx, nh, nkv, hd, bs, 144 ** -0.5, 50.0, 0, chunk, ws.ptr, ws.nbytes, rt.stream)
        assert np.abs(rt.download_f32(out) - want).max() < 0.02
    # one byte less and the call is refused before anything is launched
    from zse_amd.runtime.device import DeviceError
    with pytest.raises(DeviceError, match="workspace too small"):
        k.zk_attention_bf16(Q.ptr, nh * hd, KC.ptr, VT.ptr, TBL.ptr, max_blocks, QS.ptr, CL.ptr, out.ptr, R, 0,
                            1, max_ctx, nh, nkv, hd, bs, 144 ** -0.5, 50.0, 0, 64, ws.ptr, ws.nbytes - 4, rt.stream)
    # a context beyond what the joining kernel can weigh is refused with its own message
    too_long = int(k.zk_attention_bf16_max_context(nh, nkv, hd, 64)) + 1
    with pytest.raises(DeviceError, match="context too long"):
        k.zk_attention_bf16(Q.ptr, nh * hd, KC.ptr, VT.ptr, TBL.ptr, max_blocks, QS.ptr, CL.ptr, out.ptr, R, 0,
                            1, too_long, nh, nkv, hd, bs, 144 ** -0.5, 50.0, 0, 64, ws.ptr, 1 << 40, rt.stream)


# ------------------------------------------------------------------ row-wise kernels
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,H,V", [(5, 96, 1000), (3, 2304, 300), (1, 70, 17)])
def test_embed(rt, dtype, T, H, V):
    k = rt.kernels(dtype)
    rng = np.random.default_rng(T + H)
    table = rng.normal(size=(V, H)).astype(np.float32)
    if dtype == "bfloat16":
        table = bf16(table)
    toks = rng.integers(0, V, T).astype(np.int32)
    toks[0] = V - 1
    out = rt.empty((T, H), "float32")
    k.zk_embed(ptr(up(rt, table, dtype)), ptr(rt.upload(toks)), out.ptr, 9.8125, T, H, V, 0, rt.stream)
    assert np.array_equal(rt.download(out), table[toks] * np.float32(9.8125))      # (ref) rows of the table


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,H,eps,uo", [(4, 96, 1e-5, 1), (3, 2304, 1e-6, 1), (2, 70, 1e-6, 0), (2, 9000, 1e-6, 1),
                                        (3, 3584, 1e-6, 1), (2, 4608, 1e-6, 1), (2, 7000, 1e-6, 0),
                                        # rows of 2,048 to 8,192 values in bfloat16: up to 64 of them
                                        # take the kernel of 1,024 threads a row, more the one of 256
                                        (8, 4096, 1e-6, 1), (64, 4608, 1e-6, 1), (65, 4608, 1e-6, 1), (5, 8192, 1e-5, 0),
                                        (7, 2048, 1e-6, 1), (3, 2044, 1e-6, 1)])
def test_rmsnorm_and_the_fused_joins(rt, dtype, T, H, eps, uo):
    k = rt.kernels(dtype)
    rng = np.random.default_rng(H)
    tol = 1e-5 if dtype == "float32" else 2.0 ** -7
    x = rng.normal(size=(T, H)).astype(np.float32) * 3
    w = rng.normal(size=H).astype(np.float32) * 0.3
    w2 = rng.normal(size=H).astype(np.float32) * 0.3
    gain = lambda v: (1 + v) if uo else v
    norm = lambda a, v: a / np.sqrt((a * a).mean(-1, keepdims=True) + eps) * gain(v)
    W, W2 = rt.upload(w), rt.upload(w2)
    out = rt.empty((T, H), dtype)
    k.zk_rmsnorm(ptr(rt.upload(x)), 1, None, W.ptr, out.ptr, eps, uo, T, H, rt.stream)
    want = norm(x.astype(np.float64), w)
    assert np.abs(rt.download_f32(out) - want).max() <= tol * np.abs(want).max()
    # rows picked by index
    rows = np.array([T - 1, 0], np.int32)
    out2 = rt.empty((2, H), dtype)
    k.zk_rmsnorm(ptr(rt.upload(x)), 1, ptr(rt.upload(rows)), W.ptr, out2.ptr, eps, uo, 2, H, rt.stream)
    assert np.abs(rt.download_f32(out2) - want[rows]).max() <= tol * np.abs(want).max()
    # (ref) all ones with unit gain come out as ones
    ones = rt.empty((1, H), dtype)
    k.zk_rmsnorm(ptr(rt.upload(np.ones((1, H), np.float32))), 1, None, ptr(rt.upload(np.zeros(H, np.float32))),
                 ones.ptr, 1e-6, 1, 1, H, rt.stream)
    assert np.abs(rt.download_f32(ones) - 1.0).max() < 1e-3
    # h += N_post(sub); out = N_next(h)
    sub = rng.normal(size=(T, H)).astype(np.float32)
    if dtype == "bfloat16":
        sub = bf16(sub)
    h = rng.normal(size=(T, H)).astype(np.float32)
    Hd = rt.upload(h)
    nxt = rt.empty((T, H), dtype)
    k.zk_norm_add_norm(ptr(up(rt, sub, dtype)), 0, W.ptr, eps, uo, Hd.ptr, W2.ptr, eps * 2, uo, nxt.ptr, T, H, rt.stream)
    h_want = h.astype(np.float64) + norm(sub.astype(np.float64), w)
    assert np.abs(rt.download(Hd) - h_want).max() < 1e-5 * max(1, np.abs(h_want).max())     # the stream stays float
    x_want = h_want / np.sqrt((h_want * h_want).mean(-1, keepdims=True) + eps * 2) * gain(w2)
    assert np.abs(rt.download_f32(nxt) - x_want).max() <= tol * np.abs(x_want).max()
    # no post norm: a plain residual sum; no next norm: nothing else is written
    Hd2 = rt.upload(h)
    k.zk_norm_add_norm(ptr(up(rt, sub, dtype)), 0, None, 0.0, 0, Hd2.ptr, None, 0.0, 0, None, T, H, rt.stream)
    assert np.abs(rt.download(Hd2) - (h.astype(np.float64) + sub)).max() < 1e-6
    # the sublayer's output as planes of partial sums (three; six or eleven for the wide rows,
    # whose kernels take them four or eight a turn): the same bits as their sum in plane order, rounded to the
    # activation type, gives when handed over as one tensor
    P = 3 if H < 3000 else (11 if H == 4608 else 6)        # eleven: a second turn of eight
    planes = rng.normal(size=(P, T, H)).astype(np.float32)
    total = planes[0]
    for q in range(1, P):
        total = total + planes[q]
    if dtype == "bfloat16":
        total = bf16(total)
    got = []
    for src, parts in ((up(rt, total, dtype), 0), (rt.upload(planes), P)):
        Hd3, nxt3 = rt.upload(h), rt.empty((T, H), dtype)
        k.zk_norm_add_norm(src.ptr, parts, W.ptr, eps, uo, Hd3.ptr, W2.ptr, eps * 2, uo, nxt3.ptr, T, H, rt.stream)
        got.append((rt.download(Hd3), rt.download_f32(nxt3)))
    assert np.array_equal(got[0][0], got[1][0]) and np.array_equal(got[0][1], got[1][1])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gated_activation_and_softcap(rt, dtype):
    k = rt.kernels(dtype)
    rng = np.random.default_rng(3)
    T, I = 3, 330
    gu = rng.normal(size=(T, 2 * I)).astype(np.float32) * 2
    if dtype == "bfloat16":
        gu = bf16(gu)
    g, u = gu[:, :I].astype(np.float64), gu[:, I:].astype(np.float64)
    tol = 1e-5 if dtype == "float32" else 2.0 ** -7
    for act, want in ((0, gelu(g) * u), (1, g / (1 + np.exp(-g)) * u)):
        out = rt.empty((T, I), dtype)
        k.zk_gated_act(ptr(up(rt, gu, dtype)), out.ptr, T, I, act, rt.stream)
        assert np.abs(rt.download_f32(out) - want).max() <= tol * max(1, np.abs(want).max())
    z = (rng.normal(size=1001) * 40).astype(np.float32)
    Z = rt.upload(z)
    k.zk_softcap(Z.ptr, 1001, 30.0, rt.stream)
    assert np.abs(rt.download(Z) - 30 * np.tanh(z.astype(np.float64) / 30)).max() < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T", [27, 75])          # a block per (token, head); from 64 tokens a block per token
@pytest.mark.parametrize("nh,nkv,hd,rot,bs,vt", [(4, 2, 16, 16, 4, 0), (6, 1, 32, 32, 8, 1), (8, 4, 256, 256, 16, 1),
                                                (3, 3, 64, 32, 16, 0), (2, 2, 48, 0, 4, 1)])
def test_rope_and_cache_write(rt, dtype, T, nh, nkv, hd, rot, bs, vt):
    k = rt.kernels(dtype)
    rng = np.random.default_rng(hd)
    pages = 12
    qkv = rng.normal(size=(T, (nh + 2 * nkv) * hd)).astype(np.float32)
    if dtype == "bfloat16":
        qkv = bf16(qkv)
    pos = np.concatenate([[0, 1, 5, 1000, 8191, 17, 3], rng.integers(0, 4000, T - 7)]).astype(np.int32)
    slots = np.full(T, -1, np.int32)                         # tokens 27.. are not stored
    slots[:27] = rng.permutation(9 * bs)[:27]                # scattered over pages 0..8
    slots[2] = -1                                            # nothing stored for this token
    slots[8:16] = 9 * bs + np.arange(8) % bs                 # eight in a row from a page's start (if it has eight)
    if bs < 8:
        slots[12:16] = 10 * bs + np.arange(4) % bs
    slots[16:24] = 11 * bs + (3 + np.arange(8)) % bs if bs >= 16 else slots[16:24]      # in a row, not aligned
    assert len(set(slots[slots >= 0].tolist())) == (slots >= 0).sum()
    theta = 10000.0
    inv = (1.0 / theta ** (2.0 * np.arange(rot // 2) / max(rot, 1))).astype(np.float32)
    Q = up(rt, qkv, dtype)
    KC = rt.zeros((pages, nkv, bs, hd), dtype)
    VC = rt.zeros((pages, nkv, hd, bs) if vt else (pages, nkv, bs, hd), dtype)
    k.zk_rope_cache_write(Q.ptr, ptr(rt.upload(pos)), ptr(rt.upload(slots)), ptr(rt.upload(inv)) if rot else None, rot,
                          KC.ptr, VC.ptr, T, nh, nkv, hd, bs, vt, rt.stream)

    def rotate(x):                                           # x [T, heads, hd]
        x = x.astype(np.float64)
        if not rot:
            return x
        ang = pos[:, None].astype(np.float64) * inv.astype(np.float64)[None, :]
        c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
        a, b = x[..., :rot // 2], x[..., rot // 2:rot]
        return np.concatenate([a * c - b * s, b * c + a * s, x[..., rot:]], axis=-1)

    q = qkv[:, :nh * hd].reshape(T, nh, hd)
    kk = qkv[:, nh * hd:(nh + nkv) * hd].reshape(T, nkv, hd)
    vv = qkv[:, (nh + nkv) * hd:].reshape(T, nkv, hd)
    tol = 2e-3 if dtype == "float32" else 0.03               # float angles at position 8191
    got = rt.download_f32(Q)
    assert np.abs(got[:, :nh * hd].reshape(T, nh, hd) - rotate(q)).max() < tol
    assert np.array_equal(got[:, nh * hd:], qkv[:, nh * hd:])            # k and v rows are left as they were
    kc, vc = rt.download_f32(KC), rt.download_f32(VC)
    want_k, want_v = np.zeros_like(kc), np.zeros_like(vc)
    rk = rotate(kk)
    for t in range(T):
        if slots[t] < 0:
            continue
        p, o = divmod(int(slots[t]), bs)
        want_k[p, :, o, :] = rk[t]
        if vt:
            want_v[p, :, :, o] = vv[t]
        else:
            want_v[p, :, o, :] = vv[t]
    assert np.abs(kc - want_k).max() < tol and np.array_equal(vc, want_v)


@pytest.mark.parametrize("M,K,nh,nkv,hd,bs,vt,strip", [(5, 96, 6, 1, 32, 8, 1, 1), (16, 200, 3, 3, 64, 16, 0, 0),
                                                        (8, 2304, 8, 4, 256, 16, 1, 1), (1, 2048, 2, 2, 96, 4, 1, 1),
                                                        (3, 160, 4, 0, 32, 4, 1, 1), (11, 64, 5, 5, 160, 8, 0, 1),
                                                        (7, 96, 3, 1, 48, 8, 1, 1), (9, 72, 2, 1, 16, 4, 0, 0)])
def test_qkv_product_that_rotates_and_stores(rt, M, K, nh, nkv, hd, bs, vt, strip):
    """The fused product of decoded tokens leaves the same bits as the product followed by the
    rotation kernel: in q, and in the cache (which starts from a pattern, so that a store to a
    wrong place shows as well as a missing one)."""
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(M * 1000 + hd)
    N = (nh + 2 * nkv) * hd
    pages = 7
    a = bf16(rng.normal(size=(M, K)).astype(np.float32))
    w = bf16(rng.normal(size=(N, K)).astype(np.float32) / math.sqrt(K))
    pos = np.concatenate([[8191, 0, 1000], rng.integers(0, 8192, 16)])[:M].astype(np.int32)
    slots = rng.permutation(pages * bs)[:M].astype(np.int32)
    if M > 2:
        slots[2] = -1
    inv = (1.0 / 10000.0 ** (2.0 * np.arange(hd // 2) / hd)).astype(np.float32)
    A, W = up(rt, a, "bfloat16"), up(rt, w, "bfloat16")
    WS = W
    if strip:
        WS = rt.empty(((N + 15) // 16 * 16, K), "bfloat16")
        k.zk_strip_layout(W.ptr, WS.ptr, N, K, rt.stream)
    P, S, I = rt.upload(pos), rt.upload(slots), rt.upload(inv)
    pattern = bf16(rng.normal(size=(pages, max(nkv, 1), bs, hd)).astype(np.float32))
    assert k.zk_qkv_rope_bf16_supports(M, K, hd, hd)
    got = []
    for fused in (False, True):
        Q = up(rt, np.zeros((M, N), np.float32), "bfloat16")
        KC = up(rt, pattern, "bfloat16")
        VC = up(rt, pattern.reshape(pages, max(nkv, 1), hd, bs) if vt else pattern, "bfloat16")
        if fused:
            k.zk_qkv_rope_bf16(A.ptr, K, WS.ptr, Q.ptr, N, M, K, strip, P.ptr, S.ptr if nkv else None, I.ptr,
                               KC.ptr, VC.ptr, nh, nkv, hd, bs, vt, rt.stream)
        else:
            k.zk_gemm_bf16(A.ptr, K, WS.ptr, Q.ptr, N, 0, M, N, K, 0, 0.0, strip, None, 0, None, rt.stream)
            k.zk_rope_cache_write(Q.ptr, P.ptr, S.ptr if nkv else None, I.ptr, hd, KC.ptr, VC.ptr, M, nh, nkv, hd,
                                  bs, vt, rt.stream)
        got.append((rt.download_f32(Q)[:, :nh * hd], rt.download_f32(KC), rt.download_f32(VC)))
    for x, y in zip(*got):
        assert np.array_equal(x, y)
    assert not k.zk_qkv_rope_bf16_supports(17, K, hd, hd) and not k.zk_qkv_rope_bf16_supports(M, K, 40, 40)
    assert not k.zk_qkv_rope_bf16_supports(M, K, hd, hd // 2)


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("T,nh,nkv,hd,bs,vt,rot", [(5, 3, 1, 48, 8, 1, 48), (40, 8, 4, 64, 16, 1, 64), (64, 2, 2, 256, 16, 1, 256),
                                                 (100, 4, 2, 32, 8, 0, 32), (23, 2, 1, 64, 4, 0, 32), (72, 3, 3, 16, 8, 1, 16)])
def test_rotation_that_adds_up_partial_sums_itself(rt, dtype, T, nh, nkv, hd, bs, vt, rot):
    """The rows of [q | k | v] as three planes of float partial sums, added up by the kernel that
    rotates and stores: the same bits, in q and in the cache, as from the rows added up in order and
    rounded to the storage type beforehand.  Eight tokens in a row land in eight slots in a row of
    one page (the transposed store of whole groups) and one token is stored nowhere."""
    k = rt.kernels(dtype)
    rng = np.random.default_rng(T * 10 + hd)
    width = (nh + 2 * nkv) * hd
    planes = (rng.normal(size=(3, T, width)) * np.array([1.0, 1e-2, 1e-4])[:, None, None]).astype(np.float32)
    summed = (planes[0] + planes[1]) + planes[2]
    rows = bf16(summed) if dtype == "bfloat16" else summed
    pages = (T + bs - 1) // bs + 3
    free = [x for x in range(pages * bs) if x // bs != 2]
    slots = rng.permutation(free)[:T].astype(np.int32)
    if T >= 16 and bs >= 8:
        slots[8:16] = 2 * bs + np.arange(8)
    slots[min(3, T - 1)] = -1
    pos = rng.integers(0, 5000, T).astype(np.int32)
    inv = (1.0 / 10000.0 ** (2.0 * np.arange(rot // 2) / rot)).astype(np.float32)
    P, S, I = rt.upload(pos), rt.upload(slots), rt.upload(inv)
    pattern = rng.normal(size=(pages, nkv, bs, hd)).astype(np.float32)
    got = []
    for sums in (0, 3):
        Q = up(rt, rows if not sums else np.zeros_like(rows), dtype)
        KC = up(rt, pattern, dtype)
        VC = up(rt, pattern.reshape(pages, nkv, hd, bs) if vt else pattern, dtype)
        if sums:
            k.zk_rope_cache_write_sums(Q.ptr, ptr(rt.upload(planes)), 3, P.ptr, S.ptr, I.ptr, rot, KC.ptr, VC.ptr, T, nh, nkv,
                                       hd, bs, vt, rt.stream)
        else:
            k.zk_rope_cache_write(Q.ptr, P.ptr, S.ptr, I.ptr, rot, KC.ptr, VC.ptr, T, nh, nkv, hd, bs, vt, rt.stream)
        got.append((rt.download_f32(Q)[:, :nh * hd], rt.download_f32(KC), rt.download_f32(VC)))
    for x, y in zip(*got):
        assert np.array_equal(x, y)
    assert not np.array_equal(got[0][1], bf16(pattern) if dtype == "bfloat16" else pattern)      # something was stored


def test_convert_and_fill(rt):
    rng = np.random.default_rng(0)
    x = rng.normal(size=1003).astype(np.float32)
    from zse_amd.weights.safetensors import f32_to_bf16_bits
    kb, kf = rt.kernels("bfloat16"), rt.kernels("float32")
    out = rt.empty((1003,), "bfloat16")
    kb.zk_convert(ptr(rt.upload(x)), 0, out.ptr, 1, 1003, rt.stream)
    assert np.array_equal(rt.download(out), f32_to_bf16_bits(x))         # round to nearest even, as on the host
    half = x.astype(np.float16)
    out32 = rt.empty((1003,), "float32")
    kf.zk_convert(ptr(rt.upload(half.view(np.uint16), "bfloat16")), 2, out32.ptr, 0, 1003, rt.stream)
    assert np.array_equal(rt.download(out32), half.astype(np.float32))
    kf.zk_convert(ptr(rt.upload(f32_to_bf16_bits(x), "bfloat16")), 1, out32.ptr, 1, 1003, rt.stream)
    assert np.array_equal(rt.download(out32), bf16(x))
    big = rt.empty((200001,), "float32")
    kf.zk_fill_normal(big.ptr, 0, 200001, 5, 9, 0.5, 0.02, rt.stream)
    a = rt.download(big)
    assert abs(a.mean() - 0.5) < 3e-4 and abs(a.std() - 0.02) < 3e-4
    kf.zk_fill_normal(out32.ptr, 0, 1003, 5, 9, 0.5, 0.02, rt.stream)
    assert np.array_equal(rt.download(out32), a[:1003])                   # a function of (seed, stream, index)
    kf.zk_fill_normal(out32.ptr, 0, 1003, 6, 9, 0.5, 0.02, rt.stream)
    assert not np.array_equal(rt.download(out32), a[:1003])
    kf.zk_zero(big.ptr, 200000, rt.stream)
    z = rt.download(big)
    assert not z[:50000].any() and z[50000] != 0


def test_argmax_and_sampling(rt):
    from plain import gemma2_plain as P
    k = rt.kernels("float32")
    rng = np.random.default_rng(1)
    rows, V = 5, 256003
    z = rng.normal(size=(rows, V)).astype(np.float32) * 3
    z[1, 777] = z[1, 200000] = 50.0                          # a tie: the lower index wins
    z[2, V - 1] = 60.0
    z[3, 5] = np.nan
    Z = rt.upload(z)
    ids = rt.empty((rows,), "int32")
    scratch = rt.empty((rows * 64 * 5,), "float32")
    k.zk_argmax(Z.ptr, ids.ptr, rows, V, scratch.ptr, rt.stream)
    got = rt.download(ids)
    want = [int(np.nanargmax(r)) for r in z]
    want[1] = 777
    assert list(got) == want
    # (ref) the sampler vectors of tests/test_orchestrator.py:175-190
    small = np.array([[0.1, 0.5, 0.3, 0.9, 0.2], [-1.0, -0.5, -2.0, -3.0, -9.0]], np.float32)
    k.zk_argmax(ptr(rt.upload(small)), ids.ptr, 2, 5, scratch.ptr, rt.stream)
    assert list(rt.download(ids)[:2]) == [3, 1]
    # temperature sampling: the plain sampler's draw for the same uniform number
    z = rng.normal(size=(rows, 1000)).astype(np.float32) * 2
    temps = np.array([0.8, 1.0, 0.3, 2.0, 1.0], np.float32)
    us = np.array([0.0, 0.999999, 0.5, 0.25, 0.75])
    k.zk_sample(ptr(rt.upload(z)), ptr(rt.upload(temps)), ptr(rt.upload(us)), None, None, ids.ptr, rows, 1000, scratch.ptr, rt.stream)
    assert list(rt.download(ids)) == [P.sample(z[i], us[i], temperature=float(temps[i])) for i in range(rows)]
    # the frequencies follow softmax(z / T)
    z1 = np.array([[2.0, 1.0, 0.0, -1.0]], np.float32).repeat(4000, 0)
    from zse_amd.sampling import uniform
    u = np.array([uniform(3, i) for i in range(4000)])
    out = rt.empty((4000,), "int32")
    k.zk_sample(ptr(rt.upload(z1)), ptr(rt.upload(np.full(4000, 0.7, np.float32))), ptr(rt.upload(u)), None, None, out.ptr,
                4000, 4, ptr(rt.empty((4000 * 64 * 5,), "float32")), rt.stream)
    freq = np.bincount(rt.download(out), minlength=4) / 4000.0
    assert np.abs(freq - P.softmax(z1[0] / 0.7)).max() < 0.03


@pytest.mark.parametrize("V,ties", [(5003, False), (5003, True), (256000, False), (37, True)])
def test_top_k_top_p_and_penalty_on_the_device(rt, V, ties):
    """Every combination goes through the device sampler and picks what the host implementation
    (float64, sorting) picks for the same uniform number; with logits on a coarse grid many are
    equal, also at the cut-offs, where top-k keeps all of them and top-p the first few."""
    from zse_amd.sampling import DeviceSampler, SamplingParams, sample_host, uniform
    rng = np.random.default_rng(V + ties)
    combos = [dict(top_k=k_, top_p=p_, temperature=t_, repetition_penalty=r_)
              for k_ in (0, 1, 5, 50, V + 10) for p_ in (1.0, 0.9, 0.5, 0.02) for t_, r_ in ((0.7, 1.0), (1.3, 1.5))]
    combos += [dict(temperature=0.0, repetition_penalty=3.0), dict(temperature=0.0, top_k=3)]
    n = len(combos)
    z = (rng.normal(size=(n, V)) * 3).astype(np.float32)
    if ties:
        z = (np.round(z * 2) / 2).astype(np.float32)
    sampler = DeviceSampler(rt, rt.kernels("float32"), n)
    for trial in range(3):
        rows = []
        for i, c in enumerate(combos):
            order = np.argsort(-z[i])
            past = set(order[:3].tolist()) | set(rng.integers(0, V, 5).tolist())
            rows.append({"params": SamplingParams(**c), "u": uniform(trial * 1000 + i, 7) if trial else (0.0, 0.999999)[i % 2],
                         "past": past})
        got = sampler.sample(rt.upload(z), rows)                 # the penalty changes the logits in place: a fresh copy
        want = [sample_host(z[i], r["params"], r["u"], r["past"]) for i, r in enumerate(rows)]
        assert got == want, [(i, combos[i], g, w) for i, (g, w) in enumerate(zip(got, want)) if g != w]


def test_cut_offs_on_awkward_rows(rt):
    """All logits equal, two values only, minus infinity among them, a spread that leaves most
    weights at zero, a share that only the largest logit holds: the device still draws what
    the host implementation draws."""
    from zse_amd.sampling import DeviceSampler, SamplingParams, sample_host, uniform
    rng = np.random.default_rng(9)
    V = 1000
    flat = np.zeros(V, np.float32)
    two = np.where(rng.random(V) < 0.3, 2.0, -1.0).astype(np.float32)
    holes = (rng.normal(size=V) * 2).astype(np.float32)
    holes[rng.random(V) < 0.5] = -np.inf
    wide = (rng.normal(size=V) * 3000).astype(np.float32)
    rows_z = [flat, two, holes, wide]
    combos = [dict(top_k=10), dict(top_p=0.4995), dict(top_k=300, top_p=0.9), dict(top_p=1e-6), dict(top_k=999, top_p=0.9995)]      # (no share that a whole number of equal logits holds exactly)
    z = np.stack([r for r in rows_z for _ in combos])
    params = [SamplingParams(temperature=0.9, **c) for _ in rows_z for c in combos]
    sampler = DeviceSampler(rt, rt.kernels("float32"), len(params))
    for trial in range(4):
        rows = [{"params": p_, "u": uniform(trial, i), "past": ()} for i, p_ in enumerate(params)]
        got = sampler.sample(rt.upload(z), rows)
        want = [sample_host(z[i], r["params"], r["u"]) for i, r in enumerate(rows)]
        assert got == want, [(i, g, w) for i, (g, w) in enumerate(zip(got, want)) if g != w]


# ------------------------------------------------------------------ the LM head at full size
def test_lm_head_product_at_full_vocabulary(rt):
    """N = 256,000 rows of K = 2,304 in strip layout (1.18 GB, 16,000 strips), soft cap in the
    epilogue, float logits: every row count the engine uses (skinny 1 and 8, mid 40, tile 200)
    against the plain product on 3,000 sampled columns, the first and last strips among them."""
    from zse_amd.weights.normal import normal
    from zse_amd.weights.safetensors import f32_to_bf16_bits
    k = rt.kernels("bfloat16")
    N, K, cap, seed, stream = 256000, 2304, 30.0, 5, 99
    W = rt.empty((N, K), "bfloat16")
    k.zk_fill_normal(W.ptr, 1, N * K, seed, stream, 0.0, 0.05, rt.stream)
    Ws = rt.empty((N, K), "bfloat16")
    k.zk_strip_layout(W.ptr, Ws.ptr, N, K, rt.stream)
    rt.sync()
    rng = np.random.default_rng(3)
    cols = np.unique(np.concatenate([np.arange(0, 40), np.arange(N - 40, N), rng.integers(0, N, 2920),
                                     [65535, 65536, 131071, 131072]]))
    w_cols = np.stack([normal(K, seed, stream, 0.0, 0.05, first=int(c) * K) for c in cols])      # the same rows, made on the host
    Wc = rt.upload(f32_to_bf16_bits(w_cols), "bfloat16")
    ws = gemm_workspace(rt)
    for M in (1, 8, 40, 200):
        a = bf16(rng.normal(size=(M, K)))
        A = up(rt, a, "bfloat16")
        want = rt.empty((M, len(cols)), "float32")
        k.zk_gemm_plain(A.ptr, K, Wc.ptr, want.ptr, len(cols), 1, M, len(cols), K, rt.stream)
        want = rt.download(want).astype(np.float64)
        want = cap * np.tanh(want / cap)
        got = rt.zeros((M, N), "float32")
        k.zk_gemm_bf16(A.ptr, K, Ws.ptr, got.ptr, N, 1, M, N, K, 1, cap, 1, ws.ptr, ws.nbytes, None, rt.stream)
        got = rt.download(got)
        assert np.abs(want).max() > 5 and np.all(np.abs(got) < cap)
        err = np.abs(got[:, cols] - want)
        assert err.max() < 1e-4 * math.sqrt(K), f"M={M}: {err.max()} at column {cols[err.max(axis=0).argmax()]}"
        # no column outside the sample is left unwritten or wildly off: each has the spread of a logit
        assert np.all(got.std(axis=0) > 0) if M >= 8 else np.count_nonzero(got) > N * 0.99


def test_the_head_that_picks_without_writing_logits(rt):
    """zk_head_pick_bf16 against the product with the soft cap followed by zk_argmax, on the
    full vocabulary of 256,000 (and one that is no whole number of strips), 1 to 64 rows, with
    ties: rows of W that are copies of each other (equal logits: the lower column wins), and
    activations so large that the cap saturates and hundreds of columns hold the same largest
    value.  The same ids, bit for bit; nothing but the ids and the strips' picks is written."""
    k = rt.kernels("bfloat16")
    K, cap = 2304, 30.0
    rng = np.random.default_rng(11)
    for N in (256000, 4999):
        w = bf16(rng.normal(size=(N, K)) * 0.05)
        for a, b in ((17, 3), (N - 1, 4000), (N // 2 + 5, N // 2 + 4)):       # copies: later columns equal earlier ones
            w[a] = w[b]
        W = up(rt, w, "bfloat16")
        rows = (N + 15) // 16 * 16
        Ws = rt.zeros((rows, K), "bfloat16")
        k.zk_strip_layout(W.ptr, Ws.ptr, N, K, rt.stream)
        ws = gemm_workspace(rt)
        for M in (1, 8, 16, 24, 64):
            a = rng.normal(size=(M, K))
            a[0] = w[3] * 40                           # row 0 points at column 3 and its copy, column 17
            if M > 1:
                a[M - 1] = w[4000 % N] * 40
            if M > 2:
                a[1] *= 100                            # far beyond the cap: many columns saturate at 30.0
            a = bf16(a)
            A = up(rt, a, "bfloat16")
            logits = rt.zeros((M, N), "float32")
            k.zk_gemm_bf16(A.ptr, K, Ws.ptr, logits.ptr, N, 1, M, N, K, 1, cap, 1, ws.ptr, ws.nbytes, None, rt.stream)
            want = rt.zeros((M,), "int32")
            scratch = rt.zeros((M * 64 * 2,), "float32")
            k.zk_argmax(logits.ptr, want.ptr, M, N, scratch.ptr, rt.stream)
            picks = rt.zeros((k.zk_head_pick_bf16_workspace(M, N) // 4 + 4,), "float32")
            got = rt.zeros((M,), "int32")
            k.zk_head_pick_bf16(A.ptr, K, Ws.ptr, M, N, K, cap, 1, picks.ptr, picks.nbytes, got.ptr, rt.stream)
            want, got, z = rt.download(want), rt.download(got), rt.download(logits)
            assert np.array_equal(got, want), (N, M, got, want)
            assert np.array_equal(want, z.argmax(axis=1))             # NumPy's argmax keeps the first maximum too
            assert want[0] == 3 and (z[0, 17] == z[0, 3])
            if M > 2:
                assert np.count_nonzero(z[1] == z[1].max()) > 50, "the cap was meant to saturate"
        # row-major weights (no strip layout) serve up to 16 rows
        A = up(rt, bf16(rng.normal(size=(5, K))), "bfloat16")
        logits, want, got = rt.zeros((5, N), "float32"), rt.zeros((5,), "int32"), rt.zeros((5,), "int32")
        k.zk_gemm_bf16(A.ptr, K, W.ptr, logits.ptr, N, 1, 5, N, K, 1, cap, 0, ws.ptr, ws.nbytes, None, rt.stream)
        scratch = rt.zeros((5 * 64 * 2,), "float32")
        k.zk_argmax(logits.ptr, want.ptr, 5, N, scratch.ptr, rt.stream)
        picks = rt.zeros((k.zk_head_pick_bf16_workspace(5, N) // 4 + 4,), "float32")
        k.zk_head_pick_bf16(A.ptr, K, W.ptr, 5, N, K, cap, 0, picks.ptr, picks.nbytes, got.ptr, rt.stream)
        assert np.array_equal(rt.download(got), rt.download(want))
    from zse_amd.runtime.device import DeviceError
    with pytest.raises(DeviceError, match="1 to 64 rows"):
        k.zk_head_pick_bf16(A.ptr, K, Ws.ptr, 65, N, K, cap, 1, picks.ptr, picks.nbytes, got.ptr, rt.stream)
    with pytest.raises(DeviceError, match="scratch too small"):
        k.zk_head_pick_bf16(A.ptr, K, Ws.ptr, 5, N, K, cap, 1, picks.ptr, 64, got.ptr, rt.stream)


# ------------------------------------------------------------------ random weights
@pytest.mark.parametrize("n", [1, 2, 7, 4096, 1_000_003])
def test_device_random_weights_equal_the_host_function_bit_for_bit(rt, n):
    from zse_amd.weights.normal import normal
    from zse_amd.weights.safetensors import f32_to_bf16_bits
    for seed, stream, mean, std in [(0, 1234567, 0.0, 0.02), (2 ** 40 + 3, 2 ** 32 - 1, 0.5, 1.0)]:
        want = normal(n, seed, stream, mean, std)
        for dtype in ("float32", "bfloat16"):
            k = rt.kernels(dtype)
            out32 = rt.zeros((n,), "float32")
            k.zk_fill_normal(out32.ptr, 0, n, seed, stream, mean, std, rt.stream)
            got = rt.download(out32)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (
                f"{dtype} library, float output: first difference at {np.argmax(got != want)}")
        outb = rt.zeros((n,), "bfloat16")
        rt.kernels("bfloat16").zk_fill_normal(outb.ptr, 1, n, seed, stream, mean, std, rt.stream)
        assert np.array_equal(rt.download(outb), f32_to_bf16_bits(want))


def test_a_model_made_on_the_device_equals_the_folder_written_on_the_host(rt, tmp_path):
    """Same configuration, seed and deviations: ``random_model`` (weights drawn by the device in
    place) and ``write_random_model`` + ``load_model`` (drawn on the host, written, read, copied)
    are the same model: the same logits, bit for bit, in both types."""
    from conftest import TINY
    from zse_amd.engine.loading import load_model, random_model
    from zse_amd.engine.runner import StepEntry, StepRunner
    from zse_amd.weights import write_random_model
    cfg = TINY["B"][0]
    toks = np.random.default_rng(0).integers(0, cfg["vocab_size"], 19).tolist()
    for dtype in ("float32", "bfloat16"):
        folder = write_random_model(str(tmp_path / dtype), cfg, seed=21, std=0.07, gain_std=0.15, dtype=dtype,
                                    std_of={"embed_tokens": 0.02})
        rows = []
        for model in (load_model(folder, dtype, rt),
                      random_model(cfg, dtype, seed=21, std=0.07, gain_std=0.15, rt=rt, std_of={"embed_tokens": 0.02})):
            runner = StepRunner(model, rt, dtype, page_size=8, cache_tokens=64, max_seqs=2, max_batch_tokens=64,
                                max_model_len=64, use_graphs=False)
            rows.append(runner.step([StepEntry("a", toks, range(len(toks)))]))
        assert np.abs(rows[0]).max() > 0.1 and np.array_equal(rows[0], rows[1]), dtype


def test_the_two_ways_to_the_cut_offs(rt):
    """Rows made for the borders between the short way (a few candidates near the maximum, sorted by
    one block) and the long way (the search over the whole row): as many equal logits at the top as
    the candidates' room holds and one more, a k-th largest logit far below the maximum, a row of a
    real model's kind (a few hundred likely tokens over a flat rest), logits on the edges of the
    histogram's buckets, NaN among them.  Each row goes the way it is meant to and draws what the
    host implementation draws."""
    from zse_amd.sampling import DeviceSampler, SamplingParams, sample_host, uniform
    rng = np.random.default_rng(21)
    V = 70001
    cap = 2048
    def base():
        return (rng.normal(size=V) * 2 - 40).astype(np.float32)
    cases = []            # (logits, params, the way)
    full = base(); full[rng.choice(V, cap, replace=False)] = 3.0
    cases.append((full, dict(top_k=cap, top_p=0.7), 1))
    cases.append((full, dict(top_k=100), 1))
    over = base(); over[rng.choice(V, cap + 1, replace=False)] = 3.0
    cases.append((over, dict(top_k=100, top_p=0.9), 2))
    far = (rng.normal(size=V) * 2).astype(np.float32); far[12345] = 90.0
    cases.append((far, dict(top_k=50), 2))
    cases.append((far, dict(top_p=0.9), 1))                   # one logit holds it all
    peaked = base(); idx = rng.choice(V, 300, replace=False); peaked[idx] = (rng.normal(size=300) * 3).astype(np.float32)
    cases.append((peaked, dict(top_p=0.9), 1))
    cases.append((peaked, dict(top_k=50, top_p=0.9), 1))
    cases.append((peaked, dict(top_k=50), 1))
    cases.append((peaked, dict(top_p=0.999999), 1))             # what lies 32 below the maximum weighs nothing
    edges = base(); edges[:1500] = (5.0 - np.arange(1500) / 32.0 * 0.8).astype(np.float32)      # temperature 0.8: steps of a bucket
    cases.append((edges, dict(top_k=700), 1))
    cases.append((edges, dict(top_p=0.95), 1))
    cases.append((edges, dict(top_k=1000, top_p=0.99), 1))
    cases.append((edges, dict(top_k=1500, top_p=0.99), 2))    # the k-th largest lies in the last bucket
    nans = peaked.copy(); nans[rng.choice(V, 50, replace=False)] = np.nan; nans[idx[:3]] = np.nan
    cases.append((nans, dict(top_k=20, top_p=0.8), 1))
    spread = (rng.normal(size=V) * 0.5).astype(np.float32)      # many logits above either cut-off, few in its bucket
    cases.append((spread, dict(top_p=0.9), 3))
    cases.append((spread, dict(top_k=5000), 3))
    cases.append((spread, dict(top_k=5000, top_p=0.9), 2))
    grid = (np.round(spread * 80) / 80).astype(np.float32)      # some hundred equal logits at the cut-off
    cases.append((grid, dict(top_p=0.8), 3))
    cases.append((grid, dict(top_k=3000), 3))
    zeros = grid.copy(); zeros[np.abs(zeros) < 0.2] = 0.0; zeros[::3] *= -1.0        # 0.0 and -0.0 are equal logits
    assert np.signbit(zeros[zeros == 0]).any() and not np.signbit(zeros[zeros == 0]).all()
    def share_inside_the_zeros(row):          # a share that is reached among the equal logits at zero (and by no whole number of them)
        w = np.exp(row.astype(np.float64) / 0.8)
        return float((w[row > 0].sum() + 0.41373 * w[row == 0].sum()) / w.sum())
    cases.append((zeros, dict(top_p=share_inside_the_zeros(zeros)), 2))
    few = zeros.copy(); few[1500:] -= 30.0
    cases.append((few, dict(top_p=share_inside_the_zeros(few)), 1))
    flat = np.zeros(V, np.float32)
    cases.append((flat, dict(top_k=10), 2))
    cases.append((flat, dict(top_p=0.5005), 2))
    cases.append((flat, dict(), 0))
    z = np.stack([c[0] for c in cases])
    params = [SamplingParams(temperature=0.8, **c[1]) for c in cases]
    sampler = DeviceSampler(rt, rt.kernels("float32"), len(cases) + 3)
    for trial in range(6):
        us = [(0.0, 0.999999)[trial] if trial < 2 else uniform(trial, i) for i in range(len(cases))]
        rows = [{"params": p_, "u": u_, "past": ()} for p_, u_ in zip(params, us)]
        got = sampler.sample(rt.upload(z), rows)
        assert sampler.cut_ways(len(cases)) == [c[2] for c in cases]
        zz = np.where(np.isnan(z), -np.inf, z)                 # the host implementation has no rule for NaN: never drawn
        want = [sample_host(zz[i], r["params"], r["u"]) for i, r in enumerate(rows)]
        assert got == want, [(i, cases[i][1], g, w) for i, (g, w) in enumerate(zip(got, want)) if g != w]
    # fewer rows afterwards, and more again: what a call leaves behind serves the next
    for n in (2, len(cases)):
        rows = [{"params": params[i], "u": uniform(99, i), "past": ()} for i in range(n)]
        got = sampler.sample(rt.upload(z[:n]), rows)
        zz = np.where(np.isnan(z), -np.inf, z)
        assert got == [sample_host(zz[i], r["params"], r["u"]) for i, r in enumerate(rows)]
