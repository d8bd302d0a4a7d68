"""The matrix product that allocates nothing (zk_gemm_bf16_static), called through ctypes as a
caller outside the package would, against zk_gemm_bf16 with its workspace (the same bits) and
against a float64 NumPy product (a mistake the two share would pass the first comparison), on
calls in a row of which the second is smaller, with the array's old contents in the way; the
device's free memory is the same before and after, and a call recorded into a graph, which is
where a caller cannot allocate, gives the same bits on every replay."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

VP, I, F = C.c_void_p, C.c_int, C.c_float


@pytest.fixture(scope="module")
def rt():
    from zse_amd.runtime.device import Runtime
    return Runtime.get()


@pytest.fixture(scope="module")
def dll(rt):
    from zse_amd.runtime import build
    rt.kernels("bfloat16")                       # makes sure the library is built
    lib = C.CDLL(build.lib_path("kernels_bf16"))
    lib.zk_last_error.restype = C.c_char_p
    lib.zk_gemm_bf16_static_bytes.restype = C.c_size_t
    lib.zk_gemm_bf16_static_bytes.argtypes = []
    lib.zk_gemm_bf16_static_init.restype = I
    lib.zk_gemm_bf16_static_init.argtypes = []
    lib.zk_gemm_bf16_static.restype = I
    lib.zk_gemm_bf16_static.argtypes = [VP, I, VP, VP, I, I, I, I, I, I, F, I, VP]
    lib.zk_gemm_bf16.restype = I
    lib.zk_gemm_bf16.argtypes = [VP, I, VP, VP, I, I, I, I, I, I, F, I, VP, C.c_size_t, C.POINTER(I), VP]
    lib.zk_strip_layout.restype = I
    lib.zk_strip_layout.argtypes = [VP, VP, I, I, VP]
    return lib


def bf16_bits(x):
    from zse_amd.weights.safetensors import f32_to_bf16_bits
    return f32_to_bf16_bits(np.ascontiguousarray(x, np.float32))


def from_bits(b):
    from zse_amd.weights.safetensors import bf16_bits_to_f32
    return bf16_bits_to_f32(b).astype(np.float64)


def operands(rt, dll, M, N, K, seed, strip, gated=False, host=None):
    rng = np.random.default_rng(seed)
    rows = 2 * N if gated else N
    a, w = bf16_bits(rng.normal(size=(M, K))), bf16_bits(rng.normal(size=(rows, K)) * (0.05 if gated else 1.0))
    if host is not None:
        host.extend([from_bits(a), from_bits(w)])
    A = rt.upload(a, "bfloat16")
    W = rt.upload(w, "bfloat16")
    if strip:
        Ws = rt.empty(((rows + 15) // 16 * 16, K), "bfloat16")
        assert dll.zk_strip_layout(W.ptr, Ws.ptr, rows, K, rt.stream) == 0, dll.zk_last_error()
        rt.sync()
        W = Ws
    return A, W


def both(rt, dll, ws, M, N, K, seed, strip=1, epi=0, f32_out=0):
    """(bits from the static entry point, bits from zk_gemm_bf16 with its workspace)."""
    host = []
    A, W = operands(rt, dll, M, N, K, seed, strip, gated=epi >= 2, host=host)
    dt = "float32" if f32_out else "bfloat16"
    got, want = rt.zeros((M, N), dt), rt.zeros((M, N), dt)
    rc = dll.zk_gemm_bf16_static(A.ptr, K, W.ptr, got.ptr, N, f32_out, M, N, K, epi, 0.0, strip, rt.stream)
    assert rc == 0, dll.zk_last_error().decode()
    rc = dll.zk_gemm_bf16(A.ptr, K, W.ptr, want.ptr, N, f32_out, M, N, K, epi, 0.0, strip, ws.ptr, ws.nbytes,
                          None, rt.stream)
    assert rc == 0, dll.zk_last_error().decode()
    g, w = rt.download(got), rt.download(want)
    assert np.abs(w.astype(np.float64)).max() > 0
    # and against NumPy in float64: the two entry points share their kernels, split and join
    a64, w64 = host
    z = a64 @ w64.T
    if epi >= 2:                                 # gate rows first, then up rows: gelu_tanh(gate) * up
        gate, upp = z[:, :N], z[:, N:]
        z = 0.5 * gate * (1 + np.tanh(0.7978845608028654 * (gate + 0.044715 * gate ** 3))) * upp
    out = g.astype(np.float64) if f32_out else from_bits(g)
    tol = (2e-5 if f32_out else 1e-2) * np.abs(z).max()
    assert np.abs(out - z).max() < tol, (M, N, K, np.abs(out - z).max(), np.abs(z).max())
    return g, w


def ranges_of(rt, dll, ws, M, N, K):
    """Into how many ranges zk_gemm_bf16 splits K for this shape (0: not at all)."""
    A, W = operands(rt, dll, M, N, K, 0, 1)
    out = rt.zeros((M, N), "bfloat16")
    parts = I(0)
    rc = dll.zk_gemm_bf16(A.ptr, K, W.ptr, out.ptr, N, 0, M, N, K, 0, 0.0, 1, ws.ptr, ws.nbytes,
                          C.byref(parts), rt.stream)
    assert rc == 0, dll.zk_last_error().decode()
    rt.sync()
    return parts.value


def test_static_product_equals_the_one_with_a_workspace(rt, dll):
    assert dll.zk_gemm_bf16_static_bytes() == 16 << 20
    assert dll.zk_gemm_bf16_static_init() == 0, dll.zk_last_error().decode()
    assert dll.zk_gemm_bf16_static_init() == 0           # a second set-up call changes nothing
    ws = rt.zeros((rt.kernels("bfloat16").zk_gemm_bf16_workspace() // 4,), "float32")
    # the calls below neither take nor give back device memory (beyond what the test uploads
    # itself, which it holds on to until both readings are taken)
    held = [operands(rt, dll, 40, 2304, 2304, 1, 1), rt.zeros((40, 2304), "bfloat16")]
    (A0, W0), out0 = held
    assert dll.zk_gemm_bf16_static(A0.ptr, 2304, W0.ptr, out0.ptr, 2304, 0, 40, 2304, 2304, 0, 0.0, 1, rt.stream) == 0
    rt.sync()                                    # the kernels' code is on the device now
    free_before, mine_before = rt.info().free_memory, rt.allocated
    for _ in range(3):
        assert dll.zk_gemm_bf16_static(A0.ptr, 2304, W0.ptr, out0.ptr, 2304, 0, 40, 2304, 2304, 0, 0.0, 1, rt.stream) == 0
    rt.sync()
    assert rt.info().free_memory == free_before and rt.allocated == mine_before
    # 40 rows, N = 2304: 36 column blocks, so K is split into ranges whose partial sums
    # (planes of [40, 2304] floats, 0.37 MB each) go through the static array
    g, w = both(rt, dll, ws, 40, 2304, 2304, seed=1)
    assert np.array_equal(g, w)
    assert ranges_of(rt, dll, ws, 40, 2304, 2304) >= 2     # the shape does go through the scratch memory
    # the second call is smaller: other plane sizes, over what the first call left behind
    g, w = both(rt, dll, ws, 24, 1152, 1024, seed=2)
    assert np.array_equal(g, w)
    # a third, larger again and gated (two planes a range), float output
    g, w = both(rt, dll, ws, 64, 1024, 2048, seed=3, epi=2, f32_out=1)
    assert np.array_equal(g, w)
    # many rows, few tiles and a long K: the tile kernel splits K and joins through the array
    g, w = both(rt, dll, ws, 100, 200, 2048, seed=4, strip=0, f32_out=1)
    assert np.array_equal(g, w)
    # few rows without a split: the array is not touched, the result is still the same
    g, w = both(rt, dll, ws, 8, 2304, 2048, seed=5)
    assert np.array_equal(g, w)


def test_static_product_inside_a_captured_graph(rt, dll):
    """Where a caller cannot allocate: the call is recorded between capture_begin and
    capture_end (after the set-up call, which looks the array up, has run outside), and the
    graph is replayed with other work on the array in between; every replay gives the bits of
    the eager call."""
    assert dll.zk_gemm_bf16_static_init() == 0
    M, N, K = 40, 2304, 2304
    A, W = operands(rt, dll, M, N, K, 7, 1)
    eager, out = rt.zeros((M, N), "bfloat16"), rt.zeros((M, N), "bfloat16")
    assert dll.zk_gemm_bf16_static(A.ptr, K, W.ptr, eager.ptr, N, 0, M, N, K, 0, 0.0, 1, rt.stream) == 0
    want = rt.download(eager)
    A2, W2 = operands(rt, dll, 24, 1152, 1024, 8, 1)
    other = rt.zeros((24, 1152), "bfloat16")
    rt.sync()
    free_before = rt.info().free_memory
    rt.capture_begin()
    try:
        rc = dll.zk_gemm_bf16_static(A.ptr, K, W.ptr, out.ptr, N, 0, M, N, K, 0, 0.0, 1, rt.stream)
    finally:
        graph = rt.capture_end()
    assert rc == 0, dll.zk_last_error().decode()
    assert not rt.download(out).any()              # recorded, not run
    for _ in range(3):
        rt.graph_launch(graph)
        assert np.array_equal(rt.download(out), want)
        rt.zero_(out)
        # another product scribbles over the array between the replays
        assert dll.zk_gemm_bf16_static(A2.ptr, 1024, W2.ptr, other.ptr, 1152, 0, 24, 1152, 1024, 0, 0.0, 1, rt.stream) == 0
        rt.sync()
    rt.graph_destroy(graph)
    assert rt.info().free_memory >= free_before - (64 << 20)      # the graph's own bookkeeping aside, nothing was taken


def test_static_product_refuses_what_does_not_fit(rt, dll):
    # 1024 rows, N = 1024, K = 65536: a few dozen tiles and a very long K, so K is split into
    # eight ranges, 32 MB of partial sums; the array holds 16 MB, so the call is refused and
    # nothing is launched
    M, N, K = 1024, 1024, 65536
    A = rt.zeros((M, K), "bfloat16")
    W = rt.zeros((N, K), "bfloat16")
    out = rt.zeros((M, N), "bfloat16")
    rc = dll.zk_gemm_bf16_static(A.ptr, K, W.ptr, out.ptr, N, 0, M, N, K, 0, 0.0, 0, rt.stream)
    assert rc != 0
    msg = dll.zk_last_error().decode()
    assert "static scratch array holds 16777216" in msg and "need" in msg
    rt.sync()
