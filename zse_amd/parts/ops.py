"""Operations that several parts share; the one place where a kernel is chosen."""
from __future__ import annotations

import ctypes

from ..runtime.device import BF16, F32, Tensor


EPILOGUES = {None: 0, "softcap": 1, "gelu_tanh": 2, "silu": 3}


def tuned_gemm(ctx, K: int) -> bool:
    """True when the matrix-core product serves this step (bf16, tuned kernels on,
    rows of K values that are whole 16-byte pieces)."""
    return ctx.dtype == BF16 and ctx.tuned and ctx.k.has("zk_gemm_bf16") and K % 8 == 0


def linear(ctx, x: Tensor, w: Tensor, out: Tensor, epilogue=None, cap: float = 0.0, last_of=None,
           sums_ok: bool = False) -> Tensor:
    """out[M, N] = x[M, K] @ w[N, K]^T with float accumulation.

    ``out`` may be float32 (logits) or the activation type.  In the 32-bit
    library only the plain product exists; the bf16 library picks a matrix-core
    kernel by the number of rows.  ``epilogue`` (matrix-core product only):
    "softcap" applies cap * tanh(x / cap); "gelu_tanh" / "silu" take w as
    [2N, K], gate rows first, and store act(gate) * up.

    ``last_of``: the part whose result this product is (it passes itself).  When the block
    that called that very part has said that partial sums are welcome (``ctx.sums_welcome`` is
    the part: the block's joining kernel adds them up itself) and the product splits K over
    blocks, the joining launch is left out: what comes back is a float32 tensor [P, M, N] with
    layout "parts" in the product's workspace instead of ``out``, to be read before the next
    product.  A part that another part calls is not the one the block named, so it never
    hands partial sums to a caller that does not expect them.  ``sums_ok``: the caller reads
    such a tensor itself, whoever called it.
    """
    M, K = x.shape
    gated = epilogue in ("gelu_tanh", "silu")
    N, K2 = w.shape
    if gated:
        N //= 2
    if epilogue is not None and not tuned_gemm(ctx, K):
        raise ValueError("linear: epilogues belong to the matrix-core product")
    if K != K2 or out.shape != (M, N):
        raise ValueError(f"linear: x {x.shape}, w {w.shape}, out {out.shape} do not fit")
    if x.dtype != ctx.dtype or w.dtype != ctx.dtype:
        raise ValueError(f"linear: operands must be {ctx.dtype}, got x {x.dtype}, w {w.dtype}")
    if out.dtype not in (F32, ctx.dtype):
        raise ValueError(f"linear: out must be float32 or {ctx.dtype}, got {out.dtype}")
    out_f32 = 1 if out.dtype == F32 else 0
    k = ctx.k
    strip = w.layout == "strip"
    if strip and not tuned_gemm(ctx, K):
        raise ValueError("linear: weights in strip layout need the matrix-core product")
    if tuned_gemm(ctx, K):
        ws = getattr(ctx, "gemm_workspace", None)      # lets a product of few columns split K over blocks
        welcome = sums_ok or (last_of is not None and getattr(ctx, "sums_welcome", None) is last_of)
        parts = ctypes.c_int(0) if (welcome and ws is not None) else None
        k.zk_gemm_bf16(x.ptr, K, w.ptr, out.ptr, N, out_f32, M, N, K, EPILOGUES[epilogue], float(cap),
                       1 if strip else 0, ws.ptr if ws is not None else None,
                       ws.nbytes if ws is not None else 0, ctypes.byref(parts) if parts is not None else None,
                       ctx.stream)
        if parts is not None and parts.value > 0:
            return Tensor(ws.ptr, (parts.value, M, N), F32, ws.owner, layout="parts")
    else:
        k.zk_gemm_plain(x.ptr, K, w.ptr, out.ptr, N, out_f32, M, N, K, ctx.stream)
    return out
