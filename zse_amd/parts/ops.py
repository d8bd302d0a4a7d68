"""Operations that several parts share; the one place where a kernel is chosen."""
from __future__ import annotations

from ..runtime.device import BF16, F32, Tensor


def linear(ctx, x: Tensor, w: Tensor, out: Tensor) -> Tensor:
    """out[M, N] = x[M, K] @ w[N, K]^T with float accumulation.

    ``out`` may be float32 (logits) or the activation type.  In the 32-bit
    library only the plain product exists; the bf16 library picks a matrix-core
    kernel by the number of rows.
    """
    M, K = x.shape
    N, K2 = w.shape
    if K != K2 or out.shape != (M, N):
        raise ValueError(f"linear: x {x.shape}, w {w.shape}, out {out.shape} do not fit")
    if x.dtype != ctx.dtype or w.dtype != ctx.dtype:
        raise ValueError(f"linear: operands must be {ctx.dtype}, got x {x.dtype}, w {w.dtype}")
    if out.dtype not in (F32, ctx.dtype):
        raise ValueError(f"linear: out must be float32 or {ctx.dtype}, got {out.dtype}")
    out_f32 = 1 if out.dtype == F32 else 0
    k = ctx.k
    if ctx.dtype == BF16 and ctx.tuned and k.has("zk_gemm_bf16"):
        k.zk_gemm_bf16(x.ptr, K, w.ptr, out.ptr, N, out_f32, M, N, K, ctx.stream)
    else:
        k.zk_gemm_plain(x.ptr, K, w.ptr, out.ptr, N, out_f32, M, N, K, ctx.stream)
    return out
