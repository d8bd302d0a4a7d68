"""Root-mean-square norm, gain (1 + w) or w.

Statistics and the product are float; rsqrt(mean(x^2) + eps) as in the
reference's kernel (orchestrator/kernels.py:1435-1465); the reference multiplies
by plain w and names the (1 + w) form of Gemma 2 in a comment (:1476-1478).
"""
from __future__ import annotations

from typing import List, Optional

from ..runtime.device import F32, Tensor
from .base import ROLE_GAIN, Part, TensorReq, register_part


class RMSNorm(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        self.spec = spec
        self.weight: Optional[Tensor] = None

    def tensor_reqs(self) -> List[TensorReq]:
        return [TensorReq(self.spec.weight, (self.spec.size,), ROLE_GAIN)]

    def load(self, weights, rt, dtype):
        self.weight = weights.vector(self.spec.weight)

    def forward(self, ctx, x: Tensor, out_rows=None) -> Tensor:
        """Norm of every row of ``x`` (float stream or activations), or of the rows
        ``out_rows = (device int32 pointer, count)``."""
        s = self.spec
        rows_ptr, n = (out_rows if out_rows is not None else (0, x.shape[0]))
        out = ctx.alloc((n, s.size))
        ctx.k.zk_rmsnorm(x.ptr, 1 if x.dtype == F32 else 0,
                         rows_ptr or None, self.weight.ptr, out.ptr, s.eps,
                         1 if s.unit_offset else 0, n, s.size, ctx.stream)
        return out


register_part("norm", "rmsnorm", RMSNorm)
