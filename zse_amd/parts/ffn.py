"""Gated feed-forward: act(x Wg^T) * (x Wu^T), then Wd^T.

gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))) is the
reference's GeGLU kernel (orchestrator/kernels.py:1678-1697, wiring
model_runner.py:518-530); silu is its Llama activation (kernels.py:228-244).
Gate and up are two products there (model_runner.py:1270-1275), one here.
"""
from __future__ import annotations

from typing import List

from ..runtime.device import Tensor
from .base import Part, TensorReq, register_part
from .ops import linear, tuned_gemm

ACTIVATION_CODES = {"gelu_tanh": 0, "silu": 1}


class GatedMLP(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        if spec.activation not in ACTIVATION_CODES:
            raise ValueError(f"activation must be one of {sorted(ACTIVATION_CODES)}, got {spec.activation!r}")
        self.spec = spec
        self.w_gu = self.w_down = None

    def tensor_reqs(self) -> List[TensorReq]:
        s = self.spec
        return [TensorReq(s.names["gate"], (s.intermediate_size, s.hidden_size)),
                TensorReq(s.names["up"], (s.intermediate_size, s.hidden_size)),
                TensorReq(s.names["down"], (s.hidden_size, s.intermediate_size))]

    def load(self, weights, rt, dtype):
        s = self.spec
        strip = getattr(weights, "wants_strip", None)
        gu = [s.names["gate"], s.names["up"]]
        self.w_gu = (weights.matrix(gu, strip=True) if strip and strip(s.hidden_size, s.intermediate_size)
                     else weights.matrix(gu))
        self.w_down = (weights.matrix([s.names["down"]], strip=True) if strip and strip(s.intermediate_size)
                       else weights.matrix([s.names["down"]]))

    def forward(self, ctx, x: Tensor) -> Tensor:
        s = self.spec
        T, I = x.shape[0], s.intermediate_size
        if tuned_gemm(ctx, s.hidden_size):
            a = linear(ctx, x, self.w_gu, ctx.alloc((T, I)), epilogue=s.activation)
            return linear(ctx, a, self.w_down, ctx.alloc((T, s.hidden_size)), last_of=self)
        gu = linear(ctx, x, self.w_gu, ctx.alloc((T, 2 * I)))
        a = ctx.alloc((T, I))
        ctx.k.zk_gated_act(gu.ptr, a.ptr, T, I, ACTIVATION_CODES[s.activation], ctx.stream)
        return linear(ctx, a, self.w_down, ctx.alloc((T, s.hidden_size)), last_of=self)


register_part("ffn", "gated_mlp", GatedMLP)
