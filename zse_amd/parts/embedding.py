"""Token embedding into the float stream, and the output head.

The gather writes float rows (orchestrator/kernels.py:1789-1806) times a scale,
sqrt(hidden) for Gemma (orchestrator/model_runner.py:153-158, 332-339).  The head
multiplies by the embedding matrix itself when the weights are tied
(model_runner.py:566-572) and soft-caps the float logits (kernels.py:1714-1727,
model_runner.py:573-576); only the rows that were asked for are computed, where
the reference computes all of them (model_runner.py:362-373).
"""
from __future__ import annotations

from typing import List

import numpy as np

from ..runtime.device import BF16, F32, Tensor
from .base import Part, TensorReq, register_part
from .ops import linear, tuned_gemm


class Embedding(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        self.spec = spec
        self.table = None
        self.scale = float(spec.scale)

    def tensor_reqs(self) -> List[TensorReq]:
        return [TensorReq(self.spec.weight, (self.spec.vocab_size, self.spec.hidden_size))]

    def load(self, weights, rt, dtype):
        # the table may be the head's matrix too (tied): both ask for the same layout
        strip = getattr(weights, "wants_strip", None)
        self.table = (weights.matrix([self.spec.weight], strip=True) if strip and strip(self.spec.hidden_size)
                      else weights.matrix([self.spec.weight]))
        # the scalar is kept in the table's storage type, as the reference keeps its own
        # (model_runner.py:155-158); the product is float
        s = np.float32(self.spec.scale)
        if dtype == BF16:
            from ..weights.safetensors import bf16_bits_to_f32, f32_to_bf16_bits
            s = bf16_bits_to_f32(f32_to_bf16_bits(np.array([s])))[0]
        self.scale = float(s)

    def flops_per_token(self) -> float:
        return 0.0           # rows are gathered, not multiplied

    def forward(self, ctx) -> Tensor:
        s = self.spec
        h = ctx.alloc((ctx.T, s.hidden_size), F32)
        ctx.k.zk_embed(self.table.ptr, ctx.tokens, h.ptr, self.scale, ctx.T, s.hidden_size,
                       s.vocab_size, 1 if self.table.layout == "strip" else 0, ctx.stream)
        return h


class LMHead(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        self.spec = spec
        self.weight = None

    def tensor_reqs(self) -> List[TensorReq]:
        return [TensorReq(self.spec.weight, (self.spec.vocab_size, self.spec.hidden_size))]

    def load(self, weights, rt, dtype):
        strip = getattr(weights, "wants_strip", None)
        self.weight = (weights.matrix([self.spec.weight], strip=True) if strip and strip(self.spec.hidden_size)
                       else weights.matrix([self.spec.weight]))

    PICK_ROWS = 64         # the most rows the picking product takes

    def can_pick(self, ctx, rows: int) -> bool:
        """Whether ``pick`` serves this many rows: the matrix-core product with the picking
        epilogue (up to 64 rows; more than 16 need the strip layout)."""
        return bool(tuned_gemm(ctx, self.spec.hidden_size) and ctx.k.has("zk_head_pick_bf16") and
                    1 <= rows <= self.PICK_ROWS and (rows <= 16 or self.weight.layout == "strip"))

    def pick_scratch_bytes(self, kernels, rows: int) -> int:
        return int(kernels.zk_head_pick_bf16_workspace(int(rows), self.spec.vocab_size))

    def pick(self, ctx, x: Tensor, ids: Tensor, scratch: Tensor) -> Tensor:
        """ids[r] = the column of row r's largest logit (after the soft cap; the lowest column
        among equals): the greedy choice, taken in the product's epilogue strip by strip, so
        that the [rows, vocab] logits are neither written nor read back.  The same column as
        ``forward`` followed by the argmax kernel gives."""
        s = self.spec
        ctx.k.zk_head_pick_bf16(x.ptr, s.hidden_size, self.weight.ptr, x.shape[0], s.vocab_size, s.hidden_size,
                                float(s.softcap) if s.softcap else 0.0, 1 if self.weight.layout == "strip" else 0,
                                scratch.ptr, scratch.nbytes, ids.ptr, ctx.stream)
        return ids

    def forward(self, ctx, x: Tensor, out: Tensor) -> Tensor:
        """x: normed rows [K, hidden]; out: float logits [K, vocab]."""
        s = self.spec
        if s.softcap and tuned_gemm(ctx, s.hidden_size):
            return linear(ctx, x, self.weight, out, epilogue="softcap", cap=float(s.softcap))
        linear(ctx, x, self.weight, out)
        if s.softcap:
            ctx.k.zk_softcap(out.ptr, out.numel, float(s.softcap), ctx.stream)
        return out


register_part("embedding", "embedding", Embedding)
register_part("head", "lm_head", LMHead)
