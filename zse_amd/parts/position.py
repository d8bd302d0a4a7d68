"""Position encodings for a mixer's queries and keys.

Rotary: pair (i, i + rotary_dim/2) of a head is rotated by the angle
pos * theta^(-2i/rotary_dim), the rotate-half pairing of the reference's kernel
(orchestrator/kernels.py:264-297).  The cache stores keys after rotation, so an
encoding must be a function of the absolute position alone.
"""
from __future__ import annotations

import numpy as np

from ..runtime.device import Tensor
from .base import Part, register_part


class Rotary(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        if spec.rotary_dim % 2 or not (0 < spec.rotary_dim <= spec.head_dim):
            raise ValueError(f"rotary_dim must be even and in (0, head_dim], got {spec.rotary_dim}")
        self.spec = spec
        self.inv_freq = None

    def frequencies(self) -> np.ndarray:
        s = self.spec
        i = np.arange(s.rotary_dim // 2, dtype=np.float64)
        return (1.0 / np.power(float(s.theta), 2.0 * i / s.rotary_dim)).astype(np.float32)

    def load(self, weights, rt, dtype):
        self.inv_freq = rt.upload(self.frequencies())

    def rotary_tables(self):
        return self.inv_freq, self.spec.rotary_dim

    def apply(self, ctx, qkv: Tensor, num_heads: int, num_kv_heads: int, head_dim: int):
        raise NotImplementedError("a rotary encoding is applied by the mixer's fused kernel")


class NoPosition(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        self.spec = spec

    def rotary_tables(self):
        return None

    def apply(self, ctx, qkv, num_heads, num_kv_heads, head_dim):
        return None


register_part("position", "rotary", Rotary)
register_part("position", "none", NoPosition)
