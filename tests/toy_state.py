"""A mixer the framework has never heard of, for tests: out_t = s_t W^T with the recurrence
s_t = decay * s_(t-1) + x_t kept per request in its state slot (no pages at all).  The
recurrence runs on the host (a toy); rows come in, rows go out, the state lives in the slot
between steps.  It reads the step's host-side description, so it is not safe to capture."""
from contextlib import contextmanager
from dataclasses import dataclass

import numpy as np

from zse_amd.parts import Part, StateNeed, TensorReq, register_part, unregister_part
from zse_amd.parts.ops import linear


@dataclass(frozen=True)
class DecaySpec:
    hidden_size: int
    decay: float
    weight: str
    kind: str = "toy_decay"


class DecayMixer(Part):
    def __init__(self, spec):
        self.spec, self.w = spec, None

    def tensor_reqs(self):
        return [TensorReq(self.spec.weight, (self.spec.hidden_size, self.spec.hidden_size))]

    def load(self, weights, rt_, dtype):
        self.w = weights.matrix([self.spec.weight])

    def cache_need(self):
        return StateNeed(self.spec.hidden_size * 4)

    def forward(self, ctx, x, cache):
        xs = ctx.rt.download_f32(x)
        state = ctx.rt.download(ctx.state)
        o0, n_w = cache.state_offset // 4, cache.state_bytes // 4
        out = np.empty_like(xs)
        t = 0
        for _, slot, _, n in ctx.entries:
            s = state[slot, o0:o0 + n_w].copy()
            for i in range(n):
                s = np.float32(self.spec.decay) * s + xs[t + i]
                out[t + i] = s
            state[slot, o0:o0 + n_w] = s
            t += n
        ctx.rt.copy_h2d(ctx.state.ptr, state)
        if x.dtype == "bfloat16":
            from zse_amd.weights.safetensors import f32_to_bf16_bits
            out = f32_to_bf16_bits(out)
        y = ctx.alloc(x.shape)
        ctx.rt.copy_h2d(y.ptr, out)
        return linear(ctx, y, self.w, ctx.alloc(x.shape))


@contextmanager
def toy_architecture(name, plan_of):
    """Registers the toy mixer and an architecture ``name`` whose plan is ``plan_of(config)``."""
    from zse_amd.config import Architecture, register_architecture, unregister_architecture
    register_part("mixer", "toy_decay", DecayMixer)
    register_architecture(Architecture(name, lambda d: d, plan_of))
    try:
        yield
    finally:
        unregister_part("mixer", "toy_decay")
        unregister_architecture(name)
