"""The toy mixer of ``toy_state`` with its recurrence in a kernel of its own (``toy_decay.hip``,
beside this file), brought to the framework through ``register_kernels``: the framework
compiles it, makes it a method of the kernel library and lets launch lists and captured
graphs repeat it.  Nothing under ``zse_amd/`` knows of it."""
from dataclasses import dataclass

from zse_amd.parts import Part, StateNeed, TensorReq, register_part
from zse_amd.parts.ops import linear

import toy_kernels  # noqa: F401  (registers zk_toy_decay)


@dataclass(frozen=True)
class DeviceDecaySpec:
    hidden_size: int
    decay: float
    weight: str
    kind: str = "toy_decay_device"


class DeviceDecayMixer(Part):
    graph_safe = True          # tokens, requests and slots are read by the kernel from device memory

    def __init__(self, spec):
        self.spec, self.w = spec, None

    def tensor_reqs(self):
        return [TensorReq(self.spec.weight, (self.spec.hidden_size, self.spec.hidden_size))]

    def load(self, weights, rt_, dtype):
        self.w = weights.matrix([self.spec.weight])

    def cache_need(self):
        return StateNeed(self.spec.hidden_size * 4)

    def forward(self, ctx, x, cache):
        y = ctx.alloc(x.shape)
        ctx.k.zk_toy_decay(x.ptr, y.ptr, ctx.state.ptr, ctx.state.shape[1], cache.state_offset // 4, ctx.q_start,
                           ctx.slot_of_req, ctx.R, self.spec.hidden_size, float(self.spec.decay), ctx.stream)
        return linear(ctx, y, self.w, ctx.alloc(x.shape))


register_part("mixer", "toy_decay_device", DeviceDecayMixer)
