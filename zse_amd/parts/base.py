"""What every part is: a description-driven object with tensors and a forward.

A part is built from its spec alone (no device needed), says which checkpoint
tensors it wants (``tensor_reqs``), later binds them on the device (``load``)
and runs on the tokens of a step (``forward``).  No part knows which model it
belongs to.  Kinds are looked up in the registries below; a new kind is added
with ``register_part`` from anywhere, tests included.

Interfaces, by slot:

  norm      forward(ctx, x, out_rows=None) -> Tensor[rows, size] activations.
            ``x`` is the float residual stream or an activation tensor;
            ``out_rows`` (device int32 pointer, count) picks rows.
  position  rotary_tables() -> (inv_freq Tensor float32 [rotary_dim/2], rotary_dim)
            or None; apply(ctx, qkv, num_heads, num_kv_heads, head_dim) for an
            encoding that is not a rotation by position.
  mixer     cache_need() -> PagedKV | StateNeed | None;
            forward(ctx, x, cache) -> Tensor[T, hidden]
  ffn       forward(ctx, x) -> Tensor[T, hidden]
  block     forward(ctx, h, cache): updates the float stream ``h`` in place.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Tuple

ROLE_MATRIX = "matrix"   # used in matrix products: stored in the compute dtype
ROLE_GAIN = "gain"       # norm gains and other vectors: kept as float32


@dataclass(frozen=True)
class TensorReq:
    name: str
    shape: Tuple[int, ...]
    role: str = ROLE_MATRIX
    init_std: Optional[float] = None    # random-weights mode: None = the mode's default for the role


@dataclass(frozen=True)
class PagedKV:
    """The mixer keeps keys and values per token, in pages.  ``window``: only the
    last ``window`` positions are ever read again (None: all of them)."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int]


@dataclass(frozen=True)
class StateNeed:
    """The mixer keeps ``nbytes`` of state per request, whatever its length."""
    nbytes: int


class Part:
    spec = None
    # True: every launch of the part reads what differs between steps (tokens, positions, block
    # tables, slots) from device memory, so a captured decode step may be replayed.  A part that
    # looks at the step's host-side description (``ctx.entries``) leaves this False, and the
    # runner then runs every step eagerly.
    graph_safe = False

    def tensor_reqs(self) -> List[TensorReq]:
        return []

    def load(self, weights, rt, dtype: str) -> None:
        """Bind device tensors from a weight source (see zse_amd.weights.loader)."""

    def children(self) -> List["Part"]:
        return []

    def flops_per_token(self) -> float:
        """Multiply-adds x 2 that one token costs in this part's own matrices (children not
        counted): what measurements price a step with.  The default reads it off the matrices
        the part asks for; a part that uses only some of them for a token (routed experts), or
        none (a table that is gathered from), says so itself."""
        return float(sum(2 * r.shape[0] * r.shape[1] for r in self.tensor_reqs()
                         if r.role == ROLE_MATRIX and len(r.shape) == 2))

    def flops_per_key(self) -> float:
        """A mixer over cached keys: multiply-adds x 2 per (token, key it attends to)."""
        return 0.0

    def prepare(self, kernels, dtype: str, max_seqs: int, max_model_len: int, page_size: int,
                max_batch_tokens: int = 0) -> int:
        """Called once by the step runner, with its limits, before the first step.  A part
        fixes here whatever must not change from step to step, refuses limits its kernels
        cannot serve (with the numbers, at construction and not in the middle of a run) and
        returns the bytes of the runner's shared workspace its kernels need for one launch.
        ``max_batch_tokens``: the most tokens a step brings (0: not said); a part whose
        ``prepare`` does not take it is called without."""
        return 0


_REGISTRIES: Dict[str, Dict[str, Callable]] = {
    "norm": {}, "position": {}, "mixer": {}, "ffn": {}, "block": {}, "embedding": {}, "head": {},
}


def register_part(slot: str, kind: str, factory: Callable) -> None:
    """``factory(spec) -> Part``."""
    _REGISTRIES[slot][kind] = factory


def unregister_part(slot: str, kind: str) -> None:
    _REGISTRIES[slot].pop(kind, None)


def build_part(slot: str, spec) -> Part:
    reg = _REGISTRIES[slot]
    kind = getattr(spec, "kind", None)
    if kind not in reg:
        raise KeyError(f"no {slot} part of kind {kind!r}; registered: {sorted(reg)}")
    return reg[kind](spec)


def walk(part: Part):
    yield part
    for c in part.children():
        yield from walk(c)
