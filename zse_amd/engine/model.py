"""A model: the parts a plan names, built, loaded and run in the plan's order."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

from .. import parts as _parts  # noqa: F401  (registers the built-in part kinds)
from ..config.plan import ModelPlan
from ..parts.base import PagedKV, Part, StateNeed, TensorReq, build_part, walk
from ..runtime.device import F32, Tensor


@dataclass
class CallCache:
    """What one entry of the execution order keeps between steps."""
    need: object = None              # PagedKV | StateNeed | None
    group: Optional[int] = None      # cache group of a paged need
    k: Optional[Tensor] = None       # [pages, kv heads, page size, head dim]
    v: Optional[Tensor] = None       # the same, or [pages, kv heads, head dim, page size]
    v_transposed: bool = False
    state_offset: int = 0            # byte offset inside a request's state slot
    state_bytes: int = 0


class Model:
    def __init__(self, plan: ModelPlan):
        self.plan = plan
        self.embedding = build_part("embedding", plan.embedding)
        self.blocks = [build_part("block", b) for b in plan.layers]
        self.final_norm = build_part("norm", plan.final_norm)
        self.head = build_part("head", plan.head)
        for i, call in enumerate(plan.order):
            if not (0 <= call.layer < len(self.blocks)):
                raise ValueError(f"order entry {i} names layer {call.layer}, which does not exist")
            if call.cache_of is not None and not (0 <= call.cache_of < i):
                raise ValueError(f"order entry {i} reads the cache of entry {call.cache_of}, "
                                 f"which does not run before it")
        self.loaded_dtype: Optional[str] = None
        self.tuned = True            # set at load: whether weights may sit in the tuned kernels' layouts

    def parts(self) -> List[Part]:
        out = []
        for top in [self.embedding] + self.blocks + [self.final_norm, self.head]:
            out.extend(walk(top))
        return out

    def tensor_reqs(self) -> List[TensorReq]:
        reqs = []
        for p in self.parts():
            reqs.extend(p.tensor_reqs())
        return reqs

    def load(self, weights, rt, dtype: str) -> None:
        for p in self.parts():
            p.load(weights, rt, dtype)
        self.loaded_dtype = dtype

    def cache_needs(self) -> List[object]:
        """Per entry of the order: what its mixer keeps (None for an entry that
        reads another entry's cache, or keeps nothing)."""
        out = []
        for call in self.plan.order:
            if call.cache_of is not None:
                out.append(None)
            else:
                out.append(self.blocks[call.layer].mixer.cache_need())
        return out

    # ---- what a step costs, for measurements: read off the parts, whatever the architecture
    def flops(self, portions, rows: int) -> float:
        """Flops of a step: ``portions`` is a list of (start, n) with n tokens of a request
        behind ``start`` cached ones, ``rows`` the number of logit rows asked for."""
        tokens = sum(n for _, n in portions)
        total = 0.0
        for call in self.plan.order:
            blk = self.blocks[call.layer]
            total += tokens * sum(p.flops_per_token() for p in walk(blk))
            mixer = getattr(blk, "mixer", None)
            need = mixer.cache_need() if mixer is not None else None
            if isinstance(need, PagedKV):
                for start, n in portions:
                    last = start + n          # keys the portion's last token sees, without a window
                    if need.window and last > need.window:
                        full = max(0, min(n, last - need.window))          # tokens that see a whole window
                        keys = full * need.window + sum(range(last - n + 1, last - full + 1))
                    else:
                        keys = sum(range(start + 1, last + 1))
                    total += mixer.flops_per_key() * keys
        return total + rows * self.head.flops_per_token()

    def cache_bytes_read(self, context: int, itemsize: int) -> int:
        """Bytes of cached keys and values that one token at position ``context - 1`` reads."""
        total = 0
        for need in self.cache_needs():
            if isinstance(need, PagedKV):
                seen = min(context, need.window) if need.window else context
                total += 2 * need.num_kv_heads * need.head_dim * seen * itemsize
        return total

    def forward(self, ctx, caches: List[CallCache], logit_rows, n_rows: int, logits: Tensor, pick=None):
        """Run the step's tokens through every entry of the order; write float
        logits of the rows ``logit_rows`` (device int32 pointer) into ``logits``.
        ``pick``: (ids, scratch) instead, for a step that wants nothing but each row's largest
        logit's column and whose head can give it without writing the logits (``head.can_pick``)."""
        h = self.embedding.forward(ctx)
        order = self.plan.order
        # the norm that opens a layer is computed by the kernel that closes the one before;
        # its output alternates between two buffers that outlive a layer's own
        T, H = h.shape
        handoff = [ctx.alloc((T, H)), ctx.alloc((T, H))]
        x = None
        base = ctx.arena.mark()
        for i, call in enumerate(order):
            cache = caches[call.cache_of if call.cache_of is not None else i]
            blk = self.blocks[call.layer]
            nxt = self.blocks[order[i + 1].layer] if i + 1 < len(order) else None
            if hasattr(blk, "entry_norm"):
                next_norm = nxt.entry_norm() if nxt is not None and hasattr(nxt, "entry_norm") else None
                x = blk.forward(ctx, h, cache, x_in=x, next_norm=next_norm, x_out=handoff[i % 2])
            else:
                blk.forward(ctx, h, cache)
                x = None
            ctx.arena.release(base)
        if n_rows:
            x = self.final_norm.forward(ctx, h, out_rows=(logit_rows, n_rows))
            if pick is not None:
                return self.head.pick(ctx, x, pick[0], pick[1])
            self.head.forward(ctx, x, logits)
        return logits
