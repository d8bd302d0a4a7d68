"""One layer: how a mixer and a feed-forward join the float residual stream.

"sandwich" is Gemma 2's order of four norms,
    h += post_m(mixer(pre_m(h)));  h += post_f(ffn(pre_f(h)))
the order of the reference's Gemma-family block (orchestrator/model_runner.py:425-439,
450-537).  "prenorm" leaves the post norms out (its Llama block, :1123-1297).  The
residual sum stays float throughout (orchestrator/vram_allocator.py:70-72).
"""
from __future__ import annotations

from ..runtime.device import Tensor
from .base import Part, build_part, register_part
from .norm import RMSNorm

ARRANGEMENTS = {"sandwich": ("pre_mixer", "post_mixer", "pre_ffn", "post_ffn"),
                "prenorm": ("pre_mixer", "pre_ffn")}


class Block(Part):
    def __init__(self, spec):
        if spec.arrangement not in ARRANGEMENTS:
            raise ValueError(f"arrangement must be one of {sorted(ARRANGEMENTS)}, got {spec.arrangement!r}")
        self.spec = spec
        roles = ARRANGEMENTS[spec.arrangement]
        missing = [r for r in roles if r not in spec.norms]
        if missing:
            raise ValueError(f"a {spec.arrangement} block needs norms {missing}")
        self.norms = {r: build_part("norm", spec.norms[r]) for r in roles}
        self.mixer = build_part("mixer", spec.mixer)
        self.ffn = build_part("ffn", spec.ffn)

    def children(self):
        return list(self.norms.values()) + [self.mixer, self.ffn]

    def _join(self, ctx, sub: Tensor, post, h: Tensor, nxt):
        """h += post(sub) (post None: h += sub); returns nxt(h) if nxt is given."""
        T, H = h.shape
        fused_post = post is None or isinstance(post, RMSNorm)
        fused_next = nxt is None or isinstance(nxt, RMSNorm)
        if not fused_post:
            sub, post = post.forward(ctx, sub), None
        out = ctx.alloc((T, H)) if (nxt is not None and fused_next) else None
        ps = post.spec if post is not None else None
        ns = nxt.spec if (nxt is not None and fused_next) else None
        ctx.k.zk_norm_add_norm(
            sub.ptr, post.weight.ptr if post is not None else None, ps.eps if ps else 0.0,
            int(ps.unit_offset) if ps else 0, h.ptr,
            nxt.weight.ptr if ns else None, ns.eps if ns else 0.0, int(ns.unit_offset) if ns else 0,
            out.ptr if out is not None else None, T, H, ctx.stream)
        if nxt is not None and not fused_next:
            out = nxt.forward(ctx, h)
        return out

    def forward(self, ctx, h: Tensor, cache) -> None:
        n = self.norms
        mark = ctx.arena.mark()
        x = n["pre_mixer"].forward(ctx, h)
        a = self.mixer.forward(ctx, x, cache)
        x = self._join(ctx, a, n.get("post_mixer"), h, n["pre_ffn"])
        m = self.ffn.forward(ctx, x)
        self._join(ctx, m, n.get("post_ffn"), h, None)
        ctx.arena.release(mark)


register_part("block", "block", Block)
