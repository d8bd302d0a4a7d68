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
    graph_safe = True      # its launches take what changes from step to step from device memory alone

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

    def _join(self, ctx, sub: Tensor, post, h: Tensor, nxt, out: Tensor = None):
        """h += post(sub) (post None: h += sub); returns nxt(h) if nxt is given, written
        to ``out`` when the caller brings a buffer."""
        T, H = h.shape
        fused_post = post is None or isinstance(post, RMSNorm)
        fused_next = nxt is None or isinstance(nxt, RMSNorm)
        if not fused_post:
            sub, post = post.forward(ctx, sub), None
        if nxt is None or not fused_next:
            out = None
        elif out is None:
            out = ctx.alloc((T, H))
        ps = post.spec if post is not None else None
        ns = nxt.spec if (nxt is not None and fused_next) else None
        parts = sub.shape[0] if sub.layout == "parts" else 0     # partial sums of a product that split K
        ctx.k.zk_norm_add_norm(
            sub.ptr, parts, post.weight.ptr if post is not None else None, ps.eps if ps else 0.0,
            int(ps.unit_offset) if ps else 0, h.ptr,
            nxt.weight.ptr if ns else None, ns.eps if ns else 0.0, int(ns.unit_offset) if ns else 0,
            out.ptr if out is not None else None, T, H, ctx.stream)
        if nxt is not None and not fused_next:
            out = nxt.forward(ctx, h)
        return out

    @staticmethod
    def _joins_sums(post) -> bool:
        return post is None or isinstance(post, RMSNorm)

    def entry_norm(self):
        """The norm this block applies to the stream first; the block before may apply it
        for us in the kernel that ends its own work (see ``forward``)."""
        return self.norms["pre_mixer"]

    def forward(self, ctx, h: Tensor, cache, x_in: Tensor = None, next_norm=None, x_out: Tensor = None):
        """Update the stream ``h`` in place.  ``x_in``: this block's entry norm of ``h``,
        if the caller already has it.  ``next_norm``: the entry norm of whatever runs
        next; its output is returned (computed in the same kernel as the last
        residual sum), in ``x_out`` if given."""
        n = self.norms
        x = x_in if x_in is not None else n["pre_mixer"].forward(ctx, h)
        # the joining kernel adds up the partial sums of a part's last product itself
        ctx.sums_welcome = self.mixer if self._joins_sums(n.get("post_mixer")) else None
        a = self.mixer.forward(ctx, x, cache)
        x = self._join(ctx, a, n.get("post_mixer"), h, n["pre_ffn"])
        ctx.sums_welcome = self.ffn if self._joins_sums(n.get("post_ffn")) else None
        m = self.ffn.forward(ctx, x)
        ctx.sums_welcome = None
        if not isinstance(next_norm, RMSNorm):
            next_norm = None         # a norm the closing kernel does not know: the next block applies it
        return self._join(ctx, m, n.get("post_ffn"), h, next_norm, x_out)


register_part("block", "block", Block)
