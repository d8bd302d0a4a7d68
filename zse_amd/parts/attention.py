"""Grouped-query softmax attention over the paged cache.

One forward for every kind of step: project q, k, v in one product, rotate q
and k and store k, v at each token's place in the cache, then let every token
attend to the cache alone, over the positions [max(0, pos - window + 1), pos]
(all earlier positions without a window).  The reference writes the cache
first as well (orchestrator/model_runner.py:1184-1194) but its prefill reads
contiguous K/V and never masks a window (orchestrator/kernels.py:883,
model_runner.py:489-490); its scale is fixed at 1/sqrt(head_dim)
(model_runner.py:80) where this part takes the scale and the soft cap as
parameters.  q, k, v stay separate products in the reference
(model_runner.py:1151-1165); here they are one.
"""
from __future__ import annotations

from typing import List

from ..runtime.device import BF16, Tensor
from .base import PagedKV, Part, TensorReq, build_part, register_part
from .ops import linear, tuned_gemm


class PagedAttention(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        s = self.spec = spec
        if s.num_heads % s.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if s.head_dim % 16 or s.head_dim > 256:
            raise ValueError(f"head_dim must be a multiple of 16 up to 256, got {s.head_dim}")
        self.position = build_part("position", s.position)
        self.shared_kv = "k" not in s.names        # reads another call's cache, writes none
        self.w_qkv = self.w_o = None
        self.decode_chunk = 64                     # keys a wave of the split decode attention takes

    def children(self):
        return [self.position]

    def tensor_reqs(self) -> List[TensorReq]:
        s = self.spec
        q = TensorReq(s.names["q"], (s.num_heads * s.head_dim, s.hidden_size))
        o = TensorReq(s.names["o"], (s.hidden_size, s.num_heads * s.head_dim))
        if self.shared_kv:
            return [q, o]
        kv = (s.num_kv_heads * s.head_dim, s.hidden_size)
        return [q, TensorReq(s.names["k"], kv), TensorReq(s.names["v"], kv), o]

    def load(self, weights, rt, dtype):
        s = self.spec
        names = [s.names["q"]] if self.shared_kv else [s.names[r] for r in ("q", "k", "v")]
        strip = getattr(weights, "wants_strip", None)
        self.w_qkv = weights.matrix(names, strip=True) if strip and strip(s.hidden_size) else weights.matrix(names)
        o_cols = s.num_heads * s.head_dim
        self.w_o = (weights.matrix([s.names["o"]], strip=True) if strip and strip(o_cols)
                    else weights.matrix([s.names["o"]]))

    def cache_need(self):
        s = self.spec
        return PagedKV(s.num_kv_heads, s.head_dim, s.window)

    def flops_per_key(self) -> float:
        return 4.0 * self.spec.num_heads * self.spec.head_dim        # q.k and p.v

    PORTION_RANGES_BYTES = 192 << 20

    def wants_v_transposed(self, kernels, dtype: str, page_size: int) -> bool:
        """The matrix-core kernel reads V as [page][kv head][hd][bs]."""
        s = self.spec
        return bool(dtype == BF16 and kernels.has("zk_attention_bf16") and
                    kernels.zk_attention_bf16_supports(s.num_heads, s.num_kv_heads, s.head_dim, page_size))

    def prepare(self, kernels, dtype, max_seqs, max_model_len, page_size, max_batch_tokens=0) -> int:
        """Workspace of the split attention of decoded tokens at the runner's limits, and the
        number of keys a wave of it takes.  That number fixes where the sums over keys are cut:
        it follows from the limits alone, never from a step's batch, so a request's result does
        not depend on who shares its step."""
        s = self.spec
        if not self.wants_v_transposed(kernels, dtype, page_size):
            return 0
        chunks = -(-int(max_model_len) // 64)
        self.decode_chunk = 32 if int(max_seqs) * s.num_kv_heads * chunks <= 512 else 64
        longest = int(kernels.zk_attention_bf16_max_context(s.num_heads, s.num_kv_heads, s.head_dim,
                                                            self.decode_chunk))
        if max_model_len > longest:
            raise ValueError(f"attention with {s.num_heads} heads, {s.num_kv_heads} KV heads of "
                             f"{s.head_dim}: the longest context its decode kernel takes is {longest} "
                             f"tokens, the runner asks for {max_model_len}")
        need = int(kernels.zk_attention_bf16_workspace(int(max_seqs), s.num_heads, s.head_dim, int(max_model_len)))
        # room for a launch of few, long portions to cut its keys into ranges: as much as a step's
        # tokens can ask for, but no more than PORTION_RANGES_BYTES (a launch that would need more
        # has blocks enough without the ranges, or runs on the kernels that need no workspace)
        if max_batch_tokens > 0 and kernels.has("zk_attention_bf16_portion_workspace"):
            extra = int(kernels.zk_attention_bf16_portion_workspace(int(max_batch_tokens), s.num_heads, s.num_kv_heads,
                                                                    s.head_dim))
            need = (need + 255) // 256 * 256 + min(extra, self.PORTION_RANGES_BYTES)
        return need

    def between_product_and_rotation(self, ctx, qkv: Tensor) -> None:
        """A mixer that differs from this one only in what it does to queries and keys before
        they are rotated and stored (a norm over each head, say) overrides this and changes
        ``qkv`` in place: rows are tokens, a row holds the query heads, then the key heads, then
        the value heads (the last two absent in a mixer that reads another entry's cache), each
        ``head_dim`` wide.  Everything else of the mixer stays as it is; the product that
        rotates and stores its own results is then not used, since this step lies in between."""

    def forward(self, ctx, x: Tensor, cache) -> Tensor:
        s, k = self.spec, ctx.k
        T = x.shape[0]
        nh, nkv, hd = s.num_heads, s.num_kv_heads, s.head_dim
        n_store = 0 if self.shared_kv else nkv
        width = (nh + 2 * n_store) * hd
        g = ctx.group(cache.group)
        tables = self.position.rotary_tables()
        hooked = type(self).between_product_and_rotation is not PagedAttention.between_product_and_rotation
        if (not hooked and tables is not None and tuned_gemm(ctx, s.hidden_size) and k.has("zk_qkv_rope_bf16")
                and k.zk_qkv_rope_bf16_supports(T, s.hidden_size, hd, tables[1])):
            # few decoded tokens: the product rotates and stores its own results
            qkv = ctx.alloc((T, width))
            k.zk_qkv_rope_bf16(x.ptr, s.hidden_size, self.w_qkv.ptr, qkv.ptr, width, T, s.hidden_size,
                               1 if self.w_qkv.layout == "strip" else 0, ctx.positions,
                               None if self.shared_kv else g.slot_map, tables[0].ptr, cache.k.ptr,
                               cache.v.ptr, nh, n_store, hd, g.page_size, 1 if cache.v_transposed else 0,
                               ctx.stream)
        else:
            # a product that splits K may leave the adding up of its partial sums to the kernel
            # that rotates and stores, unless something has to look at the rows in between
            direct = not hooked and tables is not None and k.has("zk_rope_cache_write_sums")
            qkv = ctx.alloc((T, width))
            got = linear(ctx, x, self.w_qkv, qkv, sums_ok=direct)
            if hooked:
                self.between_product_and_rotation(ctx, qkv)
            if tables is None:
                self.position.apply(ctx, qkv, nh, n_store, hd)
                inv_freq, rotary_dim = 0, 0
            else:
                inv_freq, rotary_dim = tables[0].ptr, tables[1]
            args = (ctx.positions, None if self.shared_kv else g.slot_map, inv_freq or None, rotary_dim, cache.k.ptr,
                    cache.v.ptr, T, nh, n_store, hd, g.page_size, 1 if cache.v_transposed else 0, ctx.stream)
            if got.layout == "parts":
                k.zk_rope_cache_write_sums(qkv.ptr, got.ptr, got.shape[0], *args)
            else:
                k.zk_rope_cache_write(qkv.ptr, *args)
        o = ctx.alloc((T, nh * hd))
        cap = float(s.softcap) if s.softcap else 0.0
        win = int(s.window) if s.window else 0
        if cache.v_transposed and ctx.tuned:
            # the matrix-core kernel; requests with more than one token come first in the batch
            k.zk_attention_bf16(qkv.ptr, width, cache.k.ptr, cache.v.ptr, g.block_table, g.max_blocks,
                                ctx.q_start, ctx.ctx_len, o.ptr, ctx.R, ctx.n_multi, ctx.max_q_len,
                                ctx.max_ctx, nh, nkv, hd, g.page_size, s.scale, cap, win,
                                self.decode_chunk, ctx.workspace.ptr, ctx.workspace.nbytes, ctx.stream)
        else:
            k.zk_attention_plain(qkv.ptr, width, cache.k.ptr, cache.v.ptr, g.block_table,
                                 g.max_blocks, ctx.req_of_token, ctx.positions, o.ptr, T, nh, nkv,
                                 hd, g.page_size, s.scale, cap, win, 1 if cache.v_transposed else 0,
                                 ctx.stream)
        return linear(ctx, o, self.w_o, ctx.alloc((T, s.hidden_size)), last_of=self)


register_part("mixer", "attention", PagedAttention)
