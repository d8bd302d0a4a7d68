"""The step function: one batch of (request, its next tokens) through the model.

``StepRunner.step(entries)`` takes, for each request, the tokens that follow
what it already has in the cache: a portion of a prompt of any length beside
single decoded tokens, cut anywhere.  All entries run as one batch: tokens are
laid out flat, each with its position, its request and, per cache group, the
place in the pages where its key and value go; attention then reads the cache
alone.  Logits come back for the places that were asked for.

The reference has three disjoint calls instead (a whole new prompt, M
sequences of one token, K tokens of one sequence: orchestrator/model_runner.py:290,
843, 761), rebuilds and uploads tokens, positions, packed block tables and
lengths for each (model_runner.py:873-884), and cannot continue a prompt
(cache/page_table.py:58-59).  Decode steps of a fixed shape are captured into a
HIP graph per batch size as there (model_runner.py:1806-1932).
"""
from __future__ import annotations

import ctypes
import inspect
import warnings

import weakref
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from ..cache.manager import CacheManager, GroupInfo, group_needs
from ..cache.pages import OutOfPages
from ..parts.base import PagedKV, StateNeed
from ..runtime.device import BF16, F32, I32, ITEMSIZE, Runtime, Tensor, canonical_dtype
from .model import CallCache, Model


@dataclass
class StepEntry:
    req: object                      # request id
    tokens: Sequence[int]            # its next tokens
    want: Sequence[int] = ()         # places among these tokens whose logits are wanted


@dataclass
class GroupView:
    block_table: int                 # device pointer, int32 [R, max_blocks]
    max_blocks: int
    slot_map: int                    # device pointer, int32 [T]
    page_size: int


class Arena:
    """Bump allocator over device memory for a step's activations.  It grows by
    whole chunks when a step needs more and keeps them; ``mark``/``release``
    give a layer's buffers back for the next layer."""

    ALIGN = 256

    def __init__(self, rt: Runtime, chunk_bytes: int = 64 << 20):
        self.rt = rt
        self.chunk_bytes = chunk_bytes
        self.chunks: List[Tensor] = []
        self.cur = 0          # chunk index
        self.off = 0
        self.frozen = False   # no growth while a graph is being captured

    def reset(self):
        self.cur, self.off = 0, 0

    def mark(self):
        return (self.cur, self.off)

    def release(self, m):
        self.cur, self.off = m

    def alloc(self, shape, dtype: str) -> Tensor:
        n = ITEMSIZE[dtype]
        for s in shape:
            n *= int(s)
        n = (max(n, 1) + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        while True:
            if self.cur < len(self.chunks) and self.off + n <= self.chunks[self.cur].nbytes:
                t = Tensor(self.chunks[self.cur].ptr + self.off, shape, dtype, self.chunks[self.cur].owner)
                self.off += n
                return t
            if self.cur + 1 < len(self.chunks):
                self.cur += 1
                self.off = 0
                continue
            if self.frozen:
                raise RuntimeError("activation arena would grow during graph capture")
            self.chunks.append(self._new_chunk(max(n, self.chunk_bytes)))
            self.cur = len(self.chunks) - 1
            self.off = 0

    def _new_chunk(self, nbytes: int) -> Tensor:
        return self.rt.empty(((nbytes + 3) // 4,), F32)


class StepContext:
    """What parts see of a step."""

    def __init__(self, runner: "StepRunner"):
        self.runner = runner
        self.rt = runner.rt
        self.k = runner.k
        self.dtype = runner.dtype
        self.tuned = runner.tuned
        self.stream = runner.rt.stream
        self.arena = runner.arena
        self.workspace = runner.workspace
        self.gemm_workspace = runner.gemm_workspace
        self.T = 0
        self.R = 0
        self.tokens = self.positions = self.req_of_token = self.q_start = self.ctx_len = 0
        self.slot_of_req = 0
        self.groups: List[GroupView] = []
        self.max_q_len = 0
        self.max_ctx = 0
        self.n_multi = 0             # requests [0, n_multi) of the batch bring more than one token
        self.entries: List[Tuple[object, int, int, int]] = []   # (req, slot, start, n) on the host
        self.state = None            # Tensor uint8-as-float32 words [max_seqs, slot_words] or None
        self.slot_bytes = 0

    def alloc(self, shape, dtype: Optional[str] = None) -> Tensor:
        return self.arena.alloc(shape, dtype or self.dtype)

    def group(self, gid: int) -> GroupView:
        return self.groups[gid]


class StepRunner:
    def __init__(self, model: Model, rt: Runtime, dtype: str, page_size: int = 16,
                 num_pages: Optional[int] = None, cache_tokens: Optional[int] = None,
                 max_seqs: int = 64, max_batch_tokens: int = 4096, max_model_len: Optional[int] = None,
                 tuned: Optional[bool] = None, use_graphs: bool = True, use_steplists: bool = True,
                 graph_max_batch: int = 16):
        self.model, self.rt = model, rt
        self.dtype = canonical_dtype(dtype)
        if model.loaded_dtype != self.dtype:
            raise ValueError(f"the model's weights are {model.loaded_dtype}, the runner wants {self.dtype}")
        self.k = rt.kernels(self.dtype)
        model_tuned = bool(getattr(model, "tuned", True))
        if tuned is not None and bool(tuned) != model_tuned:
            raise ValueError(f"the model was loaded with tuned={model_tuned}; the runner cannot run it with tuned={tuned}")
        self.tuned = model_tuned
        self.use_graphs = bool(use_graphs) and self.tuned
        # Decode steps of more requests than this are launched from their launch lists instead:
        # a graph is captured for a padded batch and the longest context it covers, and with
        # many requests of uneven lengths its attention grids are mostly blocks that end at
        # once, while a step of that size runs long enough to hide the launches of the next
        # (192 requests, 64 live, 2B shapes: 51.1 -> 54.1 k tokens a second without graphs;
        # steps of 1 to 16 requests of equal length take the same time either way).
        self.graph_max_batch = int(graph_max_batch)
        self.page_size = int(page_size)
        self.max_seqs = int(max_seqs)
        self.max_batch_tokens = int(max_batch_tokens)
        self.max_model_len = int(max_model_len or model.plan.max_position)
        self.vocab = model.plan.vocab_size

        # ---- cache layout
        needs = model.cache_needs()
        groups = group_needs(needs)
        if num_pages is None:
            tokens = cache_tokens if cache_tokens is not None else self.max_model_len
            num_pages = -(-int(tokens) // self.page_size)
        # one number for every group, or one per group in the groups' order (windowed groups
        # first, by window; the all-keys group last): a windowed group never holds more than
        # its window and a step's tokens per request, so its pool can be much the smaller
        per_group = list(num_pages) if isinstance(num_pages, (list, tuple)) else [num_pages] * len(groups)
        if len(per_group) != len(groups):
            raise ValueError(f"{len(per_group)} page counts for {len(groups)} cache groups")
        for g, n in zip(groups, per_group):
            g.num_pages = int(n)
        slot_bytes = 0
        self.caches: List[CallCache] = []
        gid_of = {}
        for gid, g in enumerate(groups):
            for c in g.calls:
                gid_of[c] = gid
        item = ITEMSIZE[self.dtype]
        for i, need in enumerate(needs):
            cc = CallCache(need=need)
            if isinstance(need, PagedKV):
                cc.group = gid_of[i]
                # page 0 of every slab is the runner's own: cleared here, never handed out and
                # never written, it is what kernels read where a table names no page
                pages = groups[cc.group].num_pages + 1
                shape = (pages, need.num_kv_heads, self.page_size, need.head_dim)
                cc.k = rt.zeros(shape, self.dtype)
                mixer = model.blocks[model.plan.order[i].layer].mixer
                cc.v_transposed = bool(self.tuned and getattr(mixer, "wants_v_transposed", None) and
                                       mixer.wants_v_transposed(self.k, self.dtype, self.page_size))
                if cc.v_transposed:
                    shape = (pages, need.num_kv_heads, need.head_dim, self.page_size)
                cc.v = rt.zeros(shape, self.dtype)
            elif isinstance(need, StateNeed):
                cc.state_offset = slot_bytes
                cc.state_bytes = int(need.nbytes)
                slot_bytes += (int(need.nbytes) + 15) // 16 * 16
            self.caches.append(cc)
        self.slot_bytes = slot_bytes
        self.manager = CacheManager(groups, self.page_size, self.max_seqs, self.max_model_len, slot_bytes,
                                    first_page=1)
        # per group: the base addresses and page sizes of its layers' slabs, for the kernel that
        # clears a page in all of them
        self._slabs = []
        for gid in range(len(groups)):
            ts = [t for cc in self.caches if cc.group == gid and cc.k is not None for t in (cc.k, cc.v)]
            ptrs = rt.upload(np.array([t.ptr for t in ts], dtype=np.uint64).view(np.float64), "float64")
            sizes = rt.upload(np.array([t.nbytes // t.shape[0] for t in ts], dtype=np.uint64).view(np.float64), "float64")
            self._slabs.append((ptrs, sizes, len(ts)))
        self.state = rt.zeros((self.max_seqs, max(slot_bytes // 4, 1)), F32) if slot_bytes else None
        # the manager tells us of every admission; a weak reference, so that runner and manager
        # do not hold each other (a runner dropped by its owner frees its memory at once)
        me = weakref.ref(self)
        self.manager.on_admit = lambda req, slot: me() is not None and me()._clear_slot(req, slot)

        # ---- step buffers
        self.arena = Arena(rt)
        # one workspace for every part's kernels (a launch at a time uses it): each part says
        # what it needs at this runner's limits, and refuses limits it cannot serve, here
        need = 0
        for part in model.parts():
            limits = (self.k, self.dtype, self.max_seqs, self.max_model_len, self.page_size)
            if "max_batch_tokens" in inspect.signature(part.prepare).parameters:
                need = max(need, int(part.prepare(*limits, max_batch_tokens=self.max_batch_tokens)))
            else:
                need = max(need, int(part.prepare(*limits)))
        try:
            self.workspace = rt.zeros((max(need // 4 + 1, 64),), F32)
        except Exception as e:
            raise RuntimeError(f"the kernels' workspace for {self.max_seqs} requests of up to "
                               f"{self.max_model_len} tokens needs {need} bytes and cannot be "
                               f"allocated: {e}") from None
        self.gemm_workspace = None
        if self.dtype == BF16 and self.k.has("zk_gemm_bf16_workspace"):
            self.gemm_workspace = rt.zeros((self.k.zk_gemm_bf16_workspace() // 4,), F32)
        G = len(groups)
        self.max_blocks = self.manager.max_blocks
        cap = self._meta_words(self.max_batch_tokens, self.max_seqs, G)
        self.meta_host = rt.pinned(cap * 4)
        self.meta_dev = rt.empty((cap,), I32)
        self.meta_copied = rt.event()
        rt.record(self.meta_copied)
        self.logits: Optional[Tensor] = None
        self.graphs: Dict[object, object] = {}   # bucket -> "warm"; (bucket, context covered) -> graph handle
        # a captured step replays the same launches with the same arguments: every part must
        # take what changes from step to step (tokens, positions, tables, slots) from device
        # memory alone.  The built-in parts do; a part says so with ``graph_safe = True``.
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in model.parts())
        # Eager steps (prompt portions, mixed batches): the first step of a shape runs call by
        # call and its launches are written down on the native side; later steps of that shape
        # are launched from there with one call (zk_steplist_run).  The same condition as for
        # graphs: what differs between steps of one shape must come from device memory.
        self.use_steplists = bool(use_steplists) and self.graph_safe
        self.steplists: Dict[tuple, int] = {}        # shape of a step -> handle of its launch list, least recently used first
        self._sighted: Dict[tuple, None] = {}        # shapes met once and not written down yet
        self.steplist_runs = 0                       # eager steps launched from a list
        self.steplist_misses = 0                     # eager steps launched call by call from Python
        self.graph_runs = 0                          # decode steps replayed from a captured graph
        self.graph_logits: Optional[Tensor] = None
        self.steps_run = 0
        # a step that wants nothing but each row's largest logit's column (``step(pick=True)``):
        # the ids' buffer and the scratch memory of the head's picking product, made on first use
        self.pick_ids: Optional[Tensor] = None
        self.pick_scratch: Optional[Tensor] = None
        self._head_picks: Dict[int, bool] = {}       # rows -> whether the head picks for that many

    # ------------------------------------------------------------------ sizes
    def _meta_words(self, T: int, R: int, G: int) -> int:
        return 4 * T + (R + 1) + 4 * R + G * (T + R * self.max_blocks) + 64

    def cache_bytes(self) -> int:
        return sum(c.k.nbytes + c.v.nbytes for c in self.caches if c.k is not None)

    # ------------------------------------------------------------------ requests
    def _clear_slot(self, req, slot: int) -> None:
        """A request became live (the manager calls this, whoever admitted it): its state slot
        starts from zero.  The clearing kernel runs on the runner's stream, after the steps
        that the slot's last owner took part in and before the first step of the new one."""
        if self.state is not None:
            self.rt.zero_(self.state.rows(slot, slot + 1))

    def add(self, req) -> int:
        return self.manager.add(req)

    def _clear_untouched(self, entries) -> None:
        """A page that a request begins to fill in this step without filling it still holds, in
        the places behind the request's last token, what the page's last owner left there.  The
        attention kernels read whole tiles of keys and values and mask afterwards; a masked
        value takes part in a matrix product with weight 0, and 0 x NaN is NaN.  So such a page is
        cleared before the step writes to it: whatever a request's table names then holds the
        request's own values or zeros, and nothing another request computed can reach it."""
        m = self.manager
        for g in range(len(m.groups)):
            pages = []
            for e in entries:
                p = m.untouched_page(e.req, g, m.computed(e.req) + len(e.tokens))
                if p is not None:
                    pages.append(p)
            if pages:
                ptrs, sizes, n = self._slabs[g]
                arr = (ctypes.c_int * len(pages))(*pages)
                self.k.zk_zero_pages(ptrs.ptr, sizes.ptr, n, arr, len(pages), self.rt.stream)

    def finish(self, req) -> None:
        self.manager.release(req)

    # ------------------------------------------------------------------ the step
    def _pack(self, entries: Sequence[StepEntry], T_pad: int, R_pad: int, feed: Optional[Sequence[int]] = None):
        """Fill the pinned host buffer; returns offsets (in words) and counts.  ``feed``: per
        entry the place among the last step's ids that holds its token, or -1; the pairs
        (place of the token in this step, place of the id) go to the device with the rest and
        ``self._fed`` says how many they are."""
        m, ps = self.manager, self.page_size
        G = len(m.groups)
        T = sum(len(e.tokens) for e in entries)
        R = len(entries)
        off = {}
        cur = 0

        def take(name, n):
            nonlocal cur
            off[name] = cur
            cur += n
            return self.meta_host.array(off[name] * 4, n, np.int32)

        tokens = take("tokens", T_pad)
        positions = take("positions", T_pad)
        req_of_token = take("req_of_token", T_pad)
        logit_rows = take("logit_rows", T_pad)
        q_start = take("q_start", R_pad + 1)
        ctx_len = take("ctx_len", R_pad)
        slot_of_req = take("slot_of_req", R_pad)
        feed_dst = take("feed_dst", R_pad)
        feed_src = take("feed_src", R_pad)
        slot_maps = [take(f"slot_map{g}", T_pad) for g in range(G)]
        tables = [take(f"table{g}", R_pad * self.max_blocks).reshape(R_pad, self.max_blocks)
                  for g in range(G)]
        tokens[T:] = 0
        positions[T:] = -1
        req_of_token[T:] = 0
        for sm in slot_maps:
            sm[T:] = -1
        # requests that bring more than one token come first: the attention kernels
        # treat the two kinds apart; logits still come back in the order of the entries
        order = sorted(range(R), key=lambda i: len(entries[i].tokens) == 1)
        n_multi = sum(1 for e in entries if len(e.tokens) > 1)
        t = 0
        host_entries = []
        first_token = [0] * R
        max_q = max_ctx = 0
        for r, i in enumerate(order):
            e = entries[i]
            n = len(e.tokens)
            start = m.computed(e.req)
            if n == 1:          # a decoded token: numbers, no arrays
                tokens[t] = e.tokens[0]
                positions[t] = start
                req_of_token[t] = r
                for g in range(G):
                    slot_maps[g][t] = m.slot_of(e.req, g, start)
            else:
                tokens[t:t + n] = np.asarray(e.tokens, dtype=np.int32)
                positions[t:t + n] = np.arange(start, start + n, dtype=np.int32)
                req_of_token[t:t + n] = r
                for g in range(G):
                    slot_maps[g][t:t + n] = m.slot_mapping(e.req, g, start, n)
            q_start[r] = t
            ctx_len[r] = start + n
            slot_of_req[r] = m.slot(e.req)
            for g in range(G):
                m.fill_table_row(e.req, g, tables[g][r])
            first_token[i] = t
            host_entries.append((e.req, m.slot(e.req), start, n))
            max_q, max_ctx = max(max_q, n), max(max_ctx, start + n)
            t += n
        # The two maxima only size the attention kernels' grids (a block past a request's own
        # rows or keys ends at once); rounded up, steps of many lengths share one launch list.
        if max_q > 1:
            max_q = -(-max_q // 32) * 32
        max_ctx = min(-(-max_ctx // 256) * 256, max(self.max_model_len, max_ctx))
        n_rows = 0
        for i, e in enumerate(entries):
            for w in e.want:
                if not (0 <= w < len(e.tokens)):
                    raise ValueError(f"request {e.req!r}: wanted place {w} is not among its "
                                     f"{len(e.tokens)} tokens")
                logit_rows[n_rows] = first_token[i] + w
                n_rows += 1
        self._fed = 0
        if feed is not None:
            for i, src in enumerate(feed):
                if src >= 0:
                    feed_dst[self._fed] = first_token[i]
                    feed_src[self._fed] = src
                    self._fed += 1
        q_start[R:] = T
        ctx_len[R:] = 0
        slot_of_req[R:] = 0
        for g in range(G):
            tables[g][R:] = -1
        return off, cur, T, R, n_rows, host_entries, max_q, max_ctx, n_multi

    def _context(self, off, T_pad, R_pad, host_entries, max_q, max_ctx, n_multi) -> StepContext:
        ctx = StepContext(self)
        base = self.meta_dev.ptr
        p = lambda name: base + off[name] * 4
        ctx.T, ctx.R = T_pad, R_pad
        ctx.tokens, ctx.positions, ctx.req_of_token = p("tokens"), p("positions"), p("req_of_token")
        ctx.q_start, ctx.ctx_len, ctx.slot_of_req = p("q_start"), p("ctx_len"), p("slot_of_req")
        ctx.logit_rows = p("logit_rows")
        ctx.groups = [GroupView(p(f"table{g}"), self.max_blocks, p(f"slot_map{g}"), self.page_size)
                      for g in range(len(self.manager.groups))]
        ctx.entries = host_entries
        ctx.max_q_len, ctx.max_ctx, ctx.n_multi = max_q, max_ctx, n_multi
        ctx.state, ctx.slot_bytes = self.state, self.slot_bytes
        return ctx

    def _ensure_logits(self, rows: int):
        if self.logits is None or self.logits.shape[0] < rows:
            self.rt.sync()
            self.logits = None
            self.logits = self.rt.empty((max(rows, 8), self.vocab), F32)

    # ------------------------------------------------------------------ picking instead of logits
    def _pick_buffers(self, rows: int):
        """(ids, scratch) if the model's head picks for ``rows`` rows without writing logits,
        else None (the step then writes logits and the argmax kernel reads them)."""
        head = self.model.head
        if self.pick_ids is None or self.pick_ids.shape[0] < rows:
            # room for the ids of every wanted row (a step may want more rows than it has requests)
            self.rt.sync()
            room = max(rows, self.max_seqs, 8)
            self.pick_ids = self.rt.empty((room,), I32)
            self.argmax_scratch = self.rt.empty((room * 64 * 2,), F32)
        if not hasattr(head, "can_pick"):
            return None
        if rows not in self._head_picks:
            self._head_picks[rows] = bool(head.can_pick(StepContext(self), rows))
        if not self._head_picks[rows]:
            return None
        if self.pick_scratch is None:
            most = min(self.pick_ids.shape[0], head.PICK_ROWS)
            self.pick_scratch = self.rt.empty(((head.pick_scratch_bytes(self.k, most) + 3) // 4,), F32)
        return (self.pick_ids, self.pick_scratch)

    def _argmax_of(self, logits: Tensor, n_rows: int) -> Tensor:
        self.k.zk_argmax(logits.ptr, self.pick_ids.ptr, n_rows, self.vocab, self.argmax_scratch.ptr, self.rt.stream)
        return self.pick_ids.rows(0, n_rows)

    # ------------------------------------------------------------------ graphs for decode steps
    def _graph_bucket(self, entries) -> int:
        """The padded batch size under which a decode-only step replays a captured graph
        (0: run eagerly).  Every entry brings one token and wants its logits."""
        if not self.use_graphs or not self.graph_safe:
            return 0
        if len(entries) > self.graph_max_batch:
            return 0
        if any(len(e.tokens) != 1 or list(e.want) != [0] for e in entries):
            return 0
        b = 1
        while b < len(entries):
            b *= 2
        return b if b <= self.max_seqs else 0

    def _feed(self, off, tokens_from: Optional[int], R: int, identity: bool) -> None:
        """After the step's arrays have been sent: the tokens that come from the last step's ids."""
        if tokens_from is None:
            return
        if identity:
            self.rt.copy_d2d(self.meta_dev.ptr + off["tokens"] * 4, tokens_from, R * 4)
        elif self._fed:
            base = self.meta_dev.ptr
            self.k.zk_feed_tokens(base + off["tokens"] * 4, tokens_from, base + off["feed_dst"] * 4,
                                  base + off["feed_src"] * 4, self._fed, self.rt.stream)

    def _graph_step(self, entries, bucket: int, tokens_from=None, pick=False, feed=None):
        """One token for each request through a graph of this bucket.  The first step of
        a bucket runs eagerly (it sizes the arena), later ones are captured and replayed.
        Kernel arguments are fixed by the graph: rows beyond the batch are padding (position
        -1, no cache slot, no request), the logits land in a buffer of the graphs' own, and
        attention covers a context length that is a step of an eighth of the longest the runner
        allows (of 1,024 tokens at least), the first that holds the step's longest request: a
        bucket has a graph for each such length it has met.  (The length only sizes the
        attention kernels' grids; a block past a request's keys ends at once, but a grid of
        mostly such blocks still costs time.)"""
        R = len(entries)
        off, words, T, _, n_rows, host_entries, _, longest, _ = self._pack(entries, bucket, bucket, feed)
        grain = 1024
        while grain * 8 < self.max_model_len:
            grain *= 2
        covered = min(-(-longest // grain) * grain, max(self.max_model_len, longest))
        logit_rows = self.meta_host.array(off["logit_rows"] * 4, bucket, np.int32)
        logit_rows[n_rows:] = 0
        self.rt.copy_h2d_async(self.meta_dev.ptr, self.meta_host.ptr, words * 4)
        self.rt.record(self.meta_copied)
        self._feed(off, tokens_from, R, feed is None)
        picks = self._pick_buffers(bucket) if pick else None
        if self.graph_logits is None and picks is None:
            self.graph_logits = self.rt.empty((self.max_seqs, self.vocab), F32)
        out = self.graph_logits.rows(0, bucket) if picks is None else None

        def result():
            if picks is not None:
                return self.pick_ids.rows(0, n_rows)
            return self._argmax_of(self.graph_logits.rows(0, n_rows), n_rows) if pick else self.graph_logits.rows(0, n_rows)
        # a graph that picks holds other launches than one that writes logits: a key of its own
        mode = "pick" if picks is not None else "logits"
        graph = self.graphs.get((bucket, covered) if mode == "logits" else (bucket, covered, mode))
        if graph is not None:
            self.rt.graph_launch(graph)
            self.graph_runs += 1
            return result()
        ctx = self._context(off, bucket, bucket, host_entries, 1, covered, 0)
        self.arena.reset()
        warm = bucket if mode == "logits" else (bucket, mode)
        if warm not in self.graphs:             # first time: eager, lets the arena grow
            self.model.forward(ctx, self.caches, ctx.logit_rows, bucket, out, pick=picks)
            self.graphs[warm] = "warm"
            return result()
        self.arena.frozen = True
        try:
            self.rt.capture_begin()
            try:
                self.model.forward(ctx, self.caches, ctx.logit_rows, bucket, out, pick=picks)
            finally:
                graph = self.rt.capture_end()
        finally:
            self.arena.frozen = False
        self.graphs[(bucket, covered) if mode == "logits" else (bucket, covered, mode)] = graph
        self.rt.graph_launch(graph)
        return result()

    def close(self) -> None:
        """Gives back what lives outside the runtime's memory pools: the captured graphs and
        the launch lists.  The runner takes no step after this."""
        self.rt.sync()
        for key, g in list(self.graphs.items()):
            if isinstance(g, int):
                self.rt.graph_destroy(g)
        self.graphs.clear()
        for h in self.steplists.values():
            self.k.steplist_destroy(h)
        self.steplists.clear()

    MAX_STEPLISTS = 256
    MAX_SIGHTED = 4096

    def _forward(self, ctx, n_rows: int, out: Optional[Tensor], shape: tuple, pick=None) -> None:
        """The model on an eager step.  Device addresses follow from the step's shape (the
        arena hands out the same addresses for the same sequence of sizes, the step's arrays
        lie at offsets fixed by the numbers of tokens and requests), so a shape that was seen
        before is launched from its written-down list.  A step of single tokens is written down
        at once (its shape comes back as long as the same requests decode); any other shape
        when it comes a second time (a mixed step's shape often never comes back, and writing
        costs as much again as the launches).  Of 256 lists the one not used for the longest
        time makes room for a new one, so the shapes that keep coming stay."""
        if not self.use_steplists:
            self.model.forward(ctx, self.caches, ctx.logit_rows, n_rows, out, pick=pick)
            self.steplist_misses += 1
            return
        handle = self.steplists.pop(shape, None)
        if handle is not None:
            self.steplists[shape] = handle           # the most recently used one is the last
            self.k.steplist_run(handle, ctx.stream)
            self.steplist_runs += 1
            return
        self.steplist_misses += 1
        if shape[0] != shape[1] and shape not in self._sighted:          # more tokens than requests: not a decode step
            if len(self._sighted) >= self.MAX_SIGHTED:
                self._sighted.pop(next(iter(self._sighted)))
            self._sighted[shape] = None
            self.model.forward(ctx, self.caches, ctx.logit_rows, n_rows, out, pick=pick)
            return
        self._sighted.pop(shape, None)
        self.k.steplist_begin()
        try:
            self.model.forward(ctx, self.caches, ctx.logit_rows, n_rows, out, pick=pick)
        except BaseException:
            h = self.k.steplist_end()
            if h is not None:
                self.k.steplist_destroy(h)
            raise
        handle = self.k.steplist_end()
        if handle is None:
            # some part launches what the native side cannot repeat: every step of this runner is
            # launched call by call from now on, and the reason is said, once
            self.use_steplists = False
            warnings.warn(f"launch lists are off for this runner: {self.k.not_written or 'an entry point'} "
                          f"is not among the calls that can be written down (see register_kernels)",
                          RuntimeWarning, stacklevel=2)
            return
        if len(self.steplists) >= self.MAX_STEPLISTS:
            old = next(iter(self.steplists))
            self.k.steplist_destroy(self.steplists.pop(old))
        self.steplists[shape] = handle

    def step(self, entries: Sequence[StepEntry], download: bool = True, tokens_from: Optional[int] = None,
             pick: bool = False, feed: Optional[Sequence[int]] = None):
        """Run one step.  Returns float32 logits [wanted, vocab] on the host
        (``download=False``: the device tensor, valid until the next step).
        ``pick``: the step wants nothing but the greedy choice of every wanted row; what comes
        back is int32 ids [wanted] instead (the lowest index among a row's largest logits).
        Where the model's head can, the ids are taken in the head product's epilogue and the
        logits never reach memory; elsewhere they are written and an argmax kernel reads them.
        ``tokens_from``: a device pointer to int32 token ids, one per entry in the order of the
        entries, for a step in which every entry brings one token: the ids the last step's
        sampling kernel left on the device are fed without a trip to the host (the entries'
        own token values are then placeholders).  ``feed``: with ``tokens_from``, for any step:
        per entry the place among those ids that holds the entry's token (the entry then
        brings one token, a placeholder), or -1 for an entry that brings its tokens itself."""
        if feed is not None:
            if tokens_from is None or len(feed) != len(entries):
                raise ValueError("feed names a place among the ids at tokens_from for every entry, or -1")
            for e, src in zip(entries, feed):
                if src >= 0 and len(e.tokens) != 1:
                    raise ValueError(f"request {e.req!r}: a token fed on the device is one token")
        entries = [e for e in entries if len(e.tokens) > 0]
        if not entries:
            if pick:
                return np.zeros((0,), np.int32) if download else None
            return np.zeros((0, self.vocab), np.float32) if download else None
        m = self.manager
        seen = set()
        for e in entries:
            if e.req in seen:
                raise ValueError(f"request {e.req!r} appears twice in one step")
            seen.add(e.req)
            lo, hi = min(e.tokens), max(e.tokens)
            if not (0 <= int(lo) and int(hi) < self.vocab):
                raise ValueError(f"request {e.req!r}: token id {lo if int(lo) < 0 else hi} is outside the "
                                 f"vocabulary of {self.vocab}")
        T = sum(len(e.tokens) for e in entries)
        R = len(entries)
        if T > self.max_batch_tokens or R > self.max_seqs:
            raise ValueError(f"step of {T} tokens in {R} requests exceeds the limits "
                             f"({self.max_batch_tokens} tokens, {self.max_seqs} requests)")
        for e in entries:
            if not m.has(e.req):
                self.add(e.req)
        for e in entries:
            upto = m.computed(e.req) + len(e.tokens)
            if not m.reserve(e.req, upto):
                raise OutOfPages(f"request {e.req!r} needs pages for {upto} tokens and the pool "
                                 f"cannot give them: {m.stats()}")
        if tokens_from is not None and feed is None and T != R:
            raise ValueError("tokens_from without feed serves steps in which every request brings one token")
        self._clear_untouched(entries)
        self.rt.wait_event(self.meta_copied)     # the last step's copy has left the host buffer
        bucket = self._graph_bucket(entries)
        if bucket:
            out = self._graph_step(entries, bucket, tokens_from, pick, feed)
        else:
            off, words, T, R, n_rows, host_entries, max_q, max_ctx, n_multi = self._pack(entries, T, R, feed)
            picks = self._pick_buffers(n_rows) if pick and n_rows else None
            if picks is None:
                self._ensure_logits(n_rows)
            self.rt.copy_h2d_async(self.meta_dev.ptr, self.meta_host.ptr, words * 4)
            self.rt.record(self.meta_copied)
            self._feed(off, tokens_from, R, feed is None)
            ctx = self._context(off, T, R, host_entries, max_q, max_ctx, n_multi)
            self.arena.reset()
            if picks is not None:
                self._forward(ctx, n_rows, None, (T, R, n_rows, n_multi, max_q, max_ctx, "pick", picks[0].ptr), pick=picks)
                out = self.pick_ids.rows(0, n_rows)
            else:
                out = self.logits.rows(0, n_rows)
                self._forward(ctx, n_rows, out, (T, R, n_rows, n_multi, max_q, max_ctx, out.ptr))
                if pick:
                    out = self._argmax_of(out, n_rows)
        for e in entries:
            m.commit(e.req, m.computed(e.req) + len(e.tokens))
        self.steps_run += 1
        if not download:
            return out
        return self.rt.download(out)
