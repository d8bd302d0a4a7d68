"""Choosing the next token: greedy, temperature, top-k, top-p, repetition penalty.

Option names, meanings and the order of operations are the reference's
(orchestrator/sampler.py:33-98; orchestrator/engine.py:37-46): repetition penalty,
then the greedy test (temperature <= 0 or < 1e-6), temperature, top-k (ties at
the threshold stay, :146-156), top-p (smallest set by descending probability
whose mass reaches p, :186-203), softmax with the maximum subtracted
(:168-173), and the first index whose running sum exceeds a uniform number
(:205-213).  Two things differ on purpose: top_k and top_p are off unless
given, and the uniform number is a pure function of (seed, index of the
output token) instead of coming from one shared generator (:30-31), so a
request samples the same tokens whatever else is in the batch.

All of it runs on the device (csrc/sampling.hip): the penalty as a small
kernel over the (row, token) pairs, then the argmax, the inverse CDF, or, for
rows with top-k or top-p, the kernels that find both cut-offs and draw among
what they leave.  The host
implementation below is the same arithmetic in float64 and what the device is
tested against; the reference samples everything on the host (:10-11).
"""
from __future__ import annotations

import math
import os
from dataclasses import dataclass, field
from typing import Dict, Iterable, List, Optional, Sequence

import numpy as np

_MASK = (1 << 64) - 1


@dataclass
class SamplingParams:
    max_tokens: int = 128
    temperature: float = 1.0          # <= 0 (or < 1e-6): greedy
    top_p: float = 1.0                # 1.0: off
    top_k: int = 0                    # 0: off
    repetition_penalty: float = 1.0   # 1.0: off
    stop_tokens: Optional[List[int]] = None
    seed: Optional[int] = None

    def __post_init__(self):
        if self.max_tokens < 0:
            raise ValueError("max_tokens must not be negative")
        if not (0.0 < self.top_p <= 1.0):
            raise ValueError("top_p must be in (0, 1]")
        if self.top_k < 0:
            raise ValueError("top_k must not be negative")
        if self.repetition_penalty <= 0:
            raise ValueError("repetition_penalty must be positive")

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0 or self.temperature < 1e-6

    @property
    def plain(self) -> bool:
        """Greedy or temperature alone."""
        return self.repetition_penalty == 1.0 and (self.greedy or (self.top_k == 0 and self.top_p >= 1.0))

    @property
    def stateless(self) -> bool:
        """Nothing but the logits and a uniform number is needed (no penalty, which looks at the
        tokens so far), so runs of steps can be enqueued without the host in between."""
        return self.repetition_penalty == 1.0


def _mix64(z: int) -> int:
    z = (z + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform(seed: int, index: int) -> float:
    """A number in [0, 1) that depends only on the request's seed and on which of
    its output tokens is being drawn."""
    return (_mix64(_mix64(int(seed) & _MASK) ^ ((int(index) * 0xD1342543DE82EF95) & _MASK)) >> 11) / float(1 << 53)


def fresh_seed() -> int:
    return int.from_bytes(os.urandom(8), "little")


# ---------------------------------------------------------------- host sampling

def penalty_scales(past: Iterable[int], penalty: float) -> Dict[int, float]:
    """Token id -> what its logit is divided (if positive) or multiplied by."""
    counts: Dict[int, int] = past if isinstance(past, dict) else {int(t): 1 for t in past}
    return {int(t): (penalty ** (1.0 + math.log2(c)) if c > 1 else penalty) for t, c in counts.items()}


def apply_repetition_penalty(z: np.ndarray, past: Iterable[int], penalty: float) -> np.ndarray:
    for tid, s in penalty_scales(past, penalty).items():
        if 0 <= tid < len(z):
            z[tid] = z[tid] / s if z[tid] > 0 else z[tid] * s
    return z


def sample_host(logits: np.ndarray, params: SamplingParams, u: float, past: Iterable[int] = ()) -> int:
    z = np.array(logits, dtype=np.float64)
    if params.repetition_penalty != 1.0 and past:
        z = apply_repetition_penalty(z, past, params.repetition_penalty)
    if params.greedy:
        return int(np.argmax(z))
    z *= 1.0 / params.temperature
    if 0 < params.top_k < len(z):
        thr = np.partition(z, len(z) - params.top_k)[len(z) - params.top_k]
        z[z < thr] = -np.inf
    if params.top_p < 1.0:
        e = np.exp(z - z.max())
        pr = e / e.sum()
        order = np.argsort(-pr, kind="stable")
        cum = np.cumsum(pr[order])
        keep_n = int(np.searchsorted(cum, params.top_p, side="left")) + 1
        mask = np.ones(len(z), dtype=bool)
        mask[order[:keep_n]] = False
        z[mask] = -np.inf
    e = np.exp(z - z.max())
    cum = np.cumsum(e / e.sum())
    return min(int(np.searchsorted(cum, u, side="right")), len(z) - 1)


# ---------------------------------------------------------------- device sampling

class PendingIds:
    """Token ids chosen on the device, on their way to the host."""

    def __init__(self, rt, device_ptr: int, host, event: int, n: int):
        self.rt, self.device_ptr, self.host, self.event, self.n = rt, device_ptr, host, event, n

    def result(self) -> List[int]:
        self.rt.wait_event(self.event)
        return [int(x) for x in self.host.array(0, self.n, np.int32)]


class DeviceSampler:
    """Runs the argmax and inverse-CDF kernels on logits that are still on the device."""

    def __init__(self, rt, kernels, max_rows: int):
        from ..runtime.device import F32, F64, I32, Tensor
        self.rt = rt
        self.k = kernels
        self.max_rows = max_rows
        self.ids = rt.empty((max_rows,), I32)
        self.ids2 = rt.empty((max_rows,), I32)
        # the rows' uniform numbers, shares, temperatures and top-k: one block on the device (24
        # bytes a row, four arrays of max_rows), so that one copy brings them all
        self.row_params = rt.empty((max_rows * 6,), F32)
        base = self.row_params.ptr
        self.u = Tensor(base, (max_rows,), F64, self.row_params)
        self.top_p = Tensor(base + max_rows * 8, (max_rows,), F64, self.row_params)
        self.temp = Tensor(base + max_rows * 16, (max_rows,), F32, self.row_params)
        self.top_k = Tensor(base + max_rows * 20, (max_rows,), I32, self.row_params)
        self.scratch = rt.empty(((kernels.zk_sample_scratch_bytes(max_rows) + 3) // 4,), F32)
        self.cut_scratch = None                             # histograms and candidates of the cut-offs, on first use
        self._pen = None                                    # (rows, tokens, scales) on the device, grown on demand
        # the same block in page-locked memory, so that its copy queues behind the step's kernels
        # instead of waiting for them (``sample`` reads its ids before it returns, so the next
        # call finds the buffer free; steps that do not wait take theirs from a ring)
        self._stage = self._new_stage()
        self._ring_stages = None
        self._ring_stage_at = 0

    def _new_stage(self):
        n = self.max_rows
        buf = self.rt.pinned(n * 24)
        return {"buf": buf, "u": buf.array(0, n, np.float64), "p": buf.array(n * 8, n, np.float64),
                "t": buf.array(n * 16, n, np.float32), "k": buf.array(n * 20, n, np.int32), "event": self.rt.event()}

    # ---- steps that do not wait for the host
    RING = 16       # results, and rows' parameters, that may be on their way at a time

    # Which kernels a batch needs.  The kernels themselves decide row by row (a top_k of the
    # vocabulary's size or more is no top-k); the host only has to launch the one that serves a
    # row, and without the vocabulary's size it launches both for a row with a top_k alone.
    @staticmethod
    def _has_cut(p: SamplingParams, vocab: Optional[int]) -> bool:
        return p.top_p < 1.0 or (p.top_k > 0 and (vocab is None or p.top_k < vocab))

    @staticmethod
    def _is_plain(p: SamplingParams, vocab: Optional[int]) -> bool:
        return p.top_p >= 1.0 and (p.top_k == 0 or vocab is None or p.top_k >= vocab)

    def can_defer(self, rows: Sequence[dict]) -> bool:
        """True when ``stage`` and ``sample_staged`` serve these rows: nothing but the logits and
        a uniform number is needed (no penalty, which looks at the tokens so far)."""
        return len(rows) <= self.max_rows and all(r["params"].stateless for r in rows)

    def stage(self, rows: Sequence[dict], vocab: Optional[int] = None) -> dict:
        """Sends the rows' parameters on their way to the device, before the step that makes the
        logits is even enqueued, so that they are there when it ends.  What comes back goes to
        ``sample_staged`` with the logits.  A batch that takes the largest logit of every row
        sends nothing: its step may pick the ids itself (``StepRunner.step(pick=True)``) and hand
        them to ``ids_deferred``."""
        n = len(rows)
        greedy = [bool(r["params"].greedy) for r in rows]
        plan = {"n": n, "all_greedy": all(greedy), "any_greedy": any(greedy), "cut": False, "plain": False}
        if plan["all_greedy"]:
            return plan
        if self._ring_stages is None:
            self._ring_stages = [self._new_stage() for _ in range(self.RING)]
        st = self._ring_stages[self._ring_stage_at % self.RING]
        self._ring_stage_at += 1
        self.rt.wait_event(st["event"])             # its last copy has left the buffer
        for i, (r, g) in enumerate(zip(rows, greedy)):
            p = r["params"]
            st["t"][i] = 0.0 if g else p.temperature        # a row that is not drawn: the kernels leave it alone
            st["u"][i] = r["u"]
            st["k"][i] = p.top_k
            st["p"][i] = p.top_p
        plan["cut"] = any(not g and self._has_cut(r["params"], vocab) for r, g in zip(rows, greedy))
        plan["plain"] = any(not g and self._is_plain(r["params"], vocab) for r, g in zip(rows, greedy))
        self.rt.copy_h2d_async(self.row_params.ptr, st["buf"].ptr, self.max_rows * 24)
        self.rt.record(st["event"])
        return plan

    def sample_staged(self, logits, plan: dict) -> "PendingIds":
        """Enqueues the sampling of a step whose rows ``stage`` has sent.  The ids stay on the
        device (``.device_ptr``, valid until the next call) and travel to the host behind the
        kernels; ``.result()`` waits for them."""
        n, V = logits.shape
        if n != plan["n"]:
            raise ValueError(f"{n} rows of logits for {plan['n']} staged rows")
        rt, k = self.rt, self.k
        if plan["all_greedy"]:
            k.zk_argmax(logits.ptr, self.ids.ptr, n, V, self.scratch.ptr, rt.stream)
            return self._send(self.ids, n)
        if plan["any_greedy"]:
            k.zk_argmax(logits.ptr, self.ids2.ptr, n, V, self.scratch.ptr, rt.stream)
        self._draw(logits, n, V, self.u.ptr, plan["cut"], plan["plain"])
        return self._send(self.ids2, n)

    def ids_deferred(self, ids) -> "PendingIds":
        """Ids that a step picked itself (``StepRunner.step(pick=True)``, device int32 [n]) on
        their way to the host: as ``sample_staged`` of a greedy batch, without its kernels."""
        return self._send(ids, ids.shape[0])

    def _send(self, dev, n: int) -> "PendingIds":
        rt = self.rt
        if getattr(self, "_ring", None) is None:
            self._ring = [(rt.pinned(self.max_rows * 4), rt.event()) for _ in range(self.RING)]
            self._ring_at = 0
        host, ev = self._ring[self._ring_at % self.RING]
        self._ring_at += 1
        rt.copy_d2h_async(host.ptr, dev.ptr, n * 4)
        rt.record(ev)
        return PendingIds(rt, dev.ptr, host, ev, n)

    def sample(self, logits, rows: Sequence[dict]) -> List[int]:
        """``logits``: device float32 [n, vocab]; ``rows``: per row a dict with
        ``params``, ``u`` and ``past``.  Returns the chosen ids."""
        n, V = logits.shape
        if n == 0:
            return []
        if n > self.max_rows:
            raise ValueError(f"{n} rows to sample, room for {self.max_rows}")
        rt, k = self.rt, self.k
        # the penalty first, in place: what follows sees the changed logits, greedy rows too
        pen = [(i, t, sc) for i, r in enumerate(rows) if r["params"].repetition_penalty != 1.0 and r.get("past")
               for t, sc in penalty_scales(r["past"], r["params"].repetition_penalty).items() if 0 <= t < V]
        if pen:
            self._penalize(logits, V, pen)
        greedy = [bool(r["params"].greedy) for r in rows]
        if any(greedy):
            k.zk_argmax(logits.ptr, self.ids.ptr, n, V, self.scratch.ptr, rt.stream)
        if not all(greedy):
            st = self._stage
            for i, (r, gr) in enumerate(zip(rows, greedy)):
                p = r["params"]
                # (a greedy row goes with temperature 0: the drawing kernels leave it alone)
                st["t"][i], st["u"][i] = (0.0 if gr else p.temperature), r["u"]
                st["k"][i], st["p"][i] = p.top_k, p.top_p
            cut = any(not g and self._has_cut(r["params"], V) for r, g in zip(rows, greedy))
            plain = any(not g and self._is_plain(r["params"], V) for r, g in zip(rows, greedy))
            rt.copy_h2d_async(self.row_params.ptr, st["buf"].ptr, self.max_rows * 24)
            self._draw(logits, n, V, self.u.ptr, cut, plain)
        g = rt.download(self.ids.rows(0, n)) if any(greedy) else None
        s = rt.download(self.ids2.rows(0, n)) if not all(greedy) else None
        return [int(g[i]) if greedy[i] else int(s[i]) for i in range(n)]

    def _draw(self, logits, n: int, V: int, u_ptr: int, cut: bool, plain: bool) -> None:
        """Ids of the rows into ``self.ids2``.  ``cut``: some rows have top-k or top-p
        (``self.top_k``, ``self.top_p``); ``plain``: some have neither."""
        k, rt = self.k, self.rt
        if plain or not cut:
            k.zk_sample(logits.ptr, self.temp.ptr, u_ptr, self.top_k.ptr if cut else None, self.top_p.ptr if cut else None,
                        self.ids2.ptr, n, V, self.scratch.ptr, rt.stream)
        if not cut:
            return
        if self.cut_scratch is None:        # zero at first, and left so by every call
            from ..runtime.device import F32
            self.cut_scratch = rt.zeros(((k.zk_sample_cut_scratch_bytes(self.max_rows) + 3) // 4,), F32)
        k.zk_sample_cut(logits.ptr, self.temp.ptr, u_ptr, self.top_k.ptr, self.top_p.ptr, self.ids2.ptr, n, V,
                        self.cut_scratch.ptr, self.max_rows, rt.stream)

    def cut_ways(self, n: int) -> List[int]:
        """Which way each of the last ``n`` rows drawn with cut-offs went (0: it had none, 1: the
        candidates down to the cut-off, sorted by one block, 3: the cut-off's bucket sorted and the
        draw over the whole row, 2: the search over the whole row); for tests and measurements."""
        k = self.k
        words = self.rt.download(self.cut_scratch).view(np.int32)
        at = k.zk_sample_cut_mode_offset() // 4
        row_words = k.zk_sample_cut_row_bytes() // 4
        return [int(words[r * row_words + at]) for r in range(n)]

    def _penalize(self, logits, V: int, pen) -> None:
        from ..runtime.device import F32, I32
        m = len(pen)
        if self._pen is None or self._pen[0].shape[0] < m:
            room = max(1024, 2 * m)
            self._pen = (self.rt.empty((room,), I32), self.rt.empty((room,), I32), self.rt.empty((room,), F32))
        rows_d, toks_d, scales_d = self._pen
        self.rt.copy_h2d(rows_d.ptr, np.array([p[0] for p in pen], dtype=np.int32))
        self.rt.copy_h2d(toks_d.ptr, np.array([p[1] for p in pen], dtype=np.int32))
        self.rt.copy_h2d(scales_d.ptr, np.array([p[2] for p in pen], dtype=np.float32))
        self.k.zk_penalize(logits.ptr, V, rows_d.ptr, toks_d.ptr, scales_d.ptr, m, self.rt.stream)
