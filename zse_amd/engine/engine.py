"""The Python entry point: a model folder in, generated token ids out.

``Engine`` stands where the reference has ``ZSEEngine`` (one request at a time,
orchestrator/engine.py:70-525) and ``ZStreamerEngine`` (continuous batching,
zstreamer/engine.py:345-584): it owns the loaded model, the step runner with its
cache, the scheduler and the sampler.  ``generate`` runs any number of prompts
to completion; ``generate_tokens`` keeps the reference's single-prompt call and
its return value of prompt plus generated tokens (orchestrator/engine.py:299-318).
Prompts are token ids: text and tokenizers are outside this engine.
"""
from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field
from typing import Dict, Iterator, List, Optional, Sequence, Union

from ..runtime.device import Runtime, canonical_dtype
from ..sampling.sampler import DeviceSampler, SamplingParams, fresh_seed, uniform
from .loading import load_model, random_model
from .model import Model
from .request import FinishReason, Request, RequestState
from .runner import StepEntry, StepRunner
from .scheduler import UNKNOWN_TOKEN, Scheduler, SchedulerConfig, StepPlan


@dataclass
class EngineStats:
    steps: int = 0
    prompt_tokens: int = 0
    generated_tokens: int = 0
    preemptions: int = 0
    seconds: float = 0.0
    # per kind of step ("prefill": prompt portions only, "decode": single tokens only,
    # "mixed": both): [steps, tokens, seconds on the host's clock]
    by_kind: Dict[str, List[float]] = field(default_factory=dict)
    peak_pages: List[int] = field(default_factory=list)        # most pages in use at once, per cache group
    # per finished request, with the reference's meanings (zstreamer/request.py:206-228)
    ttft_ms: List[float] = field(default_factory=list)
    tpot_ms: List[float] = field(default_factory=list)
    # how the steps were launched: replayed from a captured graph, from a written-down launch
    # list, or call by call from Python (a shape's first two steps, and every step of a model
    # with a part that cannot be written down)
    graph_steps: int = 0
    launch_list_steps: int = 0
    python_steps: int = 0

    @property
    def tokens_per_second(self) -> float:
        return self.generated_tokens / self.seconds if self.seconds > 0 else 0.0

    def note_step(self, kind: str, steps: int, tokens: int, seconds: float) -> None:
        e = self.by_kind.setdefault(kind, [0, 0, 0.0])
        e[0] += steps
        e[1] += tokens
        e[2] += seconds

    def note_finished(self, reqs) -> None:
        for r in reqs:
            if r.finish_reason is not None and r.finish_reason.value != "error":
                self.ttft_ms.append(r.ttft_ms)
                self.tpot_ms.append(r.tpot_ms)


class Engine:
    def __init__(self, model: Union[str, Model], dtype: str = "bfloat16", block_size: int = 16,
                 num_blocks: Optional[int] = None, max_batch_tokens: int = 4096,
                 max_batch_seqs: int = 64, prefill_chunk_size: int = 512,
                 max_seq_len: Optional[int] = None, device_index: int = 0, tuned: bool = True,
                 use_graphs: bool = True, quiet: bool = True, decode_run: int = 4):
        self.rt = Runtime.get(device_index)
        self.dtype = canonical_dtype(dtype)
        self.model = load_model(model, self.dtype, self.rt, tuned=tuned) if isinstance(model, str) else model
        max_len = min(max_seq_len or self.model.plan.max_position, self.model.plan.max_position)
        pages = self._pages_per_group(num_blocks, block_size, max_batch_seqs, max_len,
                                      min(prefill_chunk_size, max_batch_tokens))
        self.runner = StepRunner(self.model, self.rt, self.dtype, page_size=block_size,
                                 num_pages=pages, max_seqs=max_batch_seqs,
                                 max_batch_tokens=max_batch_tokens, max_model_len=max_len,
                                 use_graphs=use_graphs)
        self.scheduler = Scheduler(SchedulerConfig(max_batch_tokens, prefill_chunk_size, max_batch_seqs),
                                   self.runner.manager)
        self.sampler = DeviceSampler(self.rt, self.runner.k, max_batch_seqs)
        self._stats = EngineStats()
        self._next_id = 0
        self.quiet = quiet
        # How many steps may be enqueued before the host looks at the ids of the first of them
        # (1: it looks after every step).  The ids are fed from step to step on the device; a
        # stop token found afterwards cuts the request's output back to it.
        self.decode_run = max(1, min(int(decode_run), DeviceSampler.RING))     # results on their way at a time
        self._next_plan: Optional[StepPlan] = None
        # steps whose ids are still on their way: (the ids, [(request, its place in the output)]);
        # the last of them left its ids at _last_ids, the row of request r at _last_rows[r]
        self._pending = deque()
        self._last_ids, self._last_rows = None, {}
        self._ending: Dict[object, Request] = {}     # reached their length in a step whose ids are on their way

    def _pages_per_group(self, num_blocks: Optional[int], block_size: int, max_seqs: int, max_len: int,
                         step_tokens: int) -> List[int]:
        """Pages for each cache group, in the runner's order of groups.  A group that keeps
        every key gets ``num_blocks`` pages (not given: enough for every request slot at the
        longest context, as far as 60 % of the free memory goes).  A windowed group gets what
        its requests can hold at most: the window, the page that is leaving it and the tokens
        of one step, for every request slot; never more than the all-keys number."""
        from ..cache.manager import group_needs
        needs = self.model.cache_needs()
        groups = group_needs(needs)
        item = 2 if self.dtype == "bfloat16" else 4
        def bytes_per_page(g):
            return sum(2 * needs[c].num_kv_heads * needs[c].head_dim for c in g.calls) * item * block_size
        def windowed_pages(g):
            per_request = -(-(g.window + step_tokens) // block_size) + 2
            return max_seqs * min(per_request, -(-max_len // block_size))
        if num_blocks is None:
            budget = int(self.rt.info().free_memory * 0.6)
            budget -= sum(windowed_pages(g) * bytes_per_page(g) for g in groups if g.window is not None)
            full = sum(bytes_per_page(g) for g in groups if g.window is None)
            want = max_seqs * -(-max_len // block_size)
            num_blocks = max(1, min(want, budget // full if full else want))
        return [min(num_blocks, windowed_pages(g)) if g.window is not None else num_blocks for g in groups]

    # ---- requests
    def add_request(self, prompt_tokens: Sequence[int], params: Optional[SamplingParams] = None,
                    request_id=None) -> Request:
        params = params or SamplingParams()
        vocab = self.model.plan.vocab_size
        for t in prompt_tokens:
            if not (0 <= int(t) < vocab):
                raise ValueError(f"token id {t} is outside the vocabulary of {vocab}")
        if request_id is None:
            request_id = f"req-{self._next_id}"
        self._next_id += 1
        req = Request(request_id, [int(t) for t in prompt_tokens], params,
                      seed=params.seed if params.seed is not None else fresh_seed())
        self.scheduler.add_request(req)
        self._stats.prompt_tokens += len(req.prompt_tokens)
        return req

    def step(self) -> List[Request]:
        """Schedule, run and sample one step, or up to ``decode_run`` steps enqueued one behind
        the other where that is possible (``_can_run_ahead``); every id has reached the host
        when this returns.  Returns the requests that finished."""
        t0 = time.monotonic()
        plan = self._take_plan()
        if not plan:
            return list(plan.failed)
        kind, steps0, tokens = self._kind(plan), self._stats.steps, plan.num_tokens
        if self._can_run_ahead(plan):
            done = []
            for i in range(self.decode_run):
                done += self._enqueue(plan)
                if i + 1 == self.decode_run:
                    break
                nxt = self.scheduler.schedule()
                if not nxt or not self._can_run_ahead(nxt):
                    self._next_plan = nxt
                    break
                plan = nxt
            done += self._resolve(0)
        else:
            done = self._step_and_wait(plan)
        n = self._stats.steps - steps0
        self._stats.note_step(kind, n, tokens * max(n, 1), time.monotonic() - t0)
        self._stats.note_finished(done)
        return done

    def run(self) -> None:
        """Every request to its end.  Steps are enqueued without waiting for their ids wherever
        ``_can_run_ahead`` allows; the ids of a step are read when ``decode_run`` later steps
        have been enqueued behind it, so the device has work while the host reads, plans and
        packs."""
        t0 = time.monotonic()
        while self.scheduler.has_work() or self._pending:
            t1 = time.monotonic()
            plan = self._take_plan()
            if not plan:
                done = self._resolve(0) + list(plan.failed)
                self._stats.note_finished(done)
                continue
            kind, steps0, tokens = self._kind(plan), self._stats.steps, plan.num_tokens
            if self._can_run_ahead(plan):
                done = self._enqueue(plan) + self._resolve(self.decode_run - 1)
            else:
                done = self._resolve(0)            # the host has to see every id first
                plan.items = [s for s in plan.items if not s.request.finished]
                done += self._step_and_wait(plan) if plan.items else list(plan.failed)
            self._stats.note_step(kind, self._stats.steps - steps0, tokens, time.monotonic() - t1)
            self._stats.note_finished(done)
        self._stats.seconds += time.monotonic() - t0

    def _take_plan(self) -> StepPlan:
        plan, self._next_plan = (self._next_plan if self._next_plan is not None else self.scheduler.schedule()), None
        if plan:
            pools = self.runner.manager.pools
            if len(self._stats.peak_pages) != len(pools):
                self._stats.peak_pages = [0] * len(pools)
            self._stats.peak_pages = [max(a, p.used_pages) for a, p in zip(self._stats.peak_pages, pools)]
        return plan

    @staticmethod
    def _kind(plan: StepPlan) -> str:
        multi = any(s.count > 1 for s in plan.items)
        single = any(s.count == 1 and s.request.state == RequestState.DECODING for s in plan.items)
        return "mixed" if multi and single else ("prefill" if multi or not single else "decode")

    def _step_and_wait(self, plan: StepPlan) -> List[Request]:
        """One step whose ids the host reads before it goes on (nothing is on its way)."""
        entries = [StepEntry(s.request.request_id,
                             s.request.tokens_at(s.start, s.count),
                             [s.count - 1] if s.sample else []) for s in plan.items]
        logits = self.runner.step(entries, download=False)
        rows = []
        who = []
        for s in plan.items:
            if s.sample:
                r = s.request
                rows.append({"params": r.params, "u": uniform(r.seed, len(r.output_tokens)),
                             "past": r.penalty_counts() if r.params.repetition_penalty != 1.0 else ()})
                who.append(r.request_id)
        ids = self.sampler.sample(logits, rows) if rows else []
        done = self.scheduler.on_step_done(plan, dict(zip(who, ids)))
        self._last_rows = {}
        self._stats.steps += 1
        self._stats.generated_tokens += len(ids)
        self._stats.preemptions = self.scheduler.num_preemptions
        return done + list(plan.failed)

    # ---- steps that do not wait for the host
    def _rows(self, plan: StepPlan) -> List[dict]:
        return [{"params": s.request.params, "u": uniform(s.request.seed, len(s.request.output_tokens)),
                 "past": ()} for s in plan.items if s.sample]

    def _can_run_ahead(self, plan: StepPlan) -> bool:
        """Whether the plan's step may be enqueued before the ids of the steps before it have
        reached the host: its requests are sampled on the device from nothing but their logits
        (no repetition penalty), nothing is out of the ordinary (nobody was preempted or
        turned away), and a token that the host has not seen yet is the one token its request
        brings and was drawn by the step just before, whose ids are still on the device."""
        if self.decode_run < 2 or not plan or plan.preempted or plan.failed:
            return False
        for s in plan.items:
            if s.request.tokens_at(s.start + s.count - 1, 1)[0] == UNKNOWN_TOKEN and \
                    (s.count != 1 or s.request.request_id not in self._last_rows):
                return False
        return self.sampler.can_defer(self._rows(plan))

    def _enqueue(self, plan: StepPlan) -> List[Request]:
        """One step, nothing awaited.  A request's token that the step before has drawn and the
        host has not seen yet is fed to the step on the device; its place in the request's
        output holds a placeholder until the ids arrive (``_resolve``), and the scheduler plans
        with the numbers of tokens, which it knows.  A request that reaches its length here has
        ended for the scheduler; ``_resolve`` reports it when its last token has been read."""
        sch, runner, sampler = self.scheduler, self.runner, self.sampler
        entries, feed = [], []
        for s in plan.items:
            r = s.request
            toks = r.tokens_at(s.start, s.count)
            src = -1
            if toks[-1] == UNKNOWN_TOKEN:           # drawn by the step before, still on the device
                src, toks = self._last_rows[r.request_id], [0]
            entries.append(StepEntry(r.request_id, toks, [s.count - 1] if s.sample else []))
            feed.append(src)
        fed = any(x >= 0 for x in feed)
        rows = self._rows(plan)
        places = [(s.request, len(s.request.output_tokens)) for s in plan.items if s.sample]
        staged = sampler.stage(rows, runner.vocab) if rows else None
        kw = dict(download=False, tokens_from=self._last_ids if fed else None, feed=feed if fed else None)
        if rows and staged["all_greedy"]:
            # the step picks the largest logits itself (in the head product's epilogue where
            # the kernels can: the logits then never reach memory)
            ids = sampler.ids_deferred(runner.step(entries, pick=True, **kw))
        else:
            logits = runner.step(entries, **kw)
            ids = sampler.sample_staged(logits, staged) if rows else None
        if ids is not None:
            self._pending.append((ids, places))
            self._last_ids, self._last_rows = ids.device_ptr, {r.request_id: j for j, (r, _) in enumerate(places)}
        else:
            self._last_rows = {}
        self._stats.steps += 1
        for r in sch.on_step_done(plan, {r.request_id: None for r, _ in places}):
            self._ending[r.request_id] = r           # reached its length: reported when its last token is read
        return []

    def _resolve(self, keep: int) -> List[Request]:
        """Reads the ids of the enqueued steps, oldest first, until at most ``keep`` steps are
        still on their way: puts them where the placeholders are and ends what a stop token
        ends (the request's output is cut back to it; what was computed for it since is thrown
        away).  Returns the requests whose end is now known in full: by a stop token, or by
        their length with the last token read.  A request's times are those at which the host
        had its tokens, not those at which their steps were enqueued."""
        done = []
        while len(self._pending) > keep:
            ids, places = self._pending.popleft()
            toks = ids.result()
            now = time.monotonic()
            for (r, at), tok in zip(places, toks):
                if at >= len(r.output_tokens):          # behind a stop token found in an earlier step
                    continue
                r.output_tokens[at] = tok
                self._stats.generated_tokens += 1
                if at == 0:
                    r.first_token_time = now
                if r.params.stop_tokens and tok in r.params.stop_tokens:
                    ended_before = self._ending.pop(r.request_id, None) is not None
                    r.finish_time = None
                    if self.scheduler.finish_at(r, at + 1, FinishReason.STOP) or ended_before:
                        done.append(r)
                elif at == len(r.output_tokens) - 1 and self._ending.pop(r.request_id, None) is not None:
                    r.finish_time = now
                    done.append(r)
        if done and self._next_plan is not None:
            self._next_plan.items = [s for s in self._next_plan.items if not s.request.finished]
        self._stats.preemptions = self.scheduler.num_preemptions
        return done

    # ---- the calls users make
    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[None, SamplingParams, Sequence[SamplingParams]] = None) -> List[List[int]]:
        """Generated token ids for each prompt (the prompt itself is not repeated).
        A request that could not be served raises ``RuntimeError``."""
        if params is None or isinstance(params, SamplingParams):
            plist = [params or SamplingParams()] * len(prompts)
        else:
            plist = list(params)
            if len(plist) != len(prompts):
                raise ValueError("one SamplingParams per prompt, or one for all")
        reqs = []
        for p, sp in zip(prompts, plist):
            if sp.max_tokens == 0:
                reqs.append(None)
                continue
            reqs.append(self.add_request(p, sp))
        self.run()
        out = []
        for r in reqs:
            if r is None:
                out.append([])
                continue
            if r.finish_reason == FinishReason.ERROR:
                raise RuntimeError(f"request {r.request_id}: {r.error}")
            out.append(list(r.output_tokens))
        return out

    def generate_tokens(self, token_ids: Sequence[int], max_tokens: int = 128, temperature: float = 1.0,
                        top_p: float = 1.0, top_k: int = 0, repetition_penalty: float = 1.0,
                        stop_tokens: Optional[List[int]] = None, seed: Optional[int] = None) -> List[int]:
        """Prompt plus generated tokens of one request (orchestrator/engine.py:299-318)."""
        sp = SamplingParams(max_tokens, temperature, top_p, top_k, repetition_penalty, stop_tokens, seed)
        return list(token_ids) + self.generate([token_ids], sp)[0]

    def stream_generate_tokens(self, token_ids: Sequence[int], **kw) -> Iterator[int]:
        """Generated tokens of one request as they are produced (orchestrator/engine.py:320-367)."""
        sp = SamplingParams(**kw)
        if sp.max_tokens == 0:
            return
        req = self.add_request(token_ids, sp)
        seen = 0
        while not req.finished:
            self.step()
            while seen < len(req.output_tokens):
                yield req.output_tokens[seen]
                seen += 1
        if req.finish_reason == FinishReason.ERROR:
            raise RuntimeError(f"request {req.request_id}: {req.error}")

    def stats(self) -> EngineStats:
        if self.runner is not None:
            self._launch_counts = (self.runner.graph_runs, self.runner.steplist_runs, self.runner.steplist_misses)
        st = self._stats
        st.graph_steps, st.launch_list_steps, st.python_steps = getattr(self, "_launch_counts", (0, 0, 0))
        return st

    def close(self) -> None:
        if self.runner is not None:
            self.stats()                       # keeps the runner's launch counts
            self.runner.close()
        self.runner = None
        self.sampler = None

    destroy = close

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
