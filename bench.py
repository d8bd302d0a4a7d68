#!/usr/bin/env python3
"""Decode and prefill throughput of Gemma 2 layer shapes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B]
    python bench.py --workload 9b|27b

The default run times Gemma 2 2B shapes.  A step is one decode step of the whole batch: every
live request brings one token, the model runs from the cache, the next token is picked greedily
on the device.  Weights are seeded random values, token ids are synthetic.  One JSON line comes
out; its ``value`` is decoded tokens a second at the default batch, ``points`` holds batch 1
and 64, ``prefill`` one 2,048-token prompt in one step, ``roofline`` the decode step's bytes
over its time.  Fractions are given against the published peaks (``frac``) and against what
two probe kernels reach on this very GPU (``frac_probed``).

Before anything is timed the model is checked (``checked``): a two-layer slice of the very
model that is timed (same seed, so the same tensors) runs whole prompts, portions and single
tokens in 32-bit and in bfloat16 against the plain implementation under ``tests/plain`` on the
same weights made on the host, and at every batch size that is timed the full model's decode
steps through the timed path (captured graphs or launch lists, ids fed on the device) must pick
the same tokens as steps launched call by call.  A failed check ends the run with an error.

The same run then goes on to further sizes (``--quick`` leaves them out): the 2B shapes decoding
at a context of 8,192, and the 9B and 27B shapes (decode at batch 8, a 2,048-token prefill, and
their serving workloads through ``Engine.generate``, end to end: 9b = 32 requests with prompts of
128 to 4,096 tokens, 256 greedy tokens each, portions of 512; 27b = 8 prompts of 8,192 tokens,
128 tokens each at temperature 1.0, seed 3).  They land in ``points`` (tokens a second) and, with
their times and fractions of the peaks, in ``further``.  ``--workload 9b|27b`` runs one workload
alone.  What a step has to read and to compute is read off the model's parts (``Model.flops``,
``Model.cache_bytes_read``, the bytes of its weights), not written down here per architecture.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
PEAK_HBM = 8.0e12          # bytes/s, MI355X
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
REFERENCE_SAMPLING = {"temperature": 1.0, "top_k": 50, "top_p": 0.9}     # the reference's defaults

GEMMA2_2B = dict(
    architectures=["Gemma2ForCausalLM"], model_type="gemma2", num_hidden_layers=26, hidden_size=2304,
    num_attention_heads=8, num_key_value_heads=4, head_dim=256, query_pre_attn_scalar=256,
    intermediate_size=9216, vocab_size=256000, rope_theta=10000.0, sliding_window=4096,
    attn_logit_softcapping=50.0, final_logit_softcapping=30.0, rms_norm_eps=1e-6,
    max_position_embeddings=8192)


# further sizes of the same architecture, for looking beyond the default (--model, --workload)
GEMMA2_9B = dict(GEMMA2_2B, num_hidden_layers=42, hidden_size=3584, num_attention_heads=16, num_key_value_heads=8,
                 head_dim=256, query_pre_attn_scalar=256, intermediate_size=14336)
GEMMA2_27B = dict(GEMMA2_2B, num_hidden_layers=46, hidden_size=4608, num_attention_heads=32, num_key_value_heads=16,
                  head_dim=128, query_pre_attn_scalar=144, intermediate_size=36864)
MODELS = {"2b": GEMMA2_2B, "9b": GEMMA2_9B, "27b": GEMMA2_27B}


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


# ------------------------------------------------------------------ what this GPU reaches
def probe_peaks(rt):
    """(bytes/s a kernel streams from memory, bf16 flop/s of the matrix cores alone), each the
    best of a few launches of a probe kernel."""
    import ctypes
    k = rt.kernels("bfloat16")
    sink = rt.zeros((64,), "float32")
    nbytes = 4 << 30
    buf = rt.zeros((nbytes // 4,), "float32")
    a, b = rt.event(), rt.event()
    best_bw = 0.0
    for _ in range(6):
        rt.record(a)
        k.zk_probe_read(buf.ptr, nbytes, sink.ptr, rt.stream)
        rt.record(b)
        best_bw = max(best_bw, nbytes / (rt.elapsed_ms(a, b) * 1e-3))
    flops = ctypes.c_double(0.0)
    best_fl = 0.0
    for _ in range(4):
        rt.record(a)
        k.zk_probe_mfma_bf16(4000, sink.ptr, ctypes.byref(flops), rt.stream)
        rt.record(b)
        best_fl = max(best_fl, flops.value / (rt.elapsed_ms(a, b) * 1e-3))
    return best_bw, best_fl


# ------------------------------------------------------------------ the check before timing
def bf16_round(a):
    from zse_amd.weights.safetensors import bf16_bits_to_f32, f32_to_bf16_bits
    return bf16_bits_to_f32(f32_to_bf16_bits(np.ascontiguousarray(a, np.float32)))


def check_slice(cfg, rt, seed, std, gain_std):
    """Layers 0 and 1, embedding, final norm and head of the model that is timed (the same
    tensors: a tensor's values follow from seed, name and index) against the plain
    implementation, in 32-bit and in bfloat16, cut three ways.  The host makes the same weights
    with the host side of the random-weights function.  The plain head is restricted to the
    first 8,192 rows of the embedding (token ids are drawn below that), whose logits are
    compared; the product over the whole vocabulary has a test of its own."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from plain import gemma2_plain as P
    from zse_amd.engine.loading import random_model
    from zse_amd.engine.model import Model
    from zse_amd.engine.runner import StepEntry, StepRunner
    from zse_amd.config.base import resolve_architecture
    from zse_amd.weights.random_init import random_tensors

    small = dict(cfg, num_hidden_layers=2)
    Vc = min(8192, cfg["vocab_size"])
    host_cfg = dict(small, vocab_size=Vc)
    arch = resolve_architecture(host_cfg)
    w32 = random_tensors(Model(arch.plan(arch.config_from_dict(host_cfg))).tensor_reqs(), seed, std, gain_std)
    rng = np.random.default_rng(11)
    streams = {"a": rng.integers(0, Vc, 40).tolist(), "b": rng.integers(0, Vc, 37).tolist(),
               "c": rng.integers(0, Vc, 21).tolist()}
    # a whole; b in portions of 9, 2 and 13, then token by token beside c's portions and tokens
    steps = [[("a", 40)], [("b", 9)], [("b", 2), ("c", 5)], [("b", 13), ("c", 1)]]
    steps += [[("b", 1), ("c", 3 if i == 0 else 1)] for i in range(13)]
    out = {}
    for dtype in ("float32", "bfloat16"):
        w = w32 if dtype == "float32" else {n: bf16_round(t) for n, t in w32.items()}
        model = random_model(small, dtype, seed=seed, std=std, gain_std=gain_std, rt=rt)
        runner = StepRunner(model, rt, dtype, page_size=16, cache_tokens=512, max_seqs=4, max_batch_tokens=256,
                            max_model_len=256, use_graphs=False)
        fed = {r: 0 for r in streams}
        rows = {r: [] for r in streams}
        for st in steps:
            es = [StepEntry(r, streams[r][fed[r]:fed[r] + n], range(n)) for r, n in st if fed[r] < len(streams[r])]
            z = runner.step(es)
            at = 0
            for e in es:
                n = len(e.tokens)
                rows[e.req].append(z[at:at + n, :Vc])
                at += n
                fed[e.req] += n
        assert all(fed[r] == len(t) for r, t in streams.items()), fed
        worst = 0.0
        for r, toks in streams.items():
            want = P.forward(host_cfg, w, toks, np.float64)
            got = np.concatenate(rows[r]).astype(np.float64)
            err = np.abs(got - want).max() / max(1.0, np.abs(want).max())
            worst = max(worst, float(err))
        out[dtype] = worst
        del runner, model
    return out


def check_decode_path(model, rt, vocab, B, use_graphs):
    """The model that is timed, at a batch size that is timed: the ids that come out of the
    timed path (graphs up to 16 requests, launch lists above, ids picked on the device and fed
    to the next step from there) equal those of steps launched call by call from Python whose
    logits the host reads."""
    from zse_amd.engine.runner import StepEntry, StepRunner
    from zse_amd.sampling.sampler import DeviceSampler, SamplingParams
    rng = np.random.default_rng(5 + B)
    prompts = [rng.integers(0, vocab, 24 + 3 * (i % 11)).tolist() for i in range(B)]
    n_steps = 7
    picked = []
    for timed in (False, True):
        runner = StepRunner(model, rt, "bfloat16", page_size=16, cache_tokens=B * 96, max_seqs=B,
                            max_batch_tokens=max(2048, B), max_model_len=4096, use_graphs=timed and use_graphs,
                            use_steplists=timed)
        ids = []
        for at in range(0, B, 16):                 # the prompts, sixteen a step
            z = runner.step([StepEntry(i, prompts[i], [len(prompts[i]) - 1]) for i in range(at, min(at + 16, B))])
            ids += z.argmax(axis=1).tolist()
        ids = [ids]
        if not timed:
            for _ in range(n_steps):
                z = runner.step([StepEntry(i, [t], [0]) for i, t in enumerate(ids[-1])])
                ids.append(z.argmax(axis=1).tolist())
        else:
            sampler = DeviceSampler(rt, runner.k, B)
            fed, pending = None, []
            for _ in range(n_steps):
                toks = ids[0] if fed is None else [0] * B
                chosen = runner.step([StepEntry(i, [t], [0]) for i, t in enumerate(toks)], download=False,
                                     tokens_from=fed, pick=True)
                pending.append(sampler.ids_deferred(chosen))
                fed = pending[-1].device_ptr
            ids += [list(p.result()) for p in pending]
            if use_graphs and B <= runner.graph_max_batch and not any(isinstance(g, int) for g in runner.graphs.values()):
                raise SystemExit("bench.py: no decode step was captured into a graph")
            if B > runner.graph_max_batch and runner.steplist_runs == 0:
                raise SystemExit("bench.py: no decode step ran from its launch list")
        picked.append(ids)
        runner.close()
        del runner
    return picked[0] == picked[1]


# ------------------------------------------------------------------ workloads through the engine
def run_workload(name, a, model=None):
    """One of the two larger workloads through ``Engine.generate``; returns its record."""
    from zse_amd.engine.engine import Engine
    from zse_amd.engine.loading import random_model
    from zse_amd.runtime.device import Runtime
    from zse_amd.sampling import SamplingParams
    cfg = dict(MODELS[name])
    full_layers = cfg["num_hidden_layers"]
    if a.layers:
        cfg["num_hidden_layers"] = a.layers
    if name == "27b":
        # the workload's prompts fill Gemma 2's 8,192 positions by themselves: room for the new tokens
        cfg["max_position_embeddings"] = 8192 + 128
    rt = Runtime.get()
    t0 = time.time()
    if model is None:
        model = random_model(cfg, "bfloat16", seed=0, std=0.02, gain_std=0.1, rt=rt)
        log(f"{name}: model ready in {time.time() - t0:.1f} s, {model.weight_bytes / 1e9:.2f} GB of weights")
    rng = np.random.default_rng(0)
    V, page = cfg["vocab_size"], 16
    if name == "9b":
        lengths = rng.integers(128, 4097, 32).tolist()
        params = SamplingParams(max_tokens=256, temperature=0.0)
        what = "32 requests, prompts uniform in [128, 4096], 256 greedy tokens each, portions of 512"
    else:
        lengths = [8192] * 8
        params = SamplingParams(max_tokens=128, temperature=1.0, seed=3)
        what = "8 prompts of 8192 tokens, 128 tokens each at temperature 1.0 (seed 3), portions of 512"
    prompts = [rng.integers(0, V, n).tolist() for n in lengths]
    n_new = params.max_tokens
    max_len = max(lengths) + n_new
    blocks = sum(-(-(n + n_new) // page) for n in lengths) + 8
    eng = Engine(model, dtype="bfloat16", block_size=page, num_blocks=blocks, max_batch_tokens=4096,
                 max_batch_seqs=len(prompts), prefill_chunk_size=512, max_seq_len=max_len,
                 use_graphs=not a.no_graphs)
    # a small run first: code objects load, the arena and the first graphs are made
    eng.generate([p[:70] for p in prompts[:2]], SamplingParams(max_tokens=6, temperature=0.0))
    m = eng.runner.manager
    stats0 = eng.stats()
    stats0.by_kind.clear(), stats0.ttft_ms.clear(), stats0.tpot_ms.clear()
    stats0.peak_pages = [0] * len(m.pools)
    steps0, gen0, sec0 = stats0.steps, stats0.generated_tokens, stats0.seconds
    rt.sync()
    t1 = time.perf_counter()
    out = eng.generate(prompts, params)
    rt.sync()
    dt = time.perf_counter() - t1
    st = eng.stats()
    assert all(len(o) == n_new for o in out)
    gen = st.generated_tokens - gen0
    prompt_tokens = sum(lengths)
    needs = model.cache_needs()
    item = 2
    groups = []
    for g, pool, peak in zip(m.groups, m.pools, st.peak_pages):
        per_page = sum(2 * needs[c].num_kv_heads * needs[c].head_dim for c in g.calls) * item * page
        groups.append({"window": g.window, "layers": len(g.calls), "pages": pool.num_pages, "peak_pages": peak,
                       "peak_gb": round(peak * per_page / 1e9, 2), "pool_gb": round(pool.num_pages * per_page / 1e9, 2)})
    # what the cache would hold at the end without the window rule: every layer keeps every key
    per_token_all = sum(2 * n.num_kv_heads * n.head_dim for n in needs if n is not None) * item
    no_release_gb = sum(-(-(n + n_new) // page) * page for n in lengths) * per_token_all / 1e9
    kinds = {k: {"steps": int(v[0]), "tokens": int(v[1]), "seconds": round(v[2], 3),
                 "ms_per_step": round(1e3 * v[2] / max(v[0], 1), 3)} for k, v in st.by_kind.items()}
    res = {
        "metric": f"end-to-end generated tok/s, Gemma 2 {name.upper()} bf16 workload", "value": round(gen / dt, 1),
        "unit": "tok/s", "n_gpus": 1, "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
        "workload": what, "seconds": round(dt, 3), "generated_tokens": gen, "prompt_tokens": prompt_tokens,
        "all_tokens_per_s": round((gen + prompt_tokens) / dt, 1), "steps": st.steps - steps0,
        "preemptions": st.preemptions,
        "launched": {"graph": st.graph_steps, "launch_list": st.launch_list_steps, "python": st.python_steps},
        "config": {"model": f"gemma2-{name}-shapes-random", "layers": cfg["num_hidden_layers"], "layers_full": full_layers,
                   "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate": cfg["intermediate_size"], "vocab": V, "sliding_window": cfg["sliding_window"],
                   "requests": len(prompts), "max_tokens": n_new, "page_size": page, "prefill_chunk_size": 512,
                   "max_batch_tokens": 4096, "max_positions": cfg["max_position_embeddings"],
                   "weights_gb": round(model.weight_bytes / 1e9, 2)},
        "by_kind": kinds, "cache_groups": groups, "cache_without_window_release_gb": round(no_release_gb, 2),
        "ttft_ms_mean": round(float(np.mean(st.ttft_ms)), 1), "ttft_ms_max": round(float(np.max(st.ttft_ms)), 1),
        "tpot_ms_mean": round(float(np.mean(st.tpot_ms)), 3),
    }
    eng.close()
    return res


class Timed:
    """A model on a runner sized for the batches and the context that are timed."""

    def __init__(self, model, rt, cfg, max_b, context, prefill_tokens, graphs, page=16):
        from zse_amd.engine.runner import StepRunner
        from zse_amd.sampling.sampler import DeviceSampler
        self.model, self.rt, self.cfg, self.context, self.T = model, rt, cfg, context, prefill_tokens
        self.V = cfg["vocab_size"]
        longest = max(context, prefill_tokens)       # a prompt longer than the decode context still fits
        self.runner = StepRunner(model, rt, "bfloat16", page_size=page,
                                 num_pages=max(max_b * (-(-context // page) + 1), -(-longest // page)) + 8,
                                 max_seqs=max_b, max_batch_tokens=max(prefill_tokens, max_b), max_model_len=longest,
                                 use_graphs=graphs)
        self.sampler = DeviceSampler(rt, self.runner.k, max_b)
        self.rng = np.random.default_rng(0)
        # Steady state is what is measured.  For about a second after a process has allocated tens
        # of GB (the cache slabs, just now) kernels that wait for memory rather than stream from it
        # run up to 17 % slower (the o and down products of a decode step: 10.1 instead of 8.7 us;
        # steps at batch 1 and 8 by 3 to 4 %); later steps of the same process do not, whatever was
        # done meanwhile.  So the timed work starts two seconds after the allocations.
        rt.sync()
        time.sleep(2.0)

    def close(self):
        self.runner.close()
        self.runner = self.sampler = None

    def prefill(self, portion=None, repeats=3):
        """One prompt of ``self.T`` tokens, whole or in portions of ``portion`` tokens, logits of
        its last token wanted: (seconds, flops), the median of ``repeats`` after one untimed."""
        from zse_amd.engine.runner import StepEntry
        T, runner, rt = self.T, self.runner, self.rt
        portion = portion or T
        times = []
        for i in range(repeats + 1):
            toks = self.rng.integers(0, self.V, T).tolist()
            rt.sync()
            t1 = time.perf_counter()
            for at in range(0, T, portion):
                n = min(portion, T - at)
                runner.step([StepEntry("p", toks[at:at + n], [n - 1] if at + n == T else [])], download=False)
            rt.sync()
            times.append(time.perf_counter() - t1)
            runner.finish("p")
        flops = sum(self.model.flops([(at, min(portion, T - at))], 1 if at + portion >= T else 0)
                    for at in range(0, T, portion))
        return float(np.median(times[1:])), flops

    def decode(self, B, steps, warmup, drawn=None):
        """``steps`` decode steps of ``B`` requests that end at the full context: (tokens a
        second, seconds a step, bytes a step has to read, how the steps were launched).
        ``drawn``: keyword arguments of SamplingParams for steps that draw their tokens instead of
        taking the largest logit."""
        from zse_amd.engine.runner import StepEntry
        from zse_amd.sampling.sampler import SamplingParams
        runner, rt, sampler, rng, V = self.runner, self.rt, self.sampler, self.rng, self.V
        ctx0 = self.context - steps - warmup
        reqs = [f"d{B}_{i}" for i in range(B)]
        for r in reqs:                       # fill the cache through real prefill steps
            left = ctx0
            while left > 0:
                n = min(left, self.T)
                runner.step([StepEntry(r, rng.integers(0, V, n).tolist(), [])], download=False)
                left -= n
        first = rng.integers(0, V, B).tolist()
        rows = [{"params": SamplingParams(**(drawn or {"temperature": 0.0})), "u": 0.0} for _ in range(B)]
        # As the engine decodes: a greedy step picks the largest logits itself, a drawing step hands
        # its logits to the sampling kernels; either way the ids stay on the device, the next step
        # takes them from there, and the host reads them four steps at a time (it has to, for stop
        # tokens) while the next steps are already enqueued.
        pending, fed = [], None

        def one():
            nonlocal fed
            toks = first if fed is None else [0] * B
            entries = [StepEntry(r, [t], [0]) for r, t in zip(reqs, toks)]
            if drawn:
                for row in rows:
                    row["u"] = float(rng.random())
                staged = sampler.stage(rows, V)
                ids = sampler.sample_staged(runner.step(entries, download=False, tokens_from=fed), staged)
            else:
                ids = sampler.ids_deferred(runner.step(entries, download=False, tokens_from=fed, pick=True))
            fed = ids.device_ptr
            pending.append(ids)
            if len(pending) == 4:
                for p in pending:
                    p.result()
                pending.clear()
        lists0 = runner.steplist_runs
        for _ in range(warmup):
            one()
        rt.sync()
        t1 = time.perf_counter()
        for _ in range(steps):
            one()
        rt.sync()
        dt = time.perf_counter() - t1
        for r in reqs:
            runner.finish(r)
        how = "graph" if runner._graph_bucket([StepEntry(r, [0], [0]) for r in reqs]) else \
            ("launch list" if runner.steplist_runs > lists0 else "call by call")
        mean_ctx = int(self.context - steps / 2.0)
        byts = self.model.weight_bytes + B * self.model.cache_bytes_read(mean_ctx, 2)
        return B * steps / dt, dt / steps, byts, how


def shape_of(cfg, full_layers):
    return {"layers": cfg["num_hidden_layers"], "layers_full": full_layers, "hidden": cfg["hidden_size"],
            "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
            "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"], "sliding_window": cfg["sliding_window"]}


def further_model(name, a, rt, peak_bw, peak_fl):
    """Decode at batch 8, a 2,048-token prefill and the serving workload of one of the larger
    models, each with its fraction of the nominal peak."""
    from zse_amd.engine.loading import random_model
    cfg = dict(MODELS[name], max_position_embeddings=8192 + 128)
    t0 = time.time()
    model = random_model(cfg, "bfloat16", seed=0, std=0.02, gain_std=0.1, rt=rt)
    log(f"{name}: model ready in {time.time() - t0:.1f} s, {model.weight_bytes / 1e9:.2f} GB of weights")
    same = check_decode_path(model, rt, cfg["vocab_size"], 8, not a.no_graphs)
    if not same:
        raise SystemExit(f"bench.py: {name}: the timed decode path does not pick the tokens of eager steps")
    t = Timed(model, rt, cfg, 8, a.context, a.prefill_tokens, not a.no_graphs)
    pre_s, pf = t.prefill()
    tok_s, step_s, byts, how = t.decode(8, max(16, a.steps // 2), max(4, a.warmup // 2))
    t.close()
    out = {"config": dict(shape_of(cfg, cfg["num_hidden_layers"]), weights_gb=round(model.weight_bytes / 1e9, 2)),
           "decode_b8": {"value": round(tok_s, 1), "ms_per_step": round(step_s * 1e3, 3), "context": a.context,
                         "launched": how, "roofline_frac": round(byts / step_s / PEAK_HBM, 4),
                         "gbs": round(byts / step_s / 1e9, 1)},
           "prefill": {"value": round(a.prefill_tokens / pre_s, 1), "tokens": a.prefill_tokens, "ms": round(pre_s * 1e3, 3),
                       "frac": round(pf / pre_s / PEAK_FLOPS["bf16"], 4)}}
    log(f"{name}: decode batch 8 {step_s * 1e3:.3f} ms/step ({out['decode_b8']['roofline_frac']} of 8 TB/s), "
        f"prefill {pre_s * 1e3:.2f} ms ({out['prefill']['frac']} of 2.5 PFLOP/s)")
    w = run_workload(name, a, model=model)
    out["workload"] = {k: w[k] for k in ("value", "unit", "workload", "seconds", "generated_tokens", "prompt_tokens",
                                         "all_tokens_per_s", "steps", "preemptions", "launched", "by_kind", "ttft_ms_mean",
                                         "tpot_ms_mean")}
    log(f"{name}: workload {w['value']} generated tok/s, {w['all_tokens_per_s']} tok/s with the prompts")
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--points", default="1,64", help="further decode batch sizes, comma separated")
    ap.add_argument("--model", choices=sorted(MODELS), default="2b", help="layer sizes: Gemma 2 2B (the default), 9B or 27B")
    ap.add_argument("--workload", choices=["9b", "27b"], default=None,
                    help="run one of the larger workloads through Engine.generate instead")
    ap.add_argument("--no-graphs", action="store_true",
                    help="decode steps run eagerly (rocprofv3's kernel trace has crashed on launches of large graphs)")
    ap.add_argument("--no-check", action="store_true", help="profiling aid: skip the check before timing")
    ap.add_argument("--only", choices=["prefill", "decode"], default=None,
                    help="profiling aid: run one of the two workloads (the JSON line then lacks the other)")
    ap.add_argument("--page-size", type=int, default=16, help="tokens a page of the cache holds")
    ap.add_argument("--drawn", action="store_true",
                    help="profiling aid: every timed decode step draws its tokens with the reference's default "
                         "sampling parameters instead of taking the largest logit")
    ap.add_argument("--quick", action="store_true",
                    help="the headline alone: no decode at context 8,192, no 9B and 27B figures")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not measured")
        sys.exit(2)
    if a.workload:
        print(json.dumps(run_workload(a.workload, a)), flush=True)
        return

    from zse_amd.engine.loading import random_model
    from zse_amd.runtime.device import Runtime

    cfg = dict(MODELS[a.model])
    full_layers = cfg["num_hidden_layers"]
    if a.layers:
        cfg["num_hidden_layers"] = a.layers
    rt = Runtime.get()
    SEED, STD, GAIN_STD = 0, 0.02, 0.1

    t0 = time.time()
    model = random_model(cfg, "bfloat16", seed=SEED, std=STD, gain_std=GAIN_STD, rt=rt)
    V = cfg["vocab_size"]
    points = sorted({int(x) for x in a.points.split(",") if x} | {a.batch})
    check = None
    if not a.no_check and not a.only:
        errs = check_slice(cfg, rt, SEED, STD, GAIN_STD)
        same_ids = all(check_decode_path(model, rt, V, B, not a.no_graphs) for B in points)
        # 32-bit: summation order only (2e-5 of the largest logit seen at these widths);
        # bfloat16: inputs of every product rounded to 8 bits (under 1 % seen)
        ok = errs["float32"] < 1e-4 and errs["bfloat16"] < 0.02 and same_ids
        check = {"fp32_max_rel_err": float(f"{errs['float32']:.3g}"), "bf16_max_rel_err": float(f"{errs['bfloat16']:.3g}"),
                 "timed_path_ids_equal_eager": bool(same_ids), "at_batches": points, "slice_layers": 2,
                 "cuts": "whole, portions, token by token, mixed"}
        log(f"check: {check} ({time.time() - t0:.1f} s)")
        if not ok:
            raise SystemExit(f"bench.py: the engine does not agree with the plain implementation: {check}")
    peak_bw, peak_fl = probe_peaks(rt)
    log(f"probes: {peak_bw / 1e9:.0f} GB/s streamed, {peak_fl / 1e12:.0f} TFLOP/s bf16 on the matrix cores")

    max_b = max(points)
    t = Timed(model, rt, cfg, max_b, a.context, a.prefill_tokens, not a.no_graphs, page=a.page_size)
    runner = t.runner
    log(f"model ready in {time.time() - t0:.1f} s: {cfg['num_hidden_layers']} layers, "
        f"{model.weight_bytes / 1e9:.2f} GB of weights, cache {runner.cache_bytes() / 1e9:.2f} GB")

    # ---- prefill: one prompt of 2,048 tokens in one step, and the same prompt in portions of 512
    T = a.prefill_tokens
    prefill = None
    if a.only != "decode":
        pre_s, pf = t.prefill()
        prefill = {"value": round(T / pre_s, 1), "tokens": T, "ms": round(pre_s * 1e3, 3),
                   "frac": round(pf / pre_s / PEAK_FLOPS["bf16"], 4), "frac_probed": round(pf / pre_s / peak_fl, 4)}
        log(f"prefill {T} tokens: {pre_s * 1e3:.2f} ms")
        if T > 512:
            ch_s, ch_f = t.prefill(portion=512)
            prefill["chunked_512"] = {"value": round(T / ch_s, 1), "ms": round(ch_s * 1e3, 3), "steps": -(-T // 512),
                                      "frac": round(ch_f / ch_s / PEAK_FLOPS["bf16"], 4)}
            log(f"prefill {T} tokens in portions of 512: {ch_s * 1e3:.2f} ms")
    if a.only == "prefill":
        print(json.dumps({"prefill": prefill}), flush=True)
        return

    # ---- decode at each batch size, ending at the full context
    results = {}
    for B in points:
        k = a.steps if B == a.batch else max(16, a.steps // 2)
        w = a.warmup if B == a.batch else max(4, a.warmup // 2)
        results[B] = t.decode(B, k, w, drawn=REFERENCE_SAMPLING if a.drawn else None)
        log(f"decode batch {B}: {results[B][0]:.1f} tok/s, {results[B][1] * 1e3:.3f} ms/step, "
            f"{results[B][2] / results[B][1] / 1e9:.0f} GB/s ({results[B][3]})")
    # the same at the reference's default sampling parameters (orchestrator/engine.py:40-43)
    drawn = None
    if not a.only and a.batch in points:
        drawn = t.decode(a.batch, max(16, a.steps // 2), max(4, a.warmup // 2), drawn=REFERENCE_SAMPLING)
        log(f"decode batch {a.batch}, drawn with {REFERENCE_SAMPLING}: {drawn[0]:.1f} tok/s, {drawn[1] * 1e3:.3f} ms/step")
    graph_max_batch = runner.graph_max_batch
    t.close()

    tok_s, step_s, byts, _ = results[a.batch]
    out = {
        "metric": "decode tok/s, Gemma 2 %s bf16, batch %d" % (a.model.upper(), a.batch),
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": dict(shape_of(cfg, full_layers), model=f"gemma2-{a.model}-shapes-random", global_batch=a.batch,
                       sampling="reference defaults" if a.drawn else "greedy",
                       seq_len=a.context, prompt_len=a.prefill_tokens, page_size=a.page_size, parallelism="single-gpu",
                       graphs=int(not a.no_graphs), graph_max_batch=graph_max_batch),
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(byts / step_s / 1e9, 1), "peak": PEAK_HBM / 1e9,
                     "unit": "GB/s", "frac": round(byts / step_s / PEAK_HBM, 4),
                     "frac_probed": round(byts / step_s / peak_bw, 4)},
        "points": {f"decode_b{B}": round(results[B][0], 1) for B in points if B != a.batch},
        "points_roofline_frac": {f"decode_b{B}": round(results[B][2] / results[B][1] / PEAK_HBM, 4) for B in points},
        "points_launched": {f"decode_b{B}": results[B][3] for B in points},
        "drawn": None if drawn is None else dict(REFERENCE_SAMPLING, value=round(drawn[0], 1), batch=a.batch,
                                                   ms_per_step=round(drawn[1] * 1e3, 4)),
        "probed": {"hbm_gbs": round(peak_bw / 1e9, 1), "mfma_bf16_tflops": round(peak_fl / 1e12, 1)},
        "checked": check is not None, "check": check,
    }

    # ---- further sizes: the same model at a context of 8,192 (the window then halves what the
    # sliding layers read), and the 9B and 27B shapes with their workloads
    if not a.quick and not a.only and a.model == "2b" and not a.layers:
        t8 = Timed(model, rt, cfg, max_b, 8192, a.prefill_tokens, not a.no_graphs)
        for B in points:
            r = t8.decode(B, max(16, a.steps // 2), max(4, a.warmup // 2))
            out["points"][f"decode_b{B}_ctx8192"] = round(r[0], 1)
            out["points_roofline_frac"][f"decode_b{B}_ctx8192"] = round(r[2] / r[1] / PEAK_HBM, 4)
            out["points_launched"][f"decode_b{B}_ctx8192"] = r[3]
            log(f"decode batch {B} at context 8192: {r[0]:.1f} tok/s, {r[1] * 1e3:.3f} ms/step, {r[2] / r[1] / 1e9:.0f} GB/s")
        t8.close()
        del t8, t, runner, model
        out["further"] = {}
        for name in ("9b", "27b"):
            out["further"][name] = further_model(name, a, rt, peak_bw, peak_fl)
            out["points"][f"{name}_decode_b8"] = out["further"][name]["decode_b8"]["value"]
            out["points"][f"{name}_prefill_2048"] = out["further"][name]["prefill"]["value"]
            out["points"][f"{name}_workload"] = out["further"][name]["workload"]["value"]
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
