#!/usr/bin/env python3
"""Decode and prefill throughput of Gemma 2 2B layer shapes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B]

A step is one decode step of the whole batch: every live request brings one token, the
model runs from the cache, the next token is picked greedily on the device.  Weights are
seeded random values, token ids are synthetic.  One JSON line comes out; its ``value`` is
decoded tokens a second at the default batch, ``points`` holds batch 1 and 64, ``prefill``
one 2,048-token prompt in one step, ``roofline`` the decode step's bytes over its time.
"""
import argparse
import json
import sys
import time

import numpy as np

PEAK_HBM = 8.0e12          # bytes/s, MI355X
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

GEMMA2_2B = dict(
    architectures=["Gemma2ForCausalLM"], model_type="gemma2", num_hidden_layers=26, hidden_size=2304,
    num_attention_heads=8, num_key_value_heads=4, head_dim=256, query_pre_attn_scalar=256,
    intermediate_size=9216, vocab_size=256000, rope_theta=10000.0, sliding_window=4096,
    attn_logit_softcapping=50.0, final_logit_softcapping=30.0, rms_norm_eps=1e-6,
    max_position_embeddings=8192)


# further sizes of the same architecture, for looking beyond the default (--model)
GEMMA2_9B = dict(GEMMA2_2B, num_hidden_layers=42, hidden_size=3584, num_attention_heads=16, num_key_value_heads=8,
                 head_dim=256, query_pre_attn_scalar=256, intermediate_size=14336)
GEMMA2_27B = dict(GEMMA2_2B, num_hidden_layers=46, hidden_size=4608, num_attention_heads=32, num_key_value_heads=16,
                  head_dim=128, query_pre_attn_scalar=144, intermediate_size=36864)
MODELS = {"2b": GEMMA2_2B, "9b": GEMMA2_9B, "27b": GEMMA2_27B}


def weight_bytes(cfg, item=2):
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv, hd, L = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["num_hidden_layers"]
    per_layer = (nh + 2 * nkv) * hd * H + H * nh * hd + 3 * I * H
    return (L * per_layer + V * H) * item


def cache_bytes(cfg, ctx, item=2):
    """Bytes of keys and values one request's decode step reads at context ``ctx``."""
    nkv, hd, L, W = cfg["num_key_value_heads"], cfg["head_dim"], cfg["num_hidden_layers"], cfg["sliding_window"]
    total = 0
    for l in range(L):
        seen = min(ctx, W) if (l % 2 == 0 and W) else ctx
        total += 2 * nkv * hd * seen * item
    return total


def prefill_flops(cfg, T):
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv, hd, L, W = (cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"],
                         cfg["num_hidden_layers"], cfg["sliding_window"])
    per_layer = (nh + 2 * nkv) * hd * H + H * nh * hd + 3 * I * H
    gemm = 2.0 * T * per_layer * L
    attn = 0.0
    for l in range(L):
        w = W if (l % 2 == 0 and W) else T
        keys = sum(min(i + 1, w) for i in range(T))
        attn += 4.0 * nh * hd * keys
    return gemm + attn + 2.0 * V * H


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
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--only", choices=["prefill", "decode"], default=None,
                    help="profiling aid: run one of the two workloads (the JSON line then lacks the other)")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not measured")
        sys.exit(2)

    from zse_amd.engine.loading import random_model
    from zse_amd.engine.runner import StepEntry, StepRunner
    from zse_amd.runtime.device import Runtime
    from zse_amd.sampling.sampler import DeviceSampler, SamplingParams

    cfg = dict(MODELS[a.model])
    full_layers = cfg["num_hidden_layers"]
    if a.layers:
        cfg["num_hidden_layers"] = a.layers
    rt = Runtime.get()
    t0 = time.time()
    model = random_model(cfg, "bfloat16", seed=0, std=0.02, gain_std=0.1, rt=rt)
    points = sorted({int(x) for x in a.points.split(",") if x} | {a.batch})
    max_b = max(points)
    page = 16
    longest = max(a.context, a.prefill_tokens)       # a prompt longer than the decode context still fits
    runner = StepRunner(model, rt, "bfloat16", page_size=page,
                        num_pages=max(max_b * (-(-a.context // page) + 1), -(-longest // page)) + 8, max_seqs=max_b,
                        max_batch_tokens=max(a.prefill_tokens, max_b), max_model_len=longest,
                        use_graphs=not a.no_graphs)
    sampler = DeviceSampler(rt, runner.k, max_b)
    greedy = SamplingParams(temperature=0.0)
    V = cfg["vocab_size"]
    rng = np.random.default_rng(0)
    print(f"[bench] model ready in {time.time() - t0:.1f} s: {cfg['num_hidden_layers']} layers, "
          f"{model.weight_bytes / 1e9:.2f} GB of weights, cache {runner.cache_bytes() / 1e9:.2f} GB",
          file=sys.stderr, flush=True)

    # ---- prefill: one prompt of 2,048 tokens in one step
    T = a.prefill_tokens
    times = []
    for i in range(4 if a.only != "decode" else 0):
        toks = rng.integers(0, V, T).tolist()
        rt.sync()
        t1 = time.perf_counter()
        runner.step([StepEntry(f"p{i}", toks, [T - 1])], download=False)
        rt.sync()
        times.append(time.perf_counter() - t1)
        runner.finish(f"p{i}")
    prefill = None
    if times:
        pre_s = float(np.median(times[1:]))
        pf = prefill_flops(cfg, T)
        prefill = {"value": round(T / pre_s, 1), "tokens": T, "ms": round(pre_s * 1e3, 3),
                   "frac": round(pf / pre_s / PEAK_FLOPS["bf16"], 4)}
        print(f"[bench] prefill {T} tokens: {pre_s * 1e3:.2f} ms", file=sys.stderr, flush=True)
    if a.only == "prefill":
        print(json.dumps({"prefill": prefill}), flush=True)
        return

    # ---- decode at each batch size, ending at the full context
    def decode(B, steps, warmup):
        ctx0 = a.context - steps - warmup
        reqs = [f"d{B}_{i}" for i in range(B)]
        for r in reqs:                       # fill the cache through real prefill steps
            left = ctx0
            while left > 0:
                n = min(left, T)
                runner.step([StepEntry(r, rng.integers(0, V, n).tolist(), [])], download=False)
                left -= n
        first = rng.integers(0, V, B).tolist()
        rows = [{"params": greedy, "u": 0.0} for _ in range(B)]
        # As the engine decodes: the sampling kernel leaves the ids on the device, the next step
        # takes them from there, and the host reads them four steps at a time (it has to, for
        # stop tokens) while the next steps are already enqueued.
        sampler.prepare_run(rows, [[0.0] * B])
        pending, fed = [], None

        def one():
            nonlocal fed
            toks = first if fed is None else [0] * B
            logits = runner.step([StepEntry(r, [t], [0]) for r, t in zip(reqs, toks)], download=False,
                                 tokens_from=fed)
            ids = sampler.sample_deferred(logits, 0)
            fed = ids.device_ptr
            pending.append(ids)
            if len(pending) == 4:
                for p in pending:
                    p.result()
                pending.clear()
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
        mean_ctx = a.context - steps / 2.0
        byts = weight_bytes(cfg) + B * cache_bytes(cfg, int(mean_ctx))
        return B * steps / dt, dt / steps, byts

    results = {}
    for B in points:
        k = a.steps if B == a.batch else max(16, a.steps // 2)
        w = a.warmup if B == a.batch else max(4, a.warmup // 2)
        results[B] = decode(B, k, w)
        print(f"[bench] decode batch {B}: {results[B][0]:.1f} tok/s, {results[B][1] * 1e3:.3f} ms/step, "
              f"{results[B][2] / results[B][1] / 1e9:.0f} GB/s", file=sys.stderr, flush=True)

    tok_s, step_s, byts = results[a.batch]
    out = {
        "metric": "decode tok/s, Gemma 2 %s bf16, batch %d" % (a.model.upper(), a.batch),
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"model": f"gemma2-{a.model}-shapes-random", "layers": cfg["num_hidden_layers"],
                   "layers_full": full_layers, "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"],
                   "sliding_window": cfg["sliding_window"], "global_batch": a.batch, "seq_len": a.context,
                   "prompt_len": a.prefill_tokens, "page_size": page, "parallelism": "single-gpu",
                   "graphs": int(runner.use_graphs)},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(byts / step_s / 1e9, 1), "peak": PEAK_HBM / 1e9,
                     "unit": "GB/s", "frac": round(byts / step_s / PEAK_HBM, 4)},
        "points": {f"decode_b{B}": round(results[B][0], 1) for B in points if B != a.batch},
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
