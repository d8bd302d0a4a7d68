"""Trace replay: feed given token ids step by step, write logits, sample nothing.

The program owns no forward pass, cache or loader: it builds ``StepEntry``
lists for the engine's ``StepRunner`` and ends requests through it.  The
reference has nothing comparable; its closest test calls ``runner.prefill`` once
and compares one row (tests/test_modal_gemma4_parity.py:62-70).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Iterable, Optional

import numpy as np


def replay(runner, lines: Iterable[str], out_dir: str, log=None) -> int:
    from .runner import StepEntry
    os.makedirs(out_dir, exist_ok=True)
    n = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [StepEntry(e["id"], e["tokens"], e.get("want", ())) for e in rec.get("entries", [])]
        logits = runner.step(entries)
        if logits.shape[0] > 0:
            path = os.path.join(out_dir, f"{step}.f32")
            logits.astype("<f4", copy=False).tofile(path + ".tmp")
            os.replace(path + ".tmp", path)
        for rid in rec.get("end", []):
            runner.finish(rid)
        if log is not None:
            print(f"done {step}", file=log, flush=True)
        n += 1
    return n


def main(argv: Optional[list] = None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--max-seqs", type=int, default=8)
    ap.add_argument("--plain", action="store_true",
                    help="bfloat16 only: the plain kernels instead of the tuned ones")
    a = ap.parse_args(argv)

    from ..runtime.device import Runtime
    from .loading import load_model
    from .runner import StepRunner

    print(f"[trace_run] loading {a.model} as {a.dtype}", file=sys.stderr, flush=True)
    rt = Runtime.get()
    model = load_model(a.model, a.dtype, rt, tuned=not a.plain)
    max_len = min(model.plan.max_position, max(a.max_tokens, 64))
    runner = StepRunner(model, rt, a.dtype, page_size=a.block_size, cache_tokens=a.max_tokens,
                        max_seqs=a.max_seqs, max_batch_tokens=max(a.max_tokens, 64),
                        max_model_len=max_len, use_graphs=False)
    print(f"[trace_run] ready: {model.plan.architecture}, {len(model.plan.order)} layer calls, "
          f"pages of {a.block_size}", file=sys.stderr, flush=True)
    replay(runner, sys.stdin, a.out, log=sys.stdout)
    return 0
