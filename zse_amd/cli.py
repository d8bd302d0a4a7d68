"""Command line: ``zse generate``, ``zse replay``, ``zse bench``, ``zse info``, ``zse version``,
``zse random-weights``, ``zse build``.

The reference's ``zse`` has ``serve``, ``convert``, ``info``, ``version``,
``warm`` and ``keys`` (cli.py:220-281) and no command that generates; ``info``
and ``version`` are kept with their meaning, ``generate`` takes its options'
names from the reference's generation call (orchestrator/engine.py:263-288:
max_tokens, temperature, top_p, top_k, repetition_penalty, stop_tokens, seed)
and ``--quiet`` from its commands.  ``python -m zse_amd`` is the same program
(as __main__.py:1-3 there).
"""
from __future__ import annotations

import argparse
import json
import sys

from . import __version__


def _ids(text: str):
    return [int(t) for t in text.replace(",", " ").split()]


def _cmd_generate(a):
    from .engine.engine import Engine
    from .sampling.sampler import SamplingParams
    prompts = []
    if a.prompt_ids:
        prompts.append(_ids(a.prompt_ids))
    if a.prompt_ids_file:
        with open(a.prompt_ids_file) as f:
            for line in f:
                if line.strip():
                    prompts.append(_ids(line))
    if not prompts:
        print("zse generate: give --prompt-ids or --prompt-ids-file", file=sys.stderr)
        return 2
    model = a.model
    if a.random_weights:
        # the weights are drawn on the device, in place: nothing is written (a folder made by
        # ``zse random-weights`` from the same config and seed holds the same values)
        from .config.base import read_config_json
        from .engine.loading import random_model
        model = random_model(read_config_json(a.model), a.dtype, seed=a.weight_seed)
    eng = Engine(model, dtype=a.dtype, block_size=a.block_size, num_blocks=a.num_blocks,
                 max_batch_tokens=a.max_batch_tokens, max_batch_seqs=a.max_batch_seqs,
                 prefill_chunk_size=a.prefill_chunk_size, max_seq_len=a.max_seq_len, quiet=a.quiet)
    sp = SamplingParams(max_tokens=a.max_tokens, temperature=a.temperature, top_p=a.top_p,
                        top_k=a.top_k, repetition_penalty=a.repetition_penalty,
                        stop_tokens=_ids(a.stop_tokens) if a.stop_tokens else None, seed=a.seed)
    outs = eng.generate(prompts, sp)
    for o in outs:
        print(" ".join(str(t) for t in o))
    if not a.quiet:
        s = eng.stats()
        print(f"[zse] {s.generated_tokens} tokens in {s.steps} steps, {s.seconds:.3f} s, "
              f"{s.tokens_per_second:.1f} tok/s, {s.preemptions} preemptions", file=sys.stderr)
    return 0


def _cmd_replay(a):
    from .engine.replay import main as replay_main
    argv = ["--model", a.model, "--dtype", a.dtype, "--out", a.out, "--max-tokens", str(a.max_tokens),
            "--block-size", str(a.block_size)]
    if a.trace:
        sys.stdin = open(a.trace)
    return replay_main(argv)


def _cmd_bench(a, rest):
    """The measurement harness: ``bench.py`` beside the package, with its own options."""
    import os
    import runpy
    path = os.path.normpath(os.path.join(os.path.dirname(__file__), "..", "bench.py"))
    if not os.path.isfile(path):
        print(f"zse bench: {path} is not there (the harness ships with the source tree)", file=sys.stderr)
        return 2
    sys.argv = [path] + list(rest)
    runpy.run_path(path, run_name="__main__")
    return 0


def _cmd_info(a):
    from .runtime.device import Runtime
    i = Runtime.get().info()
    print(json.dumps({"name": i.name, "arch": i.arch, "total_memory": i.total_memory,
                      "free_memory": i.free_memory, "compute_units": i.compute_units}, indent=1))
    return 0


def _cmd_version(a):
    print(f"zse_amd {__version__}")
    return 0


def _cmd_random_weights(a):
    from .weights.random_init import write_random_model
    with open(a.config) as f:
        cfg = json.load(f)
    write_random_model(a.out, cfg, seed=a.seed, std=a.std, gain_std=a.gain_std, dtype=a.dtype)
    print(a.out)
    return 0


def _cmd_build(a):
    from .runtime import build
    build.build_all()
    return 0


def main(argv=None):
    ap = argparse.ArgumentParser(prog="zse", description="zse_amd: a small MI355X inference engine")
    sub = ap.add_subparsers(dest="command")

    g = sub.add_parser("generate", help="generate token ids from prompts of token ids")
    g.add_argument("model", help="folder with config.json and *.safetensors")
    g.add_argument("--prompt-ids", help="token ids, separated by commas or blanks")
    g.add_argument("--prompt-ids-file", help="one prompt of token ids a line")
    g.add_argument("--max-tokens", type=int, default=128)
    g.add_argument("--temperature", type=float, default=1.0, help="0 = greedy")
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--top-k", type=int, default=0)
    g.add_argument("--repetition-penalty", type=float, default=1.0)
    g.add_argument("--stop-tokens", help="token ids that end a request")
    g.add_argument("--seed", type=int, default=None)
    g.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "bf16", "float32", "fp32"])
    g.add_argument("--block-size", type=int, default=16)
    g.add_argument("--num-blocks", type=int, default=None)
    g.add_argument("--max-batch-tokens", type=int, default=4096)
    g.add_argument("--max-batch-seqs", type=int, default=64)
    g.add_argument("--prefill-chunk-size", type=int, default=512)
    g.add_argument("--max-seq-len", type=int, default=None)
    g.add_argument("--random-weights", action="store_true",
                   help="ignore the folder's weights: use its config.json with seeded random ones")
    g.add_argument("--weight-seed", type=int, default=0)
    g.add_argument("--quiet", "-q", action="store_true")

    r = sub.add_parser("replay", help="feed a trace of token ids step by step and write logits")
    r.add_argument("model")
    r.add_argument("--trace", help="file of JSON steps (default: standard input)")
    r.add_argument("--out", required=True)
    r.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    r.add_argument("--max-tokens", type=int, required=True)
    r.add_argument("--block-size", type=int, default=16)

    sub.add_parser("info", help="show the GPU")
    sub.add_parser("version", help="show the version")

    w = sub.add_parser("random-weights", help="write a model folder with seeded random weights")
    w.add_argument("config", help="a config.json")
    w.add_argument("out")
    w.add_argument("--seed", type=int, default=0)
    w.add_argument("--std", type=float, default=0.02)
    w.add_argument("--gain-std", type=float, default=0.1)
    w.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])

    sub.add_parser("build", help="compile the native libraries for gfx950")
    sub.add_parser("bench", help="decode and prefill throughput (options as bench.py's, after the command)",
                   add_help=False)

    argv = list(sys.argv[1:] if argv is None else argv)
    if argv and argv[0] == "bench":
        sys.exit(_cmd_bench(None, argv[1:]) or 0)
    a = ap.parse_args(argv)
    if not a.command:
        ap.print_help()
        sys.exit(0)
    rc = {"generate": _cmd_generate, "replay": _cmd_replay, "info": _cmd_info, "version": _cmd_version,
          "random-weights": _cmd_random_weights, "build": _cmd_build}[a.command](a)
    sys.exit(rc or 0)
