"""Engine.generate on random configurations with random requests, sampling options, portion
sizes, batch limits and small pools, in 32-bit: every request's tokens are those it gets alone
in an engine with room, whatever the scheduler had to do (portions, waiting, preemption and
recomputation, runs of decode steps, graphs)."""
import json
import shutil
import tempfile

import numpy as np
import pytest

from test_gpu_random_configs import draw

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", range(6))
def test_random_requests_under_random_limits(seed):
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling.sampler import SamplingParams
    from zse_amd.weights import write_random_model
    cfg, page = draw(seed)
    rng = np.random.default_rng(seed + 5000)
    nreq = int(rng.integers(3, 12))
    prompts = [rng.integers(0, cfg["vocab_size"], int(rng.integers(1, 70))).tolist() for _ in range(nreq)]
    params = []
    for _ in range(nreq):
        greedy = rng.random() < .5
        stop = [int(x) for x in rng.integers(0, cfg["vocab_size"], int(rng.integers(0, 40)))] if rng.random() < .5 else None
        params.append(SamplingParams(max_tokens=int(rng.integers(1, 24)),
                                     temperature=0.0 if greedy else float(rng.choice([0.7, 1.0, 1.3])),
                                     top_k=int(rng.choice([0, 0, 5, 40])), top_p=float(rng.choice([1.0, 1.0, 0.9, 0.5])),
                                     repetition_penalty=float(rng.choice([1.0, 1.0, 1.2])), stop_tokens=stop,
                                     seed=int(rng.integers(0, 1 << 30))))
    need = -(-max(len(p) + sp.max_tokens for p, sp in zip(prompts, params)) // page)
    limits = dict(block_size=page, num_blocks=int(need + rng.integers(0, 2 * need + 2)),
                  max_batch_tokens=int(rng.choice([16, 33, 64, 256])), max_batch_seqs=int(rng.choice([1, 2, 3, 5, 8])),
                  prefill_chunk_size=int(rng.choice([2, 7, 16, 64])), decode_run=int(rng.choice([1, 2, 4])),
                  use_graphs=bool(rng.random() < .6), max_seq_len=128)
    print(f"seed {seed}: {json.dumps(limits)}, {nreq} requests, " + json.dumps(cfg), flush=True)
    folder = tempfile.mkdtemp(prefix="zse_random_engine_")
    try:
        write_random_model(folder, cfg, seed=seed, std=0.08, gain_std=0.2, dtype="float32",
                           std_of={"embed_tokens": 0.02})
        eng = Engine(folder, dtype="float32", **limits)
        outs = eng.generate(prompts, params)
        eng.runner.manager.check()
        st = eng.runner.manager.stats()
        assert st["live"] == 0 and all(g["free"] == g["pages"] for g in st["groups"]), st
        eng.close()
        roomy = Engine(folder, dtype="float32", block_size=page, max_batch_seqs=2, max_seq_len=128,
                       use_graphs=False, decode_run=1)
        for i, (p, sp) in enumerate(zip(prompts, params)):
            alone = roomy.generate([p], sp)[0]
            assert list(alone) == list(outs[i]), f"request {i} ({len(p)} prompt tokens, {sp})"
        roomy.close()
    finally:
        shutil.rmtree(folder, ignore_errors=True)
