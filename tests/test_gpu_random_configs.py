"""Random small configurations of the architecture through the engine in 32-bit: sizes that no
other test has (head sizes in steps of 16 up to 256, any number of heads and groups, widths and
vocabularies that are no multiple of anything, any window, caps present or absent, an untied
head, pages of 4 to 32 tokens), every way of cutting, against the plain implementation."""
import json
import shutil
import tempfile

import numpy as np
import pytest

from conftest import read_weights
from gpu_util import (F32_ATOL, chunked_steps, make_runner, mixed_steps, run_steps, tail_decode_steps,
                      whole_steps)
from plain import gemma2_plain as P

pytestmark = pytest.mark.gpu


def draw(seed):
    rng = np.random.default_rng(seed)
    nkv = int(rng.choice([1, 2, 3, 4, 5]))
    g = int(rng.choice([1, 2, 3, 4, 6, 8]))
    hd = int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 256]))
    hidden = int(rng.choice([8, 24, 40, 72, 100, 136, 200])) if rng.random() < .7 else int(rng.integers(5, 150))
    inter = int(rng.choice([16, 40, 72, 136, 328])) if rng.random() < .7 else int(rng.integers(5, 300))
    cfg = dict(architectures=["Gemma2ForCausalLM"], model_type="gemma2",
               num_hidden_layers=int(rng.integers(1, 4)), hidden_size=hidden, num_attention_heads=nkv * g,
               num_key_value_heads=nkv, head_dim=hd, query_pre_attn_scalar=int(rng.choice([hd, 24, 100, 224])),
               intermediate_size=inter, vocab_size=int(rng.integers(40, 1200)),
               rope_theta=float(rng.choice([10000.0, 50000.0, 1e6])), sliding_window=int(rng.integers(3, 60)),
               attn_logit_softcapping=(None if rng.random() < .25 else float(rng.choice([10.0, 30.0, 50.0]))),
               final_logit_softcapping=(None if rng.random() < .25 else float(rng.choice([15.0, 30.0]))),
               rms_norm_eps=float(rng.choice([1e-6, 1e-5, 3e-4])), max_position_embeddings=512)
    if rng.random() < .3:
        cfg["tie_word_embeddings"] = False
    return cfg, int(rng.choice([4, 8, 16, 32]))


@pytest.mark.parametrize("seed", range(8))
def test_a_random_configuration_in_every_cut(seed):
    from zse_amd.weights import write_random_model
    cfg, page = draw(seed)
    print(f"seed {seed}, pages of {page}: " + json.dumps(cfg), flush=True)
    folder = tempfile.mkdtemp(prefix="zse_random_config_")
    try:
        write_random_model(folder, cfg, seed=seed, std=0.08, gain_std=0.2, dtype="float32",
                           std_of={"embed_tokens": 0.02})
        weights = read_weights(folder)
        rng = np.random.default_rng(seed + 1000)
        streams = {f"r{i}": rng.integers(0, cfg["vocab_size"], int(rng.integers(34, 90))).tolist() for i in range(4)}
        scale = np.float64(np.float32(np.sqrt(cfg["hidden_size"])))
        want = {r: P.forward(cfg, weights, t, np.float64, embed_scale=scale) for r, t in streams.items()}
        pages = sum(-(-len(t) // page) for t in streams.values())
        # room for the two longest requests and a little more: pages go round in the mixed cut
        room = sorted(-(-len(t) // page) for t in streams.values())[-2:]
        pool = sum(room) + 2
        runner = make_runner(folder, "float32", page_size=page, num_pages=pool, max_seqs=4,
                             max_batch_tokens=256, max_model_len=128)
        assert pool < pages
        first = None
        for cut, steps in (("whole", whole_steps(streams)), ("last 16 one by one", tail_decode_steps(streams, 16)),
                           ("portions", chunked_steps(streams)),
                           ("mixed", mixed_steps(streams, seed=seed, room=pool, page=page))):
            got = run_steps(runner, streams, steps)
            for r in streams:
                err = np.abs(got[r] - want[r]).max()
                assert err <= F32_ATOL, f"{cut}, request {r}: error {err:.3e}"
            if first is None:
                first = got
            else:
                for r in streams:
                    assert np.array_equal(first[r], got[r]), f"{cut}, request {r}: differs from the whole prompt's bits"
    finally:
        shutil.rmtree(folder, ignore_errors=True)
