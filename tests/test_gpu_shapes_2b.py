"""The layer shapes of Gemma 2 2B (hidden 2304, 8 heads over 4 KV heads of 256, intermediate
9216) with two layers, a small vocabulary and a short window, so that the real-size kernels
(head_dim 256, K = 2304 / 9216) are checked against the plain implementation in both types."""
import numpy as np
import pytest

from conftest import random_tokens, read_weights
from gpu_util import F32_ATOL, assert_close, bf16_round, chunked_steps, make_runner, run_steps, whole_steps
from plain import gemma2_plain as P

pytestmark = pytest.mark.gpu

CFG = dict(architectures=["Gemma2ForCausalLM"], model_type="gemma2", num_hidden_layers=2, hidden_size=2304,
           num_attention_heads=8, num_key_value_heads=4, head_dim=256, query_pre_attn_scalar=256,
           intermediate_size=9216, vocab_size=3000, rope_theta=10000.0, sliding_window=48,
           attn_logit_softcapping=50.0, final_logit_softcapping=30.0, rms_norm_eps=1e-6,
           max_position_embeddings=512)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from zse_amd.weights import write_random_model
    out = {}
    for dtype in ("float32", "bfloat16"):
        d = str(tmp_path_factory.mktemp(f"shapes2b_{dtype}"))
        write_random_model(d, CFG, seed=5, std=0.02, gain_std=0.1, dtype=dtype)
        out[dtype] = d
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_2b_layer_shapes(folders, dtype):
    folder = folders[dtype]
    toks = random_tokens(CFG["vocab_size"], 150, 1)
    scale = np.sqrt(2304.0) if dtype == "float32" else bf16_round(np.sqrt(2304.0))
    ref = P.forward(CFG, read_weights(folder), toks, np.float64, embed_scale=np.float64(scale))
    runner = make_runner(folder, dtype, page_size=16, cache_tokens=512, max_seqs=4, max_batch_tokens=256,
                         max_model_len=256)
    streams = {"a": toks}
    whole = run_steps(runner, streams, whole_steps(streams))["a"]
    steps = [([("a", 100)], [])] + [([("a", 1)], []) for _ in range(49)] + [([("a", 1)], ["a"])]
    tail = run_steps(runner, streams, steps)["a"]
    chunk = run_steps(runner, streams, chunked_steps(streams, sizes=(70, 2, 33, 5, 40)))["a"]
    if dtype == "float32":
        # sums over 2304 and 9216 terms: a bound that grows with the length of the sum
        for got, what in ((whole, "whole"), (tail, "tail"), (chunk, "portions")):
            err = np.abs(got - ref).max()
            assert err < 4 * F32_ATOL, f"{what}: {err}"
        assert np.array_equal(whole, tail) and np.array_equal(whole, chunk)
    else:
        for got, what in ((whole, "whole"), (tail, "tail"), (chunk, "portions")):
            assert_close(got, ref, dtype, what)
            agree = np.mean(np.argmax(got, -1) == np.argmax(ref, -1))
            assert agree > 0.9, f"{what}: greedy tokens agree on {agree:.2f} of positions"
