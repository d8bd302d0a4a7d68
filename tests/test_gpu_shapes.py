"""The layer shapes of Gemma 2 2B (hidden 2304, 8 heads over 4 KV heads of 256, intermediate
9216; two layers), 9B (3584, 16 over 8 of 256, 14336; one layer) and 27B (4608, 32 over 16 of
128, scale 144^-1/2, 36864; one layer) with a small vocabulary and a short window, so that the
real-size kernels (head_dim 256 and 128, K from 2048 to 36864) are checked against the plain
implementation in both types."""
import numpy as np
import pytest

from conftest import random_tokens, read_weights
from gpu_util import F32_ATOL, assert_close, bf16_round, chunked_steps, make_runner, run_steps, whole_steps
from plain import gemma2_plain as P

pytestmark = pytest.mark.gpu


def config(layers, hidden, heads, kv_heads, head_dim, qpas, inter):
    return dict(architectures=["Gemma2ForCausalLM"], model_type="gemma2", num_hidden_layers=layers,
                hidden_size=hidden, num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
                query_pre_attn_scalar=qpas, intermediate_size=inter, vocab_size=3000, rope_theta=10000.0,
                sliding_window=48, attn_logit_softcapping=50.0, final_logit_softcapping=30.0, rms_norm_eps=1e-6,
                max_position_embeddings=512)


CONFIGS = {"2b": config(2, 2304, 8, 4, 256, 256, 9216), "9b": config(1, 3584, 16, 8, 256, 256, 14336),
           "27b": config(1, 4608, 32, 16, 128, 144, 36864)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from zse_amd.weights import write_random_model
    out = {}

    def get(size, dtype):
        if (size, dtype) not in out:
            d = str(tmp_path_factory.mktemp(f"shapes_{size}_{dtype}"))
            write_random_model(d, CONFIGS[size], seed=5, std=0.02, gain_std=0.1, dtype=dtype)
            out[(size, dtype)] = d
        return out[(size, dtype)]
    return get


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("size", ["2b", "9b", "27b"])
def test_layer_shapes(folders, size, dtype):
    CFG = CONFIGS[size]
    folder = folders(size, dtype)
    toks = random_tokens(CFG["vocab_size"], 150, 1)
    H = float(CFG["hidden_size"])
    scale = np.sqrt(H) if dtype == "float32" else bf16_round(np.sqrt(H))
    ref = P.forward(CFG, read_weights(folder), toks, np.float64, embed_scale=np.float64(scale))
    runner = make_runner(folder, dtype, page_size=16, cache_tokens=512, max_seqs=4, max_batch_tokens=256,
                         max_model_len=256)
    streams = {"a": toks}
    whole = run_steps(runner, streams, whole_steps(streams))["a"]
    steps = [([("a", 100)], [])] + [([("a", 1)], []) for _ in range(49)] + [([("a", 1)], ["a"])]
    tail = run_steps(runner, streams, steps)["a"]
    chunk = run_steps(runner, streams, chunked_steps(streams, sizes=(70, 2, 33, 5, 40)))["a"]
    if dtype == "float32":
        # sums over thousands of terms (up to 36864): a bound that grows with the length of the sum
        for got, what in ((whole, "whole"), (tail, "tail"), (chunk, "portions")):
            err = np.abs(got - ref).max()
            assert err < 4 * F32_ATOL, f"{what}: {err}"
        assert np.array_equal(whole, tail) and np.array_equal(whole, chunk)
    else:
        for got, what in ((whole, "whole"), (tail, "tail"), (chunk, "portions")):
            assert_close(got, ref, dtype, what)
            agree = np.mean(np.argmax(got, -1) == np.argmax(ref, -1))
            assert agree > 0.9, f"{what}: greedy tokens agree on {agree:.2f} of positions"
