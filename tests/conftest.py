import os
import sys

import numpy as np
import pytest

ROOT = os.path.normpath(os.path.join(os.path.dirname(__file__), ".."))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
if os.path.dirname(__file__) not in sys.path:
    sys.path.insert(0, os.path.dirname(__file__))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


# Two tiny configurations that differ in every size and option.
TINY_A = dict(
    architectures=["Gemma2ForCausalLM"], model_type="gemma2",
    num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
    query_pre_attn_scalar=16, intermediate_size=128, vocab_size=512, rope_theta=10000.0,
    sliding_window=8, attn_logit_softcapping=50.0, final_logit_softcapping=30.0, rms_norm_eps=1e-6,
    max_position_embeddings=512)
TINY_B = dict(
    architectures=["Gemma2ForCausalLM"], model_type="gemma2",
    num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=1, head_dim=32,
    query_pre_attn_scalar=24, intermediate_size=320, vocab_size=1000, rope_theta=100000.0,
    sliding_window=16, attn_logit_softcapping=20.0, final_logit_softcapping=15.0, rms_norm_eps=1e-5,
    max_position_embeddings=1024)
# weights are drawn wider than a checkpoint's so that attention is not near-uniform
TINY = {"A": (TINY_A, 0, 0.05, 0.1), "B": (TINY_B, 1, 0.08, 0.2)}


@pytest.fixture(scope="session")
def tiny_folders(tmp_path_factory):
    """{(name, storage dtype): folder} of random tiny models, written once a session."""
    from zse_amd.weights import write_random_model
    out = {}
    for name, (cfg, seed, std, gstd) in TINY.items():
        for dtype in ("float32", "bfloat16"):
            d = str(tmp_path_factory.mktemp(f"tiny{name}_{dtype}"))
            # a small embedding keeps the tied head from simply echoing the last token
            write_random_model(d, cfg, seed=seed, std=std, gain_std=gstd, dtype=dtype,
                               std_of={"embed_tokens": std / 4})
            out[(name, dtype)] = d
    return out


def read_weights(folder):
    from zse_amd.weights.safetensors import read_folder_f32
    return read_folder_f32(folder)


def random_tokens(vocab, n, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()
