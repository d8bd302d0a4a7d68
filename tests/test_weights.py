"""safetensors reading and writing, random-weights mode, and weight errors (no GPU)."""
import json
import os

import numpy as np
import pytest

from conftest import TINY_A, TINY_B
from zse_amd.engine.model import Model
from zse_amd.models.gemma2 import Gemma2Config, gemma2_plan
from zse_amd.weights import WeightError, check_folder, write_random_model
from zse_amd.weights import safetensors as st


def reqs_of(cfg):
    return Model(gemma2_plan(Gemma2Config.from_dict(cfg))).tensor_reqs()


def test_bf16_round_to_nearest_even():
    x = np.array([1.0, 1.00390625, 1.01171875, -2.5, 3.0e38, 0.0, 1e-40], dtype=np.float32)
    b = st.f32_to_bf16_bits(x)
    back = st.bf16_bits_to_f32(b)
    # 1 + 2^-8 is a tie between 1 and 1 + 2^-7: goes to the even mantissa (1.0);
    # 1 + 3*2^-8 is a tie between 1 + 2^-7 and 1 + 2^-6: goes to 1 + 2^-6
    assert back[0] == 1.0 and back[1] == 1.0 and back[2] == 1.015625 and back[3] == -2.5
    assert np.all(np.abs(back[:5] - x[:5]) <= np.abs(x[:5]) * 2.0 ** -8)
    assert np.isnan(st.bf16_bits_to_f32(st.f32_to_bf16_bits(np.array([np.nan], np.float32))))[0]


def test_round_trip_and_header(tmp_path):
    a = np.arange(12, dtype=np.float32).reshape(3, 4)
    b = st.f32_to_bf16_bits(np.linspace(-1, 1, 10, dtype=np.float32))
    p = str(tmp_path / "x.safetensors")
    st.write_file(p, {"a": ("F32", a), "b": ("BF16", b)}, metadata={"k": "v"})
    h = st.read_header(p)
    assert set(h) == {"a", "b"} and h["a"].shape == (3, 4) and h["b"].dtype == "BF16"
    assert np.array_equal(st.map_tensor(h["a"]), a)
    assert np.array_equal(st.map_tensor(h["b"]), b)
    with open(p, "rb") as f:
        n = int.from_bytes(f.read(8), "little")
        assert "__metadata__" in json.loads(f.read(n))


def test_reader_against_a_file_built_by_hand(tmp_path):
    """The reader pinned without the writer: the bytes are put together here with struct.pack,
    from the format's description as the reference reads it (format/convert.py:51-82: 8-byte
    little-endian header length, JSON header, data_offsets relative to the end of the header,
    __metadata__ skipped).  Offsets are out of order and the header is padded with spaces, as
    real files are."""
    import struct
    f32 = [1.5, -2.0, 0.25, 3.0, 100.0, -0.125]                       # [2, 3] row-major
    bf = [0x3F80, 0xC000, 0x3E80, 0x4049]                             # 1.0, -2.0, 0.25, 3.140625
    f16 = [0x3C00, 0xB800]                                            # 1.0, -0.5
    data_bf = struct.pack("<4H", *bf)
    data_f32 = struct.pack("<6f", *f32)
    data_f16 = struct.pack("<2H", *f16)
    data = data_bf + data_f32 + data_f16                              # bf16 first in the file, listed last
    header = {
        "__metadata__": {"format": "pt"},
        "w.f32": {"dtype": "F32", "shape": [2, 3], "data_offsets": [8, 32]},
        "w.f16": {"dtype": "F16", "shape": [2], "data_offsets": [32, 36]},
        "w.bf16": {"dtype": "BF16", "shape": [4, 1], "data_offsets": [0, 8]},
    }
    text = json.dumps(header).encode()
    text += b" " * (-len(text) % 8)
    p = tmp_path / "model.safetensors"
    p.write_bytes(struct.pack("<Q", len(text)) + text + data)
    h = st.read_header(str(p))
    assert set(h) == {"w.f32", "w.f16", "w.bf16"}
    assert h["w.f32"].shape == (2, 3) and h["w.bf16"].shape == (4, 1) and h["w.f16"].dtype == "F16"
    assert np.array_equal(st.map_tensor(h["w.f32"]), np.array(f32, np.float32).reshape(2, 3))
    assert st.map_tensor(h["w.bf16"]).reshape(-1).tolist() == bf
    w = st.read_folder_f32(str(tmp_path))
    assert w["w.bf16"].reshape(-1).tolist() == [1.0, -2.0, 0.25, 3.140625]
    assert w["w.f16"].tolist() == [1.0, -0.5]
    assert w["w.f32"][1].tolist() == [3.0, 100.0, -0.125]
    # a header that points past the end of the file, or whose size disagrees with its shape
    bad = dict(header)
    bad["w.f32"] = {"dtype": "F32", "shape": [2, 3], "data_offsets": [8, 30]}
    text2 = json.dumps(bad).encode()
    (tmp_path / "model.safetensors").write_bytes(struct.pack("<Q", len(text2)) + text2 + data)
    with pytest.raises(Exception):
        st.map_tensor(st.read_header(str(p))["w.f32"])


def test_no_safetensors_file_is_an_error(tmp_path):
    with pytest.raises(FileNotFoundError):
        st.index_folder(str(tmp_path))


def test_random_weights_folder_matches_the_model(tmp_path):
    for name, cfg in (("a", TINY_A), ("b", TINY_B)):
        d = write_random_model(str(tmp_path / name), cfg, seed=3, dtype="bfloat16")
        assert os.path.isfile(os.path.join(d, "config.json"))
        entries = check_folder(d, reqs_of(cfg))
        L = cfg["num_hidden_layers"]
        assert len(entries) == 2 + 11 * L          # embedding, final norm, 7 matrices + 4 norms a layer
        w = st.read_folder_f32(d)
        e = w["model.embed_tokens.weight"]
        assert e.shape == (cfg["vocab_size"], cfg["hidden_size"])
        assert abs(float(e.std()) - 0.02) < 0.002
        g = w["model.layers.0.input_layernorm.weight"]
        assert abs(float(g.std()) - 0.1) < 0.05
    # same seed, same values; another seed, other values; float32 storage holds the unrounded ones
    d2 = write_random_model(str(tmp_path / "a2"), TINY_A, seed=3, dtype="bfloat16")
    d3 = write_random_model(str(tmp_path / "a3"), TINY_A, seed=4, dtype="bfloat16")
    d4 = write_random_model(str(tmp_path / "a4"), TINY_A, seed=3, dtype="float32")
    wa, w2, w3, w4 = (st.read_folder_f32(str(x)) for x in (tmp_path / "a", d2, d3, d4))
    k = "model.layers.1.mlp.down_proj.weight"
    assert np.array_equal(wa[k], w2[k]) and not np.array_equal(wa[k], w3[k])
    assert np.array_equal(st.bf16_bits_to_f32(st.f32_to_bf16_bits(w4[k])), wa[k])


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=0, dtype="float32")
    w = st.read_folder_f32(d)
    del w["model.layers.0.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.1.self_attn.q_proj.weight"] = np.zeros((64, 63), np.float32)
    w["model.layers.0.self_attn.rotary_emb.inv_freq"] = np.zeros(8, np.float32)
    w["lm_head.weight"] = np.zeros((512, 64), np.float32)     # tied model: not expected
    st.write_file(os.path.join(d, "model.safetensors"), {n: ("F32", a) for n, a in w.items()})
    with pytest.raises(WeightError) as e:
        check_folder(d, reqs_of(TINY_A))
    err = e.value
    assert err.missing == ["model.layers.0.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["lm_head.weight", "model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert err.wrong_shape == [("model.layers.1.self_attn.q_proj.weight", (64, 63), (64, 64))]
    for s in ("up_proj", "model.norm.weight", "inv_freq", "lm_head.weight", "(64, 63)", "(64, 64)"):
        assert s in str(err)


def test_names_match_with_or_without_model_prefix(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=0, dtype="float32")
    w = st.read_folder_f32(d)
    stripped = {(n[6:] if n.startswith("model.") else n): ("F32", a) for n, a in w.items()}
    st.write_file(os.path.join(d, "model.safetensors"), stripped)
    assert len(check_folder(d, reqs_of(TINY_A))) == len(w)


def test_the_optional_prefix_is_the_plans_to_name(tmp_path):
    """Which prefix a checkpoint may leave out is data of the plan (``optional_prefixes``), not a
    word in the loader: with another architecture's prefix the same file is matched, with none
    the names must be exact."""
    from zse_amd.parts.base import TensorReq
    from zse_amd.weights.loader import WeightError, check_entries
    d = str(tmp_path / "m")
    os.makedirs(d)
    st.write_file(os.path.join(d, "model.safetensors"),
                  {"transformer.wte": ("F32", np.zeros((4, 2), np.float32)), "h.0.w": ("F32", np.zeros((2, 2), np.float32))})
    reqs = [TensorReq("wte", (4, 2)), TensorReq("transformer.h.0.w", (2, 2))]
    entries = st.index_folder(d)
    got = check_entries(entries, reqs, prefixes=("transformer.",))
    assert sorted(got) == ["h.0.w", "wte"]
    with pytest.raises(WeightError) as e:
        check_entries(entries, reqs, prefixes=())
    assert sorted(e.value.missing) == ["transformer.h.0.w", "wte"] and sorted(e.value.unexpected) == ["h.0.w", "transformer.wte"]


def test_untied_model_wants_lm_head(tmp_path):
    cfg = dict(TINY_A, tie_word_embeddings=False)
    d = write_random_model(str(tmp_path / "m"), cfg, seed=0, dtype="float32")
    assert "lm_head.weight" in st.index_folder(d)
    with pytest.raises(WeightError) as e:
        check_folder(d, reqs_of(TINY_A))
    assert e.value.unexpected == ["lm_head.weight"]


def test_unsupported_dtype_is_reported(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=0, dtype="float32")
    w = {n: ("F32", a) for n, a in st.read_folder_f32(d).items()}
    w["model.norm.weight"] = ("I32", np.zeros(64, np.int32))
    st.write_file(os.path.join(d, "model.safetensors"), w)
    with pytest.raises(WeightError) as e:
        check_folder(d, reqs_of(TINY_A))
    assert e.value.wrong_dtype == [("model.norm.weight", "I32")]


def test_the_random_weights_function():
    """Values are a function of (seed, stream, element index) alone: any slice can be made
    by itself, other seeds and streams give other values, and the values are standard normal
    (the device makes the same bits; tests/test_gpu_kernels.py compares them)."""
    from zse_amd.weights.normal import normal, normal_tensor, stream_of
    x = normal(400_001, 9, 77)
    assert x.dtype == np.float32 and x.shape == (400_001,)
    assert np.array_equal(normal(1001, 9, 77, first=12_345), x[12_345:13_346])       # odd start, odd count
    assert np.array_equal(normal(2, 9, 77, first=400_000 - 1), x[-2:])
    assert not np.array_equal(normal(100, 10, 77), x[:100]) and not np.array_equal(normal(100, 9, 78), x[:100])
    assert abs(float(x.mean())) < 0.01 and abs(float(x.std()) - 1) < 0.01
    assert abs(float((x.astype(np.float64) ** 4).mean()) - 3) < 0.1 and 4 < np.abs(x).max() < 6
    # the two values of a pair are not correlated, nor are neighbours
    assert abs(np.corrcoef(x[0:-1:2], x[1::2])[0, 1]) < 0.01 and abs(np.corrcoef(x[1:-1], x[2:])[0, 1]) < 0.01
    y = normal(50_000, 9, 77, mean=1.5, std=0.02)
    assert abs(float(y.mean()) - 1.5) < 1e-3 and abs(float(y.std()) - 0.02) < 1e-3
    assert stream_of("layers.0.mlp.up_proj.weight") != stream_of("layers.1.mlp.up_proj.weight")
    t = normal_tensor((7, 5), 1, "a.b")
    assert t.shape == (7, 5) and np.array_equal(t.reshape(-1), normal(35, 1, stream_of("a.b")))
