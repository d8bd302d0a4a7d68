"""Configuration and registry (no GPU)."""
import json

import pytest

from conftest import TINY_A, TINY_B
from zse_amd import models  # noqa: F401
from zse_amd.config import ConfigError, load_config, resolve_architecture
from zse_amd.models.gemma2 import FULL, SLIDING, Gemma2Config, gemma2_plan


def test_required_keys_are_reported_together():
    with pytest.raises(ConfigError) as e:
        Gemma2Config.from_dict({"hidden_size": 64})
    msg = str(e.value)
    for k in ("num_attention_heads", "num_hidden_layers", "intermediate_size", "vocab_size"):
        assert k in msg


def test_defaults_follow_the_adapter():
    c = Gemma2Config.from_dict(dict(hidden_size=64, num_attention_heads=4, num_hidden_layers=2,
                                    intermediate_size=128, vocab_size=100))
    assert c.num_key_value_heads == 4 and c.head_dim == 16
    assert c.max_position_embeddings == 8192 and c.rope_theta == 10000.0 and c.rms_norm_eps == 1e-6
    assert c.sliding_window is None and c.tie_word_embeddings is True
    assert c.query_pre_attn_scalar == 16.0
    assert c.attn_logit_softcapping is None and c.final_logit_softcapping is None
    assert c.layer_types == (FULL, FULL)        # no window: every layer is global


def test_alternation_and_layer_types():
    c = Gemma2Config.from_dict(TINY_B)
    assert c.layer_types == (SLIDING, FULL, SLIDING)
    c2 = Gemma2Config.from_dict(dict(TINY_B, layer_types=[FULL, SLIDING, SLIDING]))
    assert c2.layer_types == (FULL, SLIDING, SLIDING)
    with pytest.raises(ConfigError):
        Gemma2Config.from_dict(dict(TINY_B, layer_types=[FULL, SLIDING]))
    with pytest.raises(ConfigError):
        Gemma2Config.from_dict(dict(TINY_B, layer_types=[FULL, "chunked", FULL]))


@pytest.mark.parametrize("bad", [
    dict(num_key_value_heads=3), dict(head_dim=15), dict(sliding_window=0),
    dict(attn_logit_softcapping=-1.0), dict(final_logit_softcapping=0.0),
    dict(hidden_activation="relu"), dict(rms_norm_eps=0.0), dict(query_pre_attn_scalar=0),
    dict(hidden_size="64"), dict(vocab_size=0)])
def test_invalid_values_are_errors(bad):
    with pytest.raises(ConfigError):
        Gemma2Config.from_dict(dict(TINY_A, **bad))


def test_plan_takes_every_size_from_the_config():
    for cfg in (TINY_A, TINY_B):
        c = Gemma2Config.from_dict(cfg)
        plan = gemma2_plan(c)
        assert len(plan.layers) == cfg["num_hidden_layers"] == len(plan.order)
        for l, b in enumerate(plan.layers):
            a = b.mixer
            assert (a.num_heads, a.num_kv_heads, a.head_dim) == (
                cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"])
            assert a.scale == pytest.approx(cfg["query_pre_attn_scalar"] ** -0.5)
            assert a.softcap == cfg["attn_logit_softcapping"]
            assert a.window == (cfg["sliding_window"] if l % 2 == 0 else None)
            assert a.position.theta == cfg["rope_theta"]
            assert b.ffn.intermediate_size == cfg["intermediate_size"]
            assert all(n.eps == cfg["rms_norm_eps"] and n.unit_offset for n in b.norms.values())
            assert set(b.norms) == {"pre_mixer", "post_mixer", "pre_ffn", "post_ffn"}
        assert plan.embedding.scale == pytest.approx(cfg["hidden_size"] ** 0.5)
        assert plan.head.weight == plan.embedding.weight      # tied
        assert plan.head.softcap == cfg["final_logit_softcapping"]


def test_untied_head_has_its_own_tensor():
    plan = gemma2_plan(Gemma2Config.from_dict(dict(TINY_A, tie_word_embeddings=False)))
    assert plan.head.weight == "lm_head.weight"


def test_registry_resolves_by_architecture_then_model_type():
    assert resolve_architecture({"architectures": ["Gemma2ForCausalLM"]}).name == "Gemma2ForCausalLM"
    assert resolve_architecture({"model_type": "gemma2"}).name == "Gemma2ForCausalLM"
    with pytest.raises(ConfigError) as e:
        resolve_architecture({"architectures": ["LlamaForCausalLM"], "model_type": "llama"})
    assert "Gemma2ForCausalLM" in str(e.value)      # names what is registered


def test_load_config_reads_the_folder(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    arch, cfg = load_config(str(tmp_path))
    assert arch.name == "Gemma2ForCausalLM" and cfg.hidden_size == 64
    assert Gemma2Config.from_dict(cfg.to_dict()) == cfg
    with pytest.raises(FileNotFoundError):
        load_config(str(tmp_path / "nothing"))
