"""Gemma 2 (``Gemma2ForCausalLM``): typed config and its plan of parts.

Keys and defaults follow the reference's adapter (format/arch/gemma2.py:26-48):
``hidden_size``, ``num_attention_heads``, ``num_hidden_layers``,
``intermediate_size``, ``vocab_size`` are required; ``num_key_value_heads``
defaults to the head count, ``head_dim`` to hidden/heads,
``max_position_embeddings`` to 8192, ``rope_theta`` to 10000.0,
``rms_norm_eps`` to 1e-6, ``sliding_window`` to none, ``tie_word_embeddings``
to true.  The adapter's docstring names further Gemma 2 features
(format/arch/gemma2.py:3-12) that its ``config_from_hf`` does not copy; they are
read here: ``query_pre_attn_scalar`` (default head_dim),
``attn_logit_softcapping``, ``final_logit_softcapping`` (default none),
``hidden_activation`` (default and only value ``gelu_pytorch_tanh``) and
``layer_types``.  Tensor names: format/arch/gemma2.py:57-85.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

from ..config.base import (Architecture, ConfigError, Problems, need,
                           register_architecture)
from ..config.plan import (AttentionSpec, BlockSpec, EmbeddingSpec, GatedMLPSpec,
                           HeadSpec, LayerCall, ModelPlan, NormSpec, RotarySpec)

SLIDING = "sliding_attention"
FULL = "full_attention"
ACTIVATIONS = {"gelu_pytorch_tanh": "gelu_tanh"}


@dataclass(frozen=True)
class Gemma2Config:
    num_hidden_layers: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    sliding_window: Optional[int]
    query_pre_attn_scalar: float
    attn_logit_softcapping: Optional[float]
    final_logit_softcapping: Optional[float]
    hidden_activation: str
    tie_word_embeddings: bool
    layer_types: Tuple[str, ...]

    @staticmethod
    def from_dict(raw: dict) -> "Gemma2Config":
        p = Problems("Gemma 2 config.json")
        H = need(raw, "hidden_size", int, p, required=True)
        nh = need(raw, "num_attention_heads", int, p, required=True)
        L = need(raw, "num_hidden_layers", int, p, required=True)
        I = need(raw, "intermediate_size", int, p, required=True)
        V = need(raw, "vocab_size", int, p, required=True)
        p.raise_if_any()
        for k, v in (("hidden_size", H), ("num_attention_heads", nh), ("num_hidden_layers", L),
                     ("intermediate_size", I), ("vocab_size", V)):
            p.require(v > 0, f"'{k}' must be positive, got {v}")
        p.raise_if_any()
        nkv = need(raw, "num_key_value_heads", int, p, default=nh)
        hd = need(raw, "head_dim", int, p, default=H // nh)
        maxpos = need(raw, "max_position_embeddings", int, p, default=8192)
        theta = need(raw, "rope_theta", float, p, default=10000.0)
        eps = need(raw, "rms_norm_eps", float, p, default=1e-6)
        window = need(raw, "sliding_window", int, p, default=None, allow_none=True)
        qpas = need(raw, "query_pre_attn_scalar", float, p, default=float(hd))
        acap = need(raw, "attn_logit_softcapping", float, p, default=None, allow_none=True)
        fcap = need(raw, "final_logit_softcapping", float, p, default=None, allow_none=True)
        act = need(raw, "hidden_activation", str, p, default="gelu_pytorch_tanh")
        if "hidden_activation" not in raw and isinstance(raw.get("hidden_act"), str):
            act = raw["hidden_act"]
        tied = need(raw, "tie_word_embeddings", bool, p, default=True)
        types = raw.get("layer_types")
        p.raise_if_any()

        p.require(nkv > 0 and nh % nkv == 0,
                  f"num_attention_heads ({nh}) must be a multiple of num_key_value_heads ({nkv})")
        p.require(hd > 0 and hd % 2 == 0, f"head_dim must be positive and even, got {hd}")
        p.require(maxpos > 0, f"max_position_embeddings must be positive, got {maxpos}")
        p.require(theta > 0, f"rope_theta must be positive, got {theta}")
        p.require(eps > 0, f"rms_norm_eps must be positive, got {eps}")
        p.require(window is None or window > 0, f"sliding_window must be positive, got {window}")
        p.require(qpas > 0, f"query_pre_attn_scalar must be positive, got {qpas}")
        p.require(acap is None or acap > 0, f"attn_logit_softcapping must be positive, got {acap}")
        p.require(fcap is None or fcap > 0, f"final_logit_softcapping must be positive, got {fcap}")
        p.require(act in ACTIVATIONS,
                  f"hidden_activation must be one of {sorted(ACTIVATIONS)}, got {act!r}")
        if types is None:
            # layer 0 is a sliding layer, layer 1 a global one, and so on;
            # without a window every layer is global.
            types = [SLIDING if (l % 2 == 0 and window is not None) else FULL for l in range(L)]
        else:
            p.require(isinstance(types, list) and len(types) == L,
                      f"layer_types must list {L} entries")
            if isinstance(types, list):
                for t in types:
                    p.require(t in (SLIDING, FULL), f"unknown layer type {t!r}")
                p.require(window is not None or SLIDING not in types,
                          "layer_types has sliding layers but sliding_window is not set")
        p.raise_if_any()
        return Gemma2Config(L, H, nh, nkv, hd, I, V, maxpos, theta, eps, window, qpas, acap, fcap,
                            act, tied, tuple(types))

    def to_dict(self) -> dict:
        """The config.json that reads back as this config."""
        return {
            "architectures": ["Gemma2ForCausalLM"], "model_type": "gemma2",
            "num_hidden_layers": self.num_hidden_layers, "hidden_size": self.hidden_size,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads, "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size, "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta, "rms_norm_eps": self.rms_norm_eps,
            "sliding_window": self.sliding_window,
            "query_pre_attn_scalar": self.query_pre_attn_scalar,
            "attn_logit_softcapping": self.attn_logit_softcapping,
            "final_logit_softcapping": self.final_logit_softcapping,
            "hidden_activation": self.hidden_activation,
            "tie_word_embeddings": self.tie_word_embeddings,
            "layer_types": list(self.layer_types),
        }


def gemma2_plan(c: Gemma2Config) -> ModelPlan:
    def norm(name):
        return NormSpec(size=c.hidden_size, eps=c.rms_norm_eps, unit_offset=True, weight=name)

    rotary = RotarySpec(head_dim=c.head_dim, rotary_dim=c.head_dim, theta=c.rope_theta)
    layers = []
    for l in range(c.num_hidden_layers):
        pre = f"model.layers.{l}."
        attn = AttentionSpec(
            hidden_size=c.hidden_size, num_heads=c.num_attention_heads,
            num_kv_heads=c.num_key_value_heads, head_dim=c.head_dim,
            scale=float(c.query_pre_attn_scalar) ** -0.5,
            softcap=c.attn_logit_softcapping,
            window=c.sliding_window if c.layer_types[l] == SLIDING else None,
            position=rotary,
            names={r: f"{pre}self_attn.{r}_proj.weight" for r in ("q", "k", "v", "o")})
        ffn = GatedMLPSpec(
            hidden_size=c.hidden_size, intermediate_size=c.intermediate_size,
            activation=ACTIVATIONS[c.hidden_activation],
            names={r: f"{pre}mlp.{r}_proj.weight" for r in ("gate", "up", "down")})
        layers.append(BlockSpec(
            arrangement="sandwich", mixer=attn, ffn=ffn,
            norms={"pre_mixer": norm(pre + "input_layernorm.weight"),
                   "post_mixer": norm(pre + "post_attention_layernorm.weight"),
                   "pre_ffn": norm(pre + "pre_feedforward_layernorm.weight"),
                   "post_ffn": norm(pre + "post_feedforward_layernorm.weight")}))
    embed_name = "model.embed_tokens.weight"
    return ModelPlan(
        architecture="Gemma2ForCausalLM",
        hidden_size=c.hidden_size, vocab_size=c.vocab_size,
        max_position=c.max_position_embeddings,
        embedding=EmbeddingSpec(c.vocab_size, c.hidden_size, math.sqrt(c.hidden_size), embed_name),
        layers=tuple(layers),
        order=tuple(LayerCall(l) for l in range(c.num_hidden_layers)),
        final_norm=norm("model.norm.weight"),
        head=HeadSpec(c.vocab_size, c.hidden_size, c.final_logit_softcapping,
                      embed_name if c.tie_word_embeddings else "lm_head.weight"),
    )


GEMMA2 = register_architecture(Architecture(
    name="Gemma2ForCausalLM", config_from_dict=Gemma2Config.from_dict, plan=gemma2_plan,
    model_types=("gemma2",)))
