"""The data an architecture hands to the engine: parts, layers, and their order.

A ``ModelPlan`` is plain data.  Every part is described by a small frozen
dataclass carrying a ``kind`` (the key of the part's class in
``zse_amd.parts.registry``), its sizes and constants, and the checkpoint
names of its tensors.  No part description names the model it belongs to.

The reference keeps one flat ``ModelConfig`` for every architecture and picks
a forward path by ``config.arch`` (format/config.py:33-95,
orchestrator/model_runner.py:127-130); here the choice is made layer by layer
from these records instead.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    """Root-mean-square norm over the last axis: x * rsqrt(mean(x^2)+eps) * gain,
    gain = (1 + w) when ``unit_offset`` else w."""
    size: int
    eps: float
    unit_offset: bool
    weight: str                      # checkpoint tensor name
    kind: str = "rmsnorm"


@dataclass(frozen=True)
class RotarySpec:
    """Rotate-half rotary encoding of the first ``rotary_dim`` channels of a head."""
    head_dim: int
    rotary_dim: int
    theta: float
    kind: str = "rotary"


@dataclass(frozen=True)
class NoPositionSpec:
    kind: str = "none"


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query softmax attention over a paged key/value cache."""
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float                     # multiplies q.k
    softcap: Optional[float]         # cap * tanh(s / cap) on scaled scores
    window: Optional[int]            # keys i-j < window visible; None = all
    position: Any                    # a position-encoding spec
    names: Dict[str, str]            # roles q, k, v, o -> checkpoint names
    kind: str = "attention"


@dataclass(frozen=True)
class GatedMLPSpec:
    """act(x Wg^T) * (x Wu^T), then Wd^T."""
    hidden_size: int
    intermediate_size: int
    activation: str                  # "gelu_tanh" | "silu"
    names: Dict[str, str]            # roles gate, up, down
    kind: str = "gated_mlp"


@dataclass(frozen=True)
class BlockSpec:
    """One layer: a mixer and a feed-forward joined to the residual stream.

    ``arrangement``:
      "sandwich": h += post_m(mixer(pre_m(h))); h += post_f(ffn(pre_f(h)))
      "prenorm" : h += mixer(pre_m(h));         h += ffn(pre_f(h))
    ``norms`` holds the roles pre_mixer, post_mixer, pre_ffn, post_ffn that the
    arrangement uses.
    """
    arrangement: str
    mixer: Any
    ffn: Any
    norms: Dict[str, Any]
    kind: str = "block"


@dataclass(frozen=True)
class EmbeddingSpec:
    vocab_size: int
    hidden_size: int
    scale: float                     # multiplies the gathered row
    weight: str
    kind: str = "embedding"


@dataclass(frozen=True)
class HeadSpec:
    vocab_size: int
    hidden_size: int
    softcap: Optional[float]
    weight: str                      # may equal the embedding's name (tied)
    kind: str = "lm_head"


@dataclass(frozen=True)
class LayerCall:
    """One entry of the execution order.

    ``layer`` indexes ``ModelPlan.layers``.  ``cache_of`` names an earlier
    entry of the order whose cache this call reads instead of keeping its own
    (None: the call owns a cache, if its mixer needs one).
    """
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelPlan:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_position: int
    embedding: EmbeddingSpec
    layers: Tuple[BlockSpec, ...]
    order: Tuple[LayerCall, ...]
    final_norm: Any
    head: HeadSpec
    ignored_tensors: Tuple[str, ...] = ()   # checkpoint names that may be present and are not used
    # what a checkpoint may or may not put in front of a tensor's name: "model.layers.0..." and
    # "layers.0..." are the same tensor (format/arch/gemma2.py:50-55 accepts both)
    optional_prefixes: Tuple[str, ...] = ("model.",)

    def describe(self) -> List[str]:
        out = []
        for i, call in enumerate(self.order):
            b = self.layers[call.layer]
            win = getattr(b.mixer, "window", None)
            out.append(f"call {i}: layer {call.layer} {b.arrangement} mixer={b.mixer.kind}"
                       f"(window={win}) ffn={b.ffn.kind}"
                       + (f" cache_of={call.cache_of}" if call.cache_of is not None else ""))
        return out
