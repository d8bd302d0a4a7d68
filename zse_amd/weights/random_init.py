"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.

Values are a pure function of (seed, tensor name, element index): matrices
N(0, std), gains N(0, gain_std), so a tensor's values do not depend on the other
tensors.  The function is the one the device uses when it makes a model's weights
in place (``zk_fill_normal``; ``zse_amd.weights.normal`` computes the same bits on
the host): a folder written here and a model made on the device from the same
configuration and seed hold the same weights.  The reference has no such mode for
models (random weights appear only in its adapter tests, orchestrator/lora_manager.py:157).
"""
from __future__ import annotations

import json
import os
from typing import Optional

import numpy as np

from ..config.base import ARCHITECTURES, resolve_architecture
from ..parts.base import ROLE_GAIN
from . import safetensors as st
from .loader import merge_reqs
from .normal import normal_tensor


def deviation_of(req, std: float, gain_std: float, std_of=None) -> float:
    """The deviation a tensor is drawn with: its own if the part names one, else the mode's
    for its role; ``std_of`` maps a piece of a tensor name to a deviation and wins."""
    s = req.init_std if req.init_std is not None else (gain_std if req.role == ROLE_GAIN else std)
    for part, v in (std_of or {}).items():
        if part in req.name:
            s = v
    return float(s)


def random_tensors(reqs, seed: int, std: float, gain_std: float, std_of=None, prefixes=None):
    """{name: float32 array} for every tensor the parts ask for (one draw per name)."""
    merged = merge_reqs(reqs) if prefixes is None else merge_reqs(reqs, prefixes)
    return {r.name: normal_tensor(r.shape, seed, key, 0.0, deviation_of(r, std, gain_std, std_of))
            for key, r in merged.items()}


def write_random_model(out_dir: str, config: dict, seed: int = 0, std: float = 0.02,
                       gain_std: float = 0.1, dtype: str = "bfloat16", std_of=None) -> str:
    """Write ``out_dir/config.json`` and ``out_dir/model.safetensors``.

    ``config`` is a config.json dictionary (it must name its architecture);
    ``dtype`` is the storage type of the file, "bfloat16" or "float32";
    ``std_of`` maps a part of a tensor name to the deviation of the tensors that carry it.
    """
    from .. import models  # noqa: F401  (registers architectures)
    from ..engine.model import Model
    arch = resolve_architecture(config)
    typed = arch.config_from_dict(config)
    model = Model(arch.plan(typed))
    tensors = random_tensors(model.tensor_reqs(), seed, std, gain_std, std_of, model.plan.optional_prefixes)
    if dtype in ("bfloat16", "bf16"):
        packed = {n: ("BF16", st.f32_to_bf16_bits(a)) for n, a in tensors.items()}
    elif dtype in ("float32", "fp32"):
        packed = {n: ("F32", a) for n, a in tensors.items()}
    else:
        raise ValueError(f"dtype must be bfloat16 or float32, got {dtype!r}")
    os.makedirs(out_dir, exist_ok=True)
    cfg = dict(config)
    cfg.setdefault("architectures", [arch.name])
    cfg["torch_dtype"] = "bfloat16" if dtype.startswith("b") else "float32"
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    st.write_file(os.path.join(out_dir, "model.safetensors"), packed,
                  metadata={"format": "pt", "seed": seed})
    return out_dir
