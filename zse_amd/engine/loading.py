"""From a model folder (or a config and a seed) to a loaded ``Model``."""
from __future__ import annotations

from typing import Optional

from .. import models as _models  # noqa: F401  (registers architectures)
from ..config.base import load_config, resolve_architecture
from ..runtime.device import Runtime, canonical_dtype
from ..weights.loader import CheckpointWeights, RandomWeights
from .model import Model


def load_model(model_dir: str, dtype: str, rt: Optional[Runtime] = None, tuned: bool = True) -> Model:
    """Read config.json, pick the architecture, check and load the safetensors.  ``tuned``:
    the model will run on the tuned kernels (weights may then sit in their layouts); False
    keeps everything row-major for the plain kernels."""
    rt = rt or Runtime.get()
    dtype = canonical_dtype(dtype)
    arch, config = load_config(model_dir)
    model = Model(arch.plan(config))
    model.config = config
    src = CheckpointWeights(rt, dtype, model_dir, model.tensor_reqs(), model.plan.ignored_tensors, tuned=tuned,
                            prefixes=model.plan.optional_prefixes)
    model.load(src, rt, dtype)
    model.tuned = bool(tuned)
    rt.sync()
    model.weight_bytes = src.bytes_on_device
    src.close()
    return model


def random_model(config: dict, dtype: str, seed: int = 0, std: float = 0.02, gain_std: float = 0.1,
                 rt: Optional[Runtime] = None, tuned: bool = True, std_of=None) -> Model:
    """A model with seeded random weights made on the device (no folder is written): the same
    weights that ``write_random_model`` writes for the same configuration, seed and deviations."""
    rt = rt or Runtime.get()
    dtype = canonical_dtype(dtype)
    arch = resolve_architecture(config)
    typed = arch.config_from_dict(config)
    model = Model(arch.plan(typed))
    model.config = typed
    src = RandomWeights(rt, dtype, model.tensor_reqs(), seed, std, gain_std, tuned=tuned, std_of=std_of,
                        prefixes=model.plan.optional_prefixes)
    model.load(src, rt, dtype)
    model.tuned = bool(tuned)
    rt.sync()
    model.weight_bytes = src.bytes_on_device
    return model
