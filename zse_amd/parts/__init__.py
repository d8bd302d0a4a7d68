"""Parts a model is put together from.  Importing the package registers the built-in kinds."""
from . import attention, block, embedding, ffn, norm, position  # noqa: F401
from .base import (PagedKV, Part, StateNeed, TensorReq, build_part, register_part,
                   unregister_part, walk)
from ..runtime.device import register_kernels  # noqa: F401  (a part that brings kernels of its own)
