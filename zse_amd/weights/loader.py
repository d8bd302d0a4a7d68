"""Weights by tensor name: checking a checkpoint against what the parts ask
for, and putting tensors on the device.

The reference looks a weight up at first use and raises ``KeyError`` there
(orchestrator/model_runner.py:1510-1519); extra tensors and shapes are never
checked.  Here the whole list is checked before anything is copied, and one
error names every missing tensor, every unexpected one and every wrong shape.
Names match with or without a leading ``model.`` (format/arch/gemma2.py:50-55,
model_runner.py:249-253).

Storage on the device: tensors used in matrix products are held in the
engine's compute type (bfloat16 or float32); gains and other vectors are held
as float32 whatever the file stores, which loses nothing; integer tensors
would be held as int32.
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Sequence, Tuple

import numpy as np

from ..parts.base import ROLE_GAIN, ROLE_MATRIX, TensorReq
from ..runtime.device import BF16, F32, Tensor
from . import safetensors as st

SRC_TAGS = {"F32": 0, "BF16": 1, "F16": 2}


class WeightError(ValueError):
    """The checkpoint does not hold what the model needs; lists every finding."""

    def __init__(self, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shape = sorted(wrong_shape)
        self.wrong_dtype = sorted(wrong_dtype)
        lines = []
        if self.missing:
            lines.append(f"missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"wrong shapes ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {tuple(g)}, expected {tuple(w)}" for n, g, w in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"unsupported dtypes ({len(self.wrong_dtype)}): " + ", ".join(
                f"{n} is {d}" for n, d in self.wrong_dtype))
        super().__init__("checkpoint does not match the model: " + "; ".join(lines))


DEFAULT_PREFIXES = ("model.",)


def _strip(name: str, prefixes: Sequence[str] = DEFAULT_PREFIXES) -> str:
    """The name without the first of ``prefixes`` it begins with: checkpoints of one
    architecture come with and without such a prefix (``ModelPlan.optional_prefixes``)."""
    for p in prefixes:
        if p and name.startswith(p):
            return name[len(p):]
    return name


def merge_reqs(reqs: Iterable[TensorReq], prefixes: Sequence[str] = DEFAULT_PREFIXES) -> Dict[str, TensorReq]:
    """One entry per name; a name asked for twice (tied weights) must agree in shape."""
    out: Dict[str, TensorReq] = {}
    for r in reqs:
        key = _strip(r.name, prefixes)
        if key in out and out[key].shape != tuple(r.shape):
            raise ValueError(f"tensor {r.name} is asked for with shapes {out[key].shape} and {r.shape}")
        out.setdefault(key, TensorReq(r.name, tuple(r.shape), r.role, r.init_std))
    return out


def check_entries(entries: Dict[str, st.TensorEntry], reqs: Iterable[TensorReq],
                  ignored: Sequence[str] = (), prefixes: Sequence[str] = DEFAULT_PREFIXES) -> Dict[str, st.TensorEntry]:
    """Match checkpoint entries to requests; raises ``WeightError`` with every finding.
    Returns stripped name -> entry."""
    want = merge_reqs(reqs, prefixes)
    have = {}
    for name, e in entries.items():
        have[_strip(name, prefixes)] = e
    skip = {_strip(n, prefixes) for n in ignored}
    missing = [want[k].name for k in want if k not in have]
    unexpected = [have[k].name for k in have if k not in want and k not in skip]
    wrong_shape = [(have[k].name, have[k].shape, want[k].shape) for k in want
                   if k in have and tuple(have[k].shape) != tuple(want[k].shape)]
    wrong_dtype = [(have[k].name, have[k].dtype) for k in want
                   if k in have and have[k].dtype not in SRC_TAGS]
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightError(missing, unexpected, wrong_shape, wrong_dtype)
    return {k: have[k] for k in want}


def check_folder(model_dir: str, reqs: Iterable[TensorReq], ignored: Sequence[str] = (),
                 prefixes: Sequence[str] = DEFAULT_PREFIXES):
    return check_entries(st.index_folder(model_dir), reqs, ignored, prefixes)


class _Source:
    """Common part of weight sources: caching, so that tied names share one tensor."""

    def __init__(self, rt, dtype: str, tuned: bool = True, prefixes: Sequence[str] = DEFAULT_PREFIXES):
        self.rt = rt
        self.prefixes = tuple(prefixes)
        self.dtype = dtype
        self.tuned = bool(tuned)      # parts may ask for layouts that only the tuned kernels read
        self.k = rt.kernels(dtype)
        self._cache: Dict[Tuple, Tensor] = {}
        self.bytes_on_device = 0

    def wants_strip(self, cols: int, gated_rows: int = 0) -> bool:
        """True when a matrix with ``cols`` columns should be held in the matrix-core kernels'
        strip layout: bf16, tuned kernels on, whole 32-wide steps (and, for a gate|up stack
        of ``gated_rows`` each, whole strips of 16)."""
        return bool(self.tuned and self.dtype == BF16 and self.k.has("zk_strip_layout") and
                    cols % 32 == 0 and gated_rows % 16 == 0)

    def matrix(self, names: Sequence[str], strip: bool = False) -> Tensor:
        """The named 2-D tensors stacked along rows, in the compute type.  ``strip``: in strip
        layout (rows padded to a multiple of 16; the shape stays the logical one)."""
        key = ("s" if strip else "m",) + tuple(_strip(n, self.prefixes) for n in names)
        if key not in self._cache and strip:
            rows = self.matrix(names)
            self._cache.pop(("m",) + tuple(_strip(n, self.prefixes) for n in names))
            self.bytes_on_device -= rows.nbytes
            n, k = rows.shape
            out = self.rt.empty(((n + 15) // 16 * 16, k), self.dtype)
            self.k.zk_strip_layout(rows.ptr, out.ptr, n, k, self.rt.stream)
            self.rt.sync()
            self.bytes_on_device += out.nbytes
            self._cache[key] = Tensor(out.ptr, (n, k), self.dtype, out.owner, layout="strip")
        if key not in self._cache:
            shapes = [self._shape(n) for n in names]
            cols = shapes[0][1]
            if any(len(s) != 2 or s[1] != cols for s in shapes):
                raise ValueError(f"cannot stack {list(zip(names, shapes))}")
            out = self.rt.empty((sum(s[0] for s in shapes), cols), self.dtype)
            row = 0
            for n, s in zip(names, shapes):
                self._fill(n, out.rows(row, row + s[0]), 1)
                row += s[0]
            self.bytes_on_device += out.nbytes
            self._cache[key] = out
        return self._cache[key]

    def vector(self, name: str) -> Tensor:
        key = ("v", _strip(name, self.prefixes))
        if key not in self._cache:
            out = self.rt.empty(self._shape(name), F32)
            self._fill(name, out, 0)
            self.bytes_on_device += out.nbytes
            self._cache[key] = out
        return self._cache[key]


class CheckpointWeights(_Source):
    """Tensors of a checked model folder, copied and converted on the device."""

    def __init__(self, rt, dtype: str, model_dir: str, reqs: Iterable[TensorReq],
                 ignored: Sequence[str] = (), tuned: bool = True, prefixes: Sequence[str] = DEFAULT_PREFIXES):
        super().__init__(rt, dtype, tuned, prefixes)
        self.entries = check_folder(model_dir, reqs, ignored, prefixes)
        self._staging = None

    def _shape(self, name):
        return self.entries[_strip(name, self.prefixes)].shape

    def _fill(self, name: str, dst: Tensor, dst_kind: int):
        e = self.entries[_strip(name, self.prefixes)]
        arr = st.map_tensor(e)
        same = (e.dtype == "F32" and dst.dtype == F32) or (e.dtype == "BF16" and dst.dtype == BF16)
        if same:
            self.rt.copy_h2d(dst.ptr, arr)
            return
        chunk_rows = max(1, (64 << 20) // max(1, e.nbytes // max(1, e.shape[0])))
        # staging buffer: big enough for one chunk of rows of this tensor
        row_bytes = e.nbytes // max(1, e.shape[0])
        need = min(e.shape[0], chunk_rows) * row_bytes
        if self._staging is None or self._staging.nbytes < need:
            self._staging = self.rt.empty((need + 3) // 4, F32)
        inner = int(np.prod(e.shape[1:])) if len(e.shape) > 1 else 1
        flat = arr.reshape(e.shape[0], inner) if e.shape else arr.reshape(1, 1)
        item = 4 if dst.dtype == F32 else 2
        for r0 in range(0, e.shape[0], chunk_rows):
            r1 = min(e.shape[0], r0 + chunk_rows)
            self.rt.copy_h2d(self._staging.ptr, flat[r0:r1])
            self.k.zk_convert(self._staging.ptr, SRC_TAGS[e.dtype], dst.ptr + r0 * inner * item,
                              dst_kind, (r1 - r0) * inner, self.rt.stream)
            self.rt.sync()

    def close(self):
        self._staging = None


class RandomWeights(_Source):
    """Seeded random tensors made on the device: matrices N(0, std), gains
    N(0, gain_std); each value is a function of (seed, tensor name, index)."""

    def __init__(self, rt, dtype: str, reqs: Iterable[TensorReq], seed: int, std: float = 0.02,
                 gain_std: float = 0.1, tuned: bool = True, std_of=None,
                 prefixes: Sequence[str] = DEFAULT_PREFIXES):
        super().__init__(rt, dtype, tuned, prefixes)
        self.reqs = merge_reqs(reqs, prefixes)
        self.seed, self.std, self.gain_std = int(seed), float(std), float(gain_std)
        self.std_of = dict(std_of or {})

    def _shape(self, name):
        return self.reqs[_strip(name, self.prefixes)].shape

    def _fill(self, name: str, dst: Tensor, dst_kind: int):
        from .normal import stream_of
        from .random_init import deviation_of
        r = self.reqs[_strip(name, self.prefixes)]
        std = deviation_of(r, self.std, self.gain_std, self.std_of)
        if dst_kind == 0 and self.dtype == BF16:
            # a vector kept as float32 in a bfloat16 model holds what a bfloat16 checkpoint
            # would: values rounded to bfloat16 (so the model equals the folder written on the host)
            tmp = self.rt.empty((dst.numel,), BF16)
            self.k.zk_fill_normal(tmp.ptr, 1, dst.numel, self.seed, stream_of(_strip(name, self.prefixes)), 0.0, std,
                                  self.rt.stream)
            self.k.zk_convert(tmp.ptr, SRC_TAGS["BF16"], dst.ptr, 0, dst.numel, self.rt.stream)
            self.rt.sync()
            return
        self.k.zk_fill_normal(dst.ptr, dst_kind, dst.numel, self.seed, stream_of(_strip(name, self.prefixes)), 0.0, std,
                              self.rt.stream)

    def close(self):
        pass
