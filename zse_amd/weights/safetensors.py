"""Reading and writing safetensors files without any library.

Format as the reference reads it (format/convert.py:51-62, 65-82, 134-145): an
8-byte little-endian header length, a JSON header mapping each tensor name to
``dtype``, ``shape`` and ``data_offsets`` (relative to the end of the header),
then the raw data; the ``__metadata__`` entry is skipped.  All
``*.safetensors`` files of a folder are read, in sorted order; none is an
error (format/convert.py:123-131).
"""
from __future__ import annotations

import glob
import json
import os
import struct
from dataclasses import dataclass
from typing import Dict, List, Tuple

import numpy as np

# safetensors dtype tag -> (numpy storage dtype, bytes per element)
DTYPES = {
    "F32": (np.float32, 4), "F16": (np.float16, 2), "BF16": (np.uint16, 2),
    "I64": (np.int64, 8), "I32": (np.int32, 4), "I16": (np.int16, 2), "I8": (np.int8, 1),
    "U8": (np.uint8, 1), "BOOL": (np.bool_, 1), "F64": (np.float64, 8),
}


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str               # safetensors tag
    shape: Tuple[int, ...]
    path: str
    begin: int               # absolute file offset of the first byte
    nbytes: int


def find_files(model_dir: str) -> List[str]:
    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no *.safetensors file in {model_dir}")
    return files


def read_header(path: str) -> Dict[str, TensorEntry]:
    size = os.path.getsize(path)
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) < 8:
            raise ValueError(f"{path}: too short for a safetensors file")
        (n,) = struct.unpack("<Q", head)
        if n <= 0 or 8 + n > size:
            raise ValueError(f"{path}: header length {n} does not fit the file ({size} bytes)")
        meta = json.loads(f.read(n).decode("utf-8"))
    base = 8 + n
    out = {}
    for name, info in meta.items():
        if name == "__metadata__":
            continue
        dtype = info["dtype"]
        shape = tuple(int(s) for s in info["shape"])
        b, e = info["data_offsets"]
        if dtype not in DTYPES:
            raise ValueError(f"{path}: tensor {name} has unsupported dtype {dtype}")
        count = 1
        for s in shape:
            count *= s
        if e - b != count * DTYPES[dtype][1] or base + e > size:
            raise ValueError(f"{path}: tensor {name} has offsets {b}:{e} that do not match "
                             f"shape {shape} of {dtype}")
        out[name] = TensorEntry(name, dtype, shape, path, base + b, e - b)
    return out


def index_folder(model_dir: str) -> Dict[str, TensorEntry]:
    """name -> entry over every safetensors file of the folder."""
    entries: Dict[str, TensorEntry] = {}
    for path in find_files(model_dir):
        for name, e in read_header(path).items():
            if name in entries:
                raise ValueError(f"tensor {name} appears in both {entries[name].path} and {path}")
            entries[name] = e
    return entries


def map_tensor(entry: TensorEntry) -> np.ndarray:
    """The tensor's bytes as a read-only memory-mapped array of its storage dtype
    (bfloat16 comes back as uint16 bit patterns)."""
    np_dtype = DTYPES[entry.dtype][0]
    if entry.nbytes == 0:
        return np.zeros(entry.shape, dtype=np_dtype)
    return np.memmap(entry.path, dtype=np_dtype, mode="r", offset=entry.begin, shape=entry.shape)


# ---------------------------------------------------------------- bfloat16 on the host

def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even conversion of float32 to bfloat16 bit patterns (uint16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = (u + (0x7FFF + ((u >> 16) & 1))) >> 16
    rounded = np.where(nan, (u >> 16) | 0x40, rounded)
    return rounded.astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_float32(arr: np.ndarray, dtype_tag: str) -> np.ndarray:
    """Any stored float tensor as float32 values."""
    if dtype_tag == "BF16":
        return bf16_bits_to_f32(arr)
    return np.array(arr, dtype=np.float32)      # a copy: the caller may rewrite the file


def read_folder_f32(model_dir: str) -> Dict[str, np.ndarray]:
    """Every tensor of a folder as float32 (small models; used by tests and tools)."""
    return {n: to_float32(map_tensor(e), e.dtype) for n, e in index_folder(model_dir).items()}


# ---------------------------------------------------------------- writing

def write_file(path: str, tensors: Dict[str, Tuple[str, np.ndarray]], metadata=None) -> None:
    """Write ``name -> (dtype tag, array in that tag's storage dtype)``."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    order = list(tensors)
    for name in order:
        tag, arr = tensors[name]
        np_dtype, size = DTYPES[tag]
        if arr.dtype != np.dtype(np_dtype):
            raise ValueError(f"{name}: array dtype {arr.dtype} does not store {tag}")
        n = int(arr.size) * size
        header[name] = {"dtype": tag, "shape": list(arr.shape), "data_offsets": [off, off + n]}
        off += n
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            f.write(np.ascontiguousarray(tensors[name][1]).tobytes())
