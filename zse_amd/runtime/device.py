"""The device side seen from Python: memory, streams, events, graphs, kernels.

Everything goes through ctypes into the libraries built from ``zse_amd/csrc``,
in the manner of the reference's ``GPUMemory`` and ``KernelLauncher``
(zse-compiler/zse_compiler/runtime/memory.py:71-447, launcher.py:72-175).  There
is no fallback: without a GPU or without the libraries, ``Runtime()`` raises.
"""
from __future__ import annotations

import ctypes as C
import struct as _struct
from dataclasses import dataclass
from typing import Dict, Optional, Sequence, Tuple

import numpy as np

from . import build

F32 = "float32"
BF16 = "bfloat16"
I32 = "int32"
F64 = "float64"
ITEMSIZE = {F32: 4, BF16: 2, I32: 4, F64: 8}
NUMPY_OF = {F32: np.float32, BF16: np.uint16, I32: np.int32, F64: np.float64}
DTYPE_ALIASES = {"float32": F32, "fp32": F32, "f32": F32, "bfloat16": BF16, "bf16": BF16}


def canonical_dtype(name: str) -> str:
    try:
        return DTYPE_ALIASES[str(name).lower()]
    except KeyError:
        raise ValueError(f"dtype must be one of {sorted(DTYPE_ALIASES)}, got {name!r}") from None


class DeviceError(RuntimeError):
    pass


class Tensor:
    """A view of device memory: pointer, shape, dtype.  Row-major, contiguous."""

    __slots__ = ("ptr", "shape", "dtype", "owner", "layout")

    def __init__(self, ptr: int, shape: Sequence[int], dtype: str, owner=None, layout: str = "rows"):
        self.ptr = int(ptr)
        self.shape = tuple(int(s) for s in shape)
        self.dtype = dtype
        self.owner = owner      # keeps the allocation alive
        self.layout = layout    # "rows": row-major; "strip": the matrix-core kernels' weight layout

    @property
    def numel(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n

    @property
    def nbytes(self) -> int:
        return self.numel * ITEMSIZE[self.dtype]

    def view(self, *shape) -> "Tensor":
        t = Tensor(self.ptr, shape, self.dtype, self.owner)
        if t.numel != self.numel:
            raise ValueError(f"cannot view {self.shape} as {shape}")
        return t

    def rows(self, begin: int, end: int) -> "Tensor":
        """Rows [begin, end) of the first axis."""
        if not (0 <= begin <= end <= self.shape[0]):
            raise IndexError(f"rows {begin}:{end} of {self.shape}")
        inner = self.numel // self.shape[0] if self.shape[0] else 0
        return Tensor(self.ptr + begin * inner * ITEMSIZE[self.dtype],
                      (end - begin,) + self.shape[1:], self.dtype, self.owner)

    def __repr__(self):
        return f"Tensor({self.dtype}, {self.shape}, 0x{self.ptr:x})"


class Allocation:
    """Owns one device allocation; freed when dropped or closed."""

    def __init__(self, rt: "Runtime", nbytes: int):
        self.rt = rt
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        rt._check(rt.lib.zrt_malloc(C.byref(p), C.c_size_t(max(self.nbytes, 4))), "malloc")
        self.ptr = p.value
        rt.allocated += self.nbytes

    def close(self):
        if self.ptr:
            self.rt.free_device(self.ptr)
            self.rt.allocated -= self.nbytes
            self.ptr = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class PinnedBuffer:
    """Page-locked host memory, seen as a numpy byte array."""

    def __init__(self, rt: "Runtime", nbytes: int):
        self.rt = rt
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        rt._check(rt.lib.zrt_host_alloc(C.byref(p), C.c_size_t(max(self.nbytes, 8))), "host alloc")
        self.ptr = p.value
        self.bytes = np.ctypeslib.as_array((C.c_uint8 * max(self.nbytes, 8)).from_address(self.ptr))

    def array(self, offset: int, count: int, dtype) -> np.ndarray:
        dt = np.dtype(dtype)
        return self.bytes[offset:offset + count * dt.itemsize].view(dt)

    def close(self):
        if self.ptr:
            self.bytes = None
            self.rt.free_host(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


@dataclass
class DeviceInfo:
    name: str
    arch: str
    total_memory: int
    free_memory: int
    compute_units: int


_VP, _I, _F, _SZ, _U64 = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_uint64

# name -> argument types (all return int; 0 = success)
KERNEL_SIGNATURES = {
    "zk_embed": [_VP, _VP, _VP, _F, _I, _I, _I, _I, _VP],
    "zk_rmsnorm": [_VP, _I, _VP, _VP, _VP, _F, _I, _I, _I, _VP],
    "zk_norm_add_norm": [_VP, _I, _VP, _F, _I, _VP, _VP, _F, _I, _VP, _I, _I, _VP],
    "zk_gated_act": [_VP, _VP, _I, _I, _I, _VP],
    "zk_softcap": [_VP, _SZ, _F, _VP],
    "zk_rope_cache_write": [_VP, _VP, _VP, _VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _VP],
    "zk_rope_cache_write_sums": [_VP, _VP, _I, _VP, _VP, _VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _VP],
    "zk_convert": [_VP, _I, _VP, _I, _SZ, _VP],
    "zk_fill_normal": [_VP, _I, _SZ, _U64, _U64, _F, _F, _VP],
    "zk_zero": [_VP, _SZ, _VP],
    "zk_feed_tokens": [_VP, _VP, _VP, _VP, _I, _VP],
    "zk_zero_pages": [_VP, _VP, _I, C.POINTER(C.c_int), _I, _VP],
    "zk_gemm_plain": [_VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _VP],
    "zk_attention_plain": [_VP, _I, _VP, _VP, _VP, _I, _VP, _VP, _VP, _I, _I, _I, _I, _I, _F, _F,
                           _I, _I, _VP],
    "zk_argmax": [_VP, _VP, _I, _I, _VP, _VP],
    "zk_sample": [_VP, _VP, _VP, _VP, _VP, _VP, _I, _I, _VP, _VP],
    "zk_sample_cut": [_VP, _VP, _VP, _VP, _VP, _VP, _I, _I, _VP, _I, _VP],
    "zk_penalize": [_VP, _I, _VP, _VP, _VP, _I, _VP],
    "zk_probe_read": [_VP, _SZ, _VP, _VP],
}
# present only in the bf16 library
BF16_KERNEL_SIGNATURES = {
    "zk_gemm_bf16": [_VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _F, _I, _VP, C.c_size_t, C.POINTER(C.c_int), _VP],
    "zk_gemm_bf16_static": [_VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _F, _I, _VP],
    "zk_strip_layout": [_VP, _VP, _I, _I, _VP],
    "zk_head_pick_bf16": [_VP, _I, _VP, _I, _I, _I, _F, _I, _VP, _SZ, _VP, _VP],
    "zk_probe_mfma_bf16": [_I, _VP, C.POINTER(C.c_double), _VP],
    "zk_qkv_rope_bf16": [_VP, _I, _VP, _VP, _I, _I, _I, _I, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _VP],
    "zk_attention_bf16": [_VP, _I, _VP, _VP, _VP, _I, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I,
                          _F, _F, _I, _I, _VP, _SZ, _VP],
}


@dataclass
class KernelExtension:
    """Kernels that a part brings along: a source file and its entry points."""
    name: str
    source: str                              # path of a .hip file
    entry_points: Dict[str, list]            # entry point -> ctypes argument types, the stream last
    written_down: bool = True
    dtypes: Tuple[str, ...] = (F32, BF16)


KERNEL_EXTENSIONS: Dict[str, KernelExtension] = {}


def register_kernels(name: str, source: str, entry_points: Dict[str, list], written_down: bool = True,
                     dtypes: Sequence[str] = (F32, BF16)) -> KernelExtension:
    """The one call through which a part brings kernels of its own.

    ``source`` is a .hip file (anywhere: beside the part).  It includes ``common.h`` and
    ``packed_call.h`` of ``zse_amd/csrc``, says ``ZK_DEFINE_HOST_SIDE`` once, defines its entry
    points as ``extern "C" int name(..., void* stream)`` returning 0 or a status with
    ``zk_fail``'s message, and ``ZK_PACKED(name)`` for each.  It is compiled once per storage type
    in ``dtypes`` (``-DZSE_ACT_BF16=0`` or ``1``, the engine's flags) into a library of its own,
    built on first use like the engine's and found by ``__graft_entry__.build()`` too.
    ``entry_points`` gives each entry point's ctypes argument types.  After this call every
    ``KernelLibrary`` of a matching type has the entry points as methods (``ctx.k.name(...)``),
    checked and raised like the engine's own.  ``written_down``: every launch reads what differs
    between steps of one shape from device memory, so a call may be repeated from a launch list
    (the entry points then join the native table of calls that a list can hold); False for an
    entry point whose arguments differ from step to step: a step that calls it is launched from
    Python every time, and the runner says so once."""
    import os
    if not os.path.isfile(source):
        raise FileNotFoundError(f"kernel source {source} does not exist")
    ext = KernelExtension(name, os.path.abspath(source), dict(entry_points), bool(written_down),
                          tuple(canonical_dtype(d) for d in dtypes))
    KERNEL_EXTENSIONS[name] = ext
    for d in ext.dtypes:
        build.register_library(_extension_library(name, d), [ext.source],
                               ["-DZSE_ACT_BF16=1" if d == BF16 else "-DZSE_ACT_BF16=0"], device=True)
    return ext


def _extension_library(name: str, dtype: str) -> str:
    return f"ext_{name}_{'bf16' if dtype == BF16 else 'f32'}"


class KernelLibrary:
    """One built kernel library; calling ``lib.zk_x(...)`` raises on a non-zero status."""

    def __init__(self, path: str, dtype: str):
        self.path = path
        self.dtype = dtype
        self._dll = C.CDLL(path)
        self._dll.zk_last_error.restype = C.c_char_p
        sigs = dict(KERNEL_SIGNATURES)
        if dtype == BF16:
            sigs.update(BF16_KERNEL_SIGNATURES)
        for name, args in sigs.items():
            try:
                fn = getattr(self._dll, name)
            except AttributeError:
                raise DeviceError(f"{path} lacks {name}: rebuild with `python -m zse_amd build`") from None
            fn.argtypes = args
            fn.restype = C.c_int
            setattr(self, name, self._wrap(name, fn))
        for name in ("zk_sample_scratch_bytes", "zk_sample_cut_scratch_bytes"):
            fn = getattr(self._dll, name)
            fn.restype, fn.argtypes = C.c_size_t, [_I]
            setattr(self, name, fn)
        for name in ("zk_sample_cut_row_bytes", "zk_sample_cut_mode_offset"):
            fn = getattr(self._dll, name)
            fn.restype, fn.argtypes = C.c_size_t, []
            setattr(self, name, fn)
        if dtype == BF16:
            self._dll.zk_attention_bf16_supports.restype = C.c_int
            self._dll.zk_attention_bf16_supports.argtypes = [_I, _I, _I, _I]
            self.zk_attention_bf16_supports = self._dll.zk_attention_bf16_supports
            self._dll.zk_attention_bf16_workspace.restype = C.c_size_t
            self._dll.zk_attention_bf16_workspace.argtypes = [_I, _I, _I, _I]
            self.zk_attention_bf16_workspace = self._dll.zk_attention_bf16_workspace
            self._dll.zk_attention_bf16_max_context.restype = C.c_longlong
            self._dll.zk_attention_bf16_max_context.argtypes = [_I, _I, _I, _I]
            self.zk_attention_bf16_max_context = self._dll.zk_attention_bf16_max_context
            self._dll.zk_attention_bf16_portion_workspace.restype = C.c_size_t
            self._dll.zk_attention_bf16_portion_workspace.argtypes = [_I, _I, _I, _I]
            self.zk_attention_bf16_portion_workspace = self._dll.zk_attention_bf16_portion_workspace
            self._dll.zk_attention_bf16_portion_kernel.restype = C.c_int
            self._dll.zk_attention_bf16_portion_kernel.argtypes = [_I]
            self.zk_attention_bf16_portion_kernel = self._dll.zk_attention_bf16_portion_kernel
            self._dll.zk_qkv_rope_bf16_supports.restype = C.c_int
            self._dll.zk_qkv_rope_bf16_supports.argtypes = [_I, _I, _I, _I]
            self.zk_qkv_rope_bf16_supports = self._dll.zk_qkv_rope_bf16_supports
            self._dll.zk_head_pick_bf16_workspace.restype = C.c_size_t
            self._dll.zk_head_pick_bf16_workspace.argtypes = [_I, _I]
            self.zk_head_pick_bf16_workspace = self._dll.zk_head_pick_bf16_workspace
            self._dll.zk_gemm_bf16_workspace.restype = C.c_size_t
            self._dll.zk_gemm_bf16_workspace.argtypes = []
            self.zk_gemm_bf16_workspace = self._dll.zk_gemm_bf16_workspace
        self._init_steplists()
        want = 1 if dtype == BF16 else 0
        if self._dll.zk_act_is_bf16() != want:
            raise DeviceError(f"{path} was built for the other storage type")
        self._attached: Dict[str, object] = {}      # extension name -> its loaded library
        self.attach_extensions()

    def has(self, name: str) -> bool:
        return hasattr(self, name)

    def attach_extensions(self) -> None:
        """Loads the libraries of every registered extension that this library has not met yet
        (built first if need be), makes their entry points methods of this object and enters
        those that may be written down into the native table of a launch list's calls."""
        for ext in list(KERNEL_EXTENSIONS.values()):
            if self.dtype not in ext.dtypes or self._attached.get(ext.name) is ext:
                continue
            path = build.ensure(_extension_library(ext.name, self.dtype))
            dll = C.CDLL(path)
            dll.zk_last_error.restype = C.c_char_p
            if dll.zk_act_is_bf16() != (1 if self.dtype == BF16 else 0):
                raise DeviceError(f"{path} was built for the other storage type")
            for name, args in ext.entry_points.items():
                try:
                    fn = getattr(dll, name)
                except AttributeError:
                    raise DeviceError(f"{path} (built from {ext.source}) lacks {name}") from None
                fn.argtypes, fn.restype = list(args), C.c_int
                setattr(self, name, self._wrap(name, fn, dll))
                self._op_ids.pop(name, None)
                if ext.written_down:
                    try:
                        packed, nargs = getattr(dll, name + "_packed"), getattr(dll, name + "_nargs")
                    except AttributeError:
                        raise DeviceError(f"{ext.source}: ZK_PACKED({name}) is missing, which an entry point "
                                          f"that may be written down needs") from None
                    nargs.restype = C.c_int
                    if nargs() != len(args):
                        raise DeviceError(f"{name}: {len(args)} argument types were registered, the entry point "
                                          f"takes {nargs()}")
                    op = self._dll.zk_steplist_register(name.encode(), len(args), C.cast(packed, C.c_void_p))
                    if op < 0:
                        raise DeviceError(f"{name} could not be entered into the table of written-down calls")
                self._owner_of[name] = dll
            self._attached[ext.name] = ext
            self._keep_alive.append(dll)

    def _wrap(self, name, fn, dll=None):
        dll = dll or self._dll
        lib = self

        def call(*a):
            rc = fn(*a)
            if rc != 0:
                raise DeviceError(f"{name} failed ({rc}): {dll.zk_last_error().decode()}")
            if lib._writing is not None:
                lib._write_down(name, fn.argtypes, a)
        call.__name__ = name
        return call

    # ---- a step's launches written down on the native side, and launched again from there
    def _init_steplists(self):
        d = self._dll
        d.zk_steplist_op.restype, d.zk_steplist_op.argtypes = C.c_int, [C.c_char_p]
        d.zk_steplist_create.restype, d.zk_steplist_create.argtypes = C.c_void_p, []
        d.zk_steplist_destroy.restype, d.zk_steplist_destroy.argtypes = None, [C.c_void_p]
        d.zk_steplist_size.restype, d.zk_steplist_size.argtypes = C.c_int, [C.c_void_p]
        d.zk_steplist_add.restype = C.c_int
        d.zk_steplist_add.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_uint64), C.c_int]
        d.zk_steplist_run.restype = C.c_int
        d.zk_steplist_run.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_int)]
        d.zk_steplist_name.restype, d.zk_steplist_name.argtypes = C.c_char_p, [C.c_void_p, C.c_int]
        d.zk_steplist_register.restype = C.c_int
        d.zk_steplist_register.argtypes = [C.c_char_p, C.c_int, C.c_void_p]
        self._owner_of: Dict[str, object] = {}      # entry point of an extension -> its library
        self._keep_alive = []
        self.not_written: Optional[str] = None      # the entry point that kept the last list from being written
        self._writing = None          # the list being written, while a step runs call by call
        self._writable = True
        self._op_ids: Dict[str, int] = {}

    def steplist_begin(self) -> int:
        """From now on every kernel call is also written into a new list (and still runs)."""
        if self._writing is not None:
            raise DeviceError("a step list is being written already")
        self._writing = self._dll.zk_steplist_create()
        self._writable = True
        return self._writing

    def steplist_end(self) -> Optional[int]:
        """Stops writing; the list's handle, or None if some call could not be written down
        (the list is then destroyed)."""
        handle, self._writing = self._writing, None
        if handle is not None and not self._writable:
            self._dll.zk_steplist_destroy(handle)
            return None
        return handle

    def steplist_run(self, handle: int, stream) -> None:
        at = C.c_int(-1)
        rc = self._dll.zk_steplist_run(handle, stream, C.byref(at))
        if rc != 0:
            name = self._dll.zk_steplist_name(handle, at.value).decode()
            owner = self._owner_of.get(name, self._dll)
            raise DeviceError(f"{name} (call {at.value} of a written-down step) failed ({rc}): "
                              f"{owner.zk_last_error().decode()}")

    def steplist_destroy(self, handle: int) -> None:
        self._dll.zk_steplist_destroy(handle)

    def steplist_size(self, handle: int) -> int:
        return self._dll.zk_steplist_size(handle)

    def _write_down(self, name, argtypes, args) -> None:
        op = self._op_ids.get(name)
        if op is None:
            op = self._op_ids[name] = self._dll.zk_steplist_op(name.encode())
        if op < 0 or not self._writable:
            if op < 0 and self._writable:
                self.not_written = name
            self._writable = False          # an entry point the native side cannot call again
            return
        words = (C.c_uint64 * len(args))()
        for i, (t, v) in enumerate(zip(argtypes, args)):
            if t is _F:
                words[i] = _struct.unpack("<I", _struct.pack("<f", v))[0]
            elif t is _I:
                words[i] = int(v) & 0xFFFFFFFFFFFFFFFF
            elif v is None:
                words[i] = 0
            elif isinstance(v, int):
                words[i] = v
            elif hasattr(v, "value"):
                words[i] = int(v.value or 0)
            else:
                words[i] = 1                # a by-reference output: the native side brings its own
        if self._dll.zk_steplist_add(self._writing, op, words, len(args)) != 0:
            self._writable = False


class Runtime:
    """The process's handle on GPU 0 (or ``device``)."""

    _instance: Optional["Runtime"] = None

    @classmethod
    def get(cls, device: int = 0) -> "Runtime":
        if cls._instance is None:
            cls._instance = Runtime(device)
        return cls._instance

    def __init__(self, device: int = 0):
        path = build.ensure("runtime")
        self.lib = C.CDLL(path)
        self.lib.zrt_last_error.restype = C.c_char_p
        for name in ("zrt_malloc", "zrt_free", "zrt_host_alloc", "zrt_host_free", "zrt_h2d", "zrt_d2h",
                     "zrt_d2d", "zrt_stream_create", "zrt_stream_destroy", "zrt_stream_sync",
                     "zrt_device_sync", "zrt_event_create", "zrt_event_record", "zrt_event_sync",
                     "zrt_event_elapsed_ms", "zrt_event_destroy", "zrt_capture_begin",
                     "zrt_capture_end", "zrt_graph_launch", "zrt_graph_destroy", "zrt_init",
                     "zrt_device_count", "zrt_device_info"):
            getattr(self.lib, name).restype = C.c_int
        self.lib.zrt_h2d.argtypes = [_VP, _VP, _SZ, _VP, _I]
        self.lib.zrt_d2h.argtypes = [_VP, _VP, _SZ, _VP, _I]
        self.lib.zrt_d2d.argtypes = [_VP, _VP, _SZ, _VP]
        self.lib.zrt_free.argtypes = [_VP]
        self.lib.zrt_host_free.argtypes = [_VP]
        self.lib.zrt_stream_sync.argtypes = [_VP]
        self.lib.zrt_stream_destroy.argtypes = [_VP]
        self.lib.zrt_event_record.argtypes = [_VP, _VP]
        self.lib.zrt_event_sync.argtypes = [_VP]
        self.lib.zrt_event_elapsed_ms.argtypes = [_VP, _VP, _VP]
        self.lib.zrt_event_destroy.argtypes = [_VP]
        self.lib.zrt_capture_begin.argtypes = [_VP]
        self.lib.zrt_capture_end.argtypes = [_VP, _VP]
        self.lib.zrt_graph_launch.argtypes = [_VP, _VP]
        self.lib.zrt_graph_destroy.argtypes = [_VP]
        n = C.c_int(0)
        rc = self.lib.zrt_device_count(C.byref(n))
        if rc != 0 or n.value < 1:
            raise DeviceError("no HIP device is visible: this engine runs on a GPU only "
                              f"({self.lib.zrt_last_error().decode()})")
        self.device = device
        self._check(self.lib.zrt_init(C.c_int(device)), "init")
        self.allocated = 0
        self._capturing = False
        self._free_later = []
        self._kernels: Dict[str, KernelLibrary] = {}
        s = C.c_void_p()
        self._check(self.lib.zrt_stream_create(C.byref(s)), "stream create")
        self.stream = s.value

    # -- errors
    def _check(self, rc: int, what: str):
        if rc != 0:
            raise DeviceError(f"{what} failed ({rc}): {self.lib.zrt_last_error().decode()}")

    # -- info
    def info(self) -> DeviceInfo:
        name = C.create_string_buffer(256)
        arch = C.create_string_buffer(256)
        total, free = C.c_size_t(), C.c_size_t()
        cus = C.c_int()
        self._check(self.lib.zrt_device_info(C.c_int(self.device), name, 256, C.byref(total),
                                             C.byref(free), C.byref(cus), arch, 256), "device info")
        return DeviceInfo(name.value.decode(), arch.value.decode(), total.value, free.value, cus.value)

    # -- kernels
    def kernels(self, dtype: str) -> KernelLibrary:
        dtype = canonical_dtype(dtype)
        if dtype not in self._kernels:
            name = "kernels_bf16" if dtype == BF16 else "kernels_f32"
            self._kernels[dtype] = KernelLibrary(build.ensure(name), dtype)
        elif len(self._kernels[dtype]._attached) != len(KERNEL_EXTENSIONS) or \
                any(self._kernels[dtype]._attached.get(n) is not e for n, e in KERNEL_EXTENSIONS.items()
                    if dtype in e.dtypes):
            self._kernels[dtype].attach_extensions()      # kernels registered since the library was loaded
        return self._kernels[dtype]

    # -- memory
    def empty(self, shape, dtype: str) -> Tensor:
        shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        n = ITEMSIZE[dtype]
        for s in shape:
            n *= s
        a = Allocation(self, n)
        return Tensor(a.ptr, shape, dtype, a)

    def zeros(self, shape, dtype: str) -> Tensor:
        t = self.empty(shape, dtype)
        self.zero_(t)
        return t

    def zero_(self, t: Tensor):
        nbytes = (t.nbytes + 3) // 4 * 4
        self.kernels(F32).zk_zero(t.ptr, nbytes, self.stream)

    def pinned(self, nbytes: int) -> PinnedBuffer:
        return PinnedBuffer(self, nbytes)

    def upload(self, arr: np.ndarray, dtype: Optional[str] = None) -> Tensor:
        """Copy a host array to a new device tensor (synchronous).  ``dtype`` only
        labels the result; the bytes go up as they are."""
        arr = np.ascontiguousarray(arr)
        if dtype is None:
            dtype = {np.dtype(np.float32): F32, np.dtype(np.int32): I32, np.dtype(np.uint16): BF16,
                     np.dtype(np.float64): F64}[arr.dtype]
        t = self.empty(arr.shape, dtype)
        if t.nbytes != arr.nbytes:
            raise ValueError(f"{arr.dtype} array does not store {dtype}")
        self.copy_h2d(t.ptr, arr)
        return t

    def copy_h2d(self, dst_ptr: int, arr: np.ndarray):
        arr = np.ascontiguousarray(arr)
        if arr.nbytes:
            self._check(self.lib.zrt_h2d(dst_ptr, arr.ctypes.data, arr.nbytes, self.stream, 0), "h2d")

    def copy_h2d_async(self, dst_ptr: int, host_ptr: int, nbytes: int):
        if nbytes:
            self._check(self.lib.zrt_h2d(dst_ptr, host_ptr, nbytes, self.stream, 1), "h2d")

    def copy_d2d(self, dst_ptr: int, src_ptr: int, nbytes: int):
        if nbytes:
            self._check(self.lib.zrt_d2d(dst_ptr, src_ptr, nbytes, self.stream), "d2d")

    def download(self, t: Tensor) -> np.ndarray:
        """Copy a device tensor to a new host array (synchronous)."""
        out = np.empty(t.shape, dtype=NUMPY_OF[t.dtype])
        if out.nbytes:
            self._check(self.lib.zrt_d2h(out.ctypes.data, t.ptr, out.nbytes, self.stream, 0), "d2h")
        return out

    def download_f32(self, t: Tensor) -> np.ndarray:
        a = self.download(t)
        if t.dtype == BF16:
            return (a.astype(np.uint32) << 16).view(np.float32)
        return a.astype(np.float32, copy=False)

    def copy_d2h_async(self, host_ptr: int, src_ptr: int, nbytes: int):
        """Enqueue a copy into pinned host memory; the data is there once an event recorded
        after it has passed."""
        if nbytes:
            self._check(self.lib.zrt_d2h(host_ptr, src_ptr, nbytes, self.stream, 1), "d2h")

    def sync(self):
        self._check(self.lib.zrt_stream_sync(self.stream), "stream sync")

    # -- events
    def event(self) -> int:
        e = C.c_void_p()
        self._check(self.lib.zrt_event_create(C.byref(e)), "event create")
        return e.value

    def record(self, ev: int):
        self._check(self.lib.zrt_event_record(ev, self.stream), "event record")

    def wait_event(self, ev: int):
        self._check(self.lib.zrt_event_sync(ev), "event sync")

    def elapsed_ms(self, a: int, b: int) -> float:
        self._check(self.lib.zrt_event_sync(b), "event sync")
        ms = C.c_float()
        self._check(self.lib.zrt_event_elapsed_ms(a, b, C.byref(ms)), "event elapsed")
        return ms.value

    def free_device(self, ptr: int) -> None:
        """Frees a device allocation; while a graph is being captured the free waits until the
        capture has ended (freeing synchronizes, which a capturing stream does not allow, and
        the garbage collector may drop a tensor at any moment)."""
        if self._capturing:
            self._free_later.append(ptr)
        else:
            self.lib.zrt_free(C.c_void_p(ptr))

    def free_host(self, ptr: int) -> None:
        """Frees page-locked host memory, after a capture in progress has ended."""
        if self._capturing:
            self._free_later.append(-ptr)
        else:
            self.lib.zrt_host_free(C.c_void_p(ptr))

    # -- graphs
    def capture_begin(self):
        self._check(self.lib.zrt_capture_begin(self.stream), "capture begin")
        self._capturing = True

    def capture_end(self) -> int:
        g = C.c_void_p()
        try:
            self._check(self.lib.zrt_capture_end(self.stream, C.byref(g)), "capture end")
        finally:
            self._capturing = False
            pending, self._free_later = self._free_later, []
            for p in pending:           # device pointers as they are, host pointers negated
                (self.lib.zrt_free if p > 0 else self.lib.zrt_host_free)(C.c_void_p(abs(p)))
        return g.value

    def graph_launch(self, g: int):
        self._check(self.lib.zrt_graph_launch(g, self.stream), "graph launch")

    def graph_destroy(self, g: int):
        self.lib.zrt_graph_destroy(g)
