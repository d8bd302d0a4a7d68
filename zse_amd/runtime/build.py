"""Building the native libraries with hipcc for gfx950.

Three libraries are built from ``zse_amd/csrc``: ``runtime`` (host-side HIP
calls), ``kernels_f32`` and ``kernels_bf16`` (the same kernel sources compiled
once per storage type, plus the bf16-only tuned kernels).  A process builds
only what it is about to load, so a 32-bit run never waits for the bf16
kernels.  The reference compiles kernel strings at run time with hiprtc and
keeps the binaries in a per-user cache (orchestrator/kernels.py:2915-3010);
here sources are files, compiled ahead of time, and the libraries sit beside
the package (or under a temporary folder when that is read-only).
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, List

CSRC = os.path.normpath(os.path.join(os.path.dirname(__file__), "..", "csrc"))
PKG_LIB_DIR = os.path.normpath(os.path.join(os.path.dirname(__file__), "..", "_lib"))
ARCH = "gfx950"

COMMON_KERNELS = ["elementwise.hip", "gemm_plain.hip", "attention_plain.hip", "sampling.hip", "probe.hip", "steplist.hip"]
BF16_KERNELS = ["gemm_bf16.hip", "attention_bf16.hip"]

LIBRARIES: Dict[str, dict] = {
    "runtime": {"sources": ["runtime.cpp"], "defines": [], "device": False},
    "kernels_f32": {"sources": COMMON_KERNELS, "defines": ["-DZSE_ACT_BF16=0"], "device": True},
    "kernels_bf16": {"sources": COMMON_KERNELS + BF16_KERNELS, "defines": ["-DZSE_ACT_BF16=1"],
                     "device": True},
}



def register_library(name: str, sources: List[str], defines: List[str], device: bool = True) -> None:
    """Adds a library to build: ``sources`` are files under ``zse_amd/csrc`` or absolute paths
    (a part's own kernels live with the part), compiled with this module's flags and the
    headers of ``zse_amd/csrc`` on the include path.  It is then built, stamped and found like
    the three above (``ensure``, ``build``, ``build_all``)."""
    if name in ("runtime", "kernels_f32", "kernels_bf16"):
        raise BuildError(f"library {name} is the engine's own")
    LIBRARIES[name] = {"sources": list(sources), "defines": list(defines), "device": bool(device)}


DEVICE_FLAGS = [f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
HOST_FLAGS = ["-O3", "-fPIC", "-std=c++17", "-Wno-unused-result"]


class BuildError(RuntimeError):
    pass


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the native "
                     "libraries cannot be built")


def _writable(d: str) -> bool:
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def lib_dir() -> str:
    """Where libraries are looked for and built: beside the package if it can be
    written, else a per-user folder under the temporary directory."""
    if os.environ.get("ZSE_AMD_LIB_DIR"):
        d = os.environ["ZSE_AMD_LIB_DIR"]
        os.makedirs(d, exist_ok=True)
        return d
    if _writable(PKG_LIB_DIR):
        return PKG_LIB_DIR
    d = os.path.join(tempfile.gettempdir(), f"zse_amd_lib_{os.getuid()}")
    os.makedirs(d, exist_ok=True)
    return d


def lib_path(name: str) -> str:
    return os.path.join(lib_dir(), f"libzse_{name}.so")


def source_digest(name: str) -> str:
    spec = LIBRARIES[name]
    h = hashlib.sha256()
    headers = [f for f in os.listdir(CSRC) if f.endswith(".h")] if os.path.isdir(CSRC) else []
    for f in sorted(spec["sources"] + headers, key=os.path.basename):
        p = os.path.join(CSRC, f)            # an absolute path stays what it is
        if os.path.isfile(p):
            h.update(os.path.basename(f).encode())     # not the folder: a copy of the tree elsewhere is the same source
            with open(p, "rb") as fh:
                h.update(fh.read())
    h.update(" ".join(spec["defines"] + DEVICE_FLAGS + HOST_FLAGS).encode())
    return h.hexdigest()[:16]


def is_current(name: str) -> bool:
    stamp = lib_path(name) + ".stamp"
    if not (os.path.isfile(lib_path(name)) and os.path.isfile(stamp)):
        return False
    with open(stamp) as f:
        return f.read().strip() == source_digest(name)


def _run(cmd: List[str], what: str) -> None:
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise BuildError(f"{what} failed ({' '.join(cmd)}):\n{p.stdout[-4000:]}")


def build(name: str, verbose: bool = True, jobs: int = 0) -> str:
    """Compile and link one library; returns its path."""
    spec = LIBRARIES[name]
    hipcc = hipcc_path()
    out = lib_path(name)
    work = os.path.join(lib_dir(), f"obj_{name}")
    os.makedirs(work, exist_ok=True)
    flags = HOST_FLAGS + spec["defines"] + (DEVICE_FLAGS if spec["device"] else [])
    srcs = [s for s in spec["sources"] if os.path.isfile(os.path.join(CSRC, s))]
    missing = [s for s in spec["sources"] if s not in srcs]
    if missing:
        raise BuildError(f"library {name}: source files missing: {missing}")
    t0 = time.time()
    done = threading.Event()

    def ticker():
        while not done.wait(20.0):
            print(f"[zse_amd] still compiling {name} ({time.time() - t0:.0f} s)", file=sys.stderr,
                  flush=True)

    if verbose:
        print(f"[zse_amd] compiling {name}: {len(srcs)} files for {ARCH} into {out}",
              file=sys.stderr, flush=True)
        threading.Thread(target=ticker, daemon=True).start()
    try:
        objs = [os.path.join(work, os.path.splitext(os.path.basename(s))[0] + ".o") for s in srcs]

        def one(i):
            _run([hipcc, "-c", os.path.join(CSRC, srcs[i]), "-o", objs[i], "-I", CSRC] + flags,
                 f"compiling {srcs[i]}")
            if verbose:
                print(f"[zse_amd]   {os.path.basename(srcs[i])} done ({time.time() - t0:.0f} s)", file=sys.stderr,
                      flush=True)

        workers = jobs or min(len(srcs), max(1, min(os.cpu_count() or 4, 16)))
        with ThreadPoolExecutor(max_workers=workers) as ex:
            list(ex.map(one, range(len(srcs))))
        tmp = out + f".tmp{os.getpid()}"
        link = [hipcc, "-shared", "-fPIC", "-o", tmp] + objs
        if spec["device"]:
            link.append(f"--offload-arch={ARCH}")
        _run(link, f"linking {name}")
        os.replace(tmp, out)
        with open(out + ".stamp", "w") as f:
            f.write(source_digest(name))
    finally:
        done.set()
        shutil.rmtree(work, ignore_errors=True)
    if verbose:
        print(f"[zse_amd] built {name} in {time.time() - t0:.0f} s", file=sys.stderr, flush=True)
    return out


def ensure(name: str, verbose: bool = True) -> str:
    """Path of a library that was built from the sources as they are now: a library whose
    stamp matches is used, anything else (none there, or one older than its sources) is
    built first.  A stale library is never loaded: without hipcc this raises."""
    out = lib_path(name)
    if os.path.isfile(out) and is_current(name):
        return out
    if os.path.isfile(out) and verbose:
        print(f"[zse_amd] {out} does not match its sources; building it again", file=sys.stderr,
              flush=True)
    return build(name, verbose=verbose)


def build_all(verbose: bool = True) -> List[str]:
    return [build(n, verbose=verbose) for n in LIBRARIES]
