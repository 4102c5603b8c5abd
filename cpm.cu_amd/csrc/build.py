"""Builds and loads the HIP libraries of this package (gfx950 only).

The kernels are grouped into a few shared libraries so that a model compiles,
at its first use, only what it needs (a model without block-sparse attention
never builds ``sparse``).  A library is rebuilt when the text of its sources or
the compiler flags change; it is written beside the sources, or into a per-user
temporary folder when that is not writable.  There is no CPU fallback: if hipcc
or a library is missing, loading raises.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, List

HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"

# library -> sources (headers are hashed with every library)
MODULES: Dict[str, List[str]] = {
    "core": ["elementwise.hip", "sampling.hip"],
    "gemm": ["gemm.hip"],
    "attention": ["attention.hip"],
    "sparse": ["sparse.hip"],
    "qkv": ["qkv_rope.hip", "strip.hip"],
}
HEADERS = ["common.h"]
# headers of single libraries
MODULE_HEADERS: Dict[str, List[str]] = {"attention": ["no_alloc.h"]}

# -packed-fp32-ops off: the compiler must not form packed float instructions on its own
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


# extra flags of single libraries
#   attention: matrix-core results stay in ordinary vector registers (with the accumulation registers the
#   compiler moves the running output there and back around every rescale); no score is ever NaN, which
#   spares a canonicalising instruction before every max
MODULE_FLAGS: Dict[str, List[str]] = {
    "attention": ["-mllvm", "-amdgpu-mfma-vgpr-form", "-fno-honor-nans"],
}


def _flags(module: str) -> List[str]:
    return HIPCC_FLAGS + MODULE_FLAGS.get(module, [])


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP libraries cannot be built")


def _digest(module: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join(_flags(module)).encode())
    for name in HEADERS + MODULE_HEADERS.get(module, []) + MODULES[module]:
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    return h.hexdigest()


def _out_dir() -> str:
    if os.access(HERE, os.W_OK):
        return HERE
    d = os.path.join(tempfile.gettempdir(), f"cpmcu_amd_build_{os.getuid()}")
    os.makedirs(d, exist_ok=True)
    return d


def lib_path(module: str, out_dir: str | None = None) -> str:
    return os.path.join(out_dir or _out_dir(), f"libcpmcu_{module}.so")


def is_built(module: str) -> bool:
    for d in {HERE, _out_dir()}:
        p = lib_path(module, d)
        if os.path.isfile(p) and os.path.isfile(p + ".stamp"):
            with open(p + ".stamp") as f:
                if f.read().strip() == _digest(module):
                    return True
    return False


def build(module: str, verbose: bool = True) -> str:
    """Compile one library now, whether or not a current one exists."""
    out = lib_path(module)
    tmp = f"{out}.{os.getpid()}.tmp"
    cmd = [_hipcc()] + _flags(module) + ["-I", HERE, "-o", tmp] + [os.path.join(HERE, s) for s in MODULES[module]]
    t0 = time.time()
    if verbose:
        print(f"[cpmcu_amd] compiling {module} ({', '.join(MODULES[module])}) for {ARCH} ...", file=sys.stderr, flush=True)
    done = threading.Event()

    def ticker():
        while not done.wait(15.0):
            print(f"[cpmcu_amd]   still compiling {module} ({time.time() - t0:.0f} s)", file=sys.stderr, flush=True)

    th = threading.Thread(target=ticker, daemon=True)
    if verbose:
        th.start()
    try:
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    finally:
        done.set()
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.unlink(tmp)
        raise BuildError(f"hipcc failed for library '{module}':\n{' '.join(cmd)}\n{proc.stdout}")
    os.replace(tmp, out)
    with open(out + ".stamp", "w") as f:
        f.write(_digest(module))
    if verbose:
        print(f"[cpmcu_amd] built {os.path.basename(out)} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    return out


def build_all(verbose: bool = True):
    for m in MODULES:
        build(m, verbose)


_loaded: Dict[str, ctypes.CDLL] = {}


def load(module: str) -> ctypes.CDLL:
    """The library, compiled first if no current build of it exists."""
    lib = _loaded.get(module)
    if lib is not None:
        return lib
    if module not in MODULES:
        raise BuildError(f"unknown library '{module}' (known: {sorted(MODULES)})")
    path = None
    digest = _digest(module)
    for d in (HERE, _out_dir()):
        p = lib_path(module, d)
        if os.path.isfile(p) and os.path.isfile(p + ".stamp"):
            with open(p + ".stamp") as f:
                if f.read().strip() == digest:
                    path = p
                    break
    if path is None:
        path = build(module)
    lib = ctypes.CDLL(path)
    _loaded[module] = lib
    return lib
