"""Run-time compilation of the kernel sources for fixed shapes: the plug-in point of the reference's
DeepEP-driven examples.

There, one `impls/*.cuh` header is replaced in an include overlay and DeepEP compiles it just in
time with top-k, experts, ranks and the hidden size as template parameters
(datasets/example080_deepep_jit_dispatch_payload/nv/build_and_run.py:154-172, `_C.init_jit(overlay_root,
cuda_home, nccl_root)` at :678; the parameters at .../empty_deepep_jit_dispatch_payload.cu:17-30).
Here the shipped library takes every shape at run time.  This module rebuilds the same sources with
hipcc and any of top-k / experts / ranks / payload row bytes / combine hidden size fixed as
constants (the MI_EP_FIXED_* macros of csrc/ep_device.h), optionally with files of an overlay folder
standing in for the shipped sources of the same name, caches the result by content, and hands back a
library with the same C ABI that refuses other shapes with MI_EP_EINVAL:

    jit.init_jit(overlay_root=None, rocm_home="/opt/rocm")
    lib = jit.activate(num_topk=8, num_experts=256, num_ranks=8, row_bytes=14336, hidden=7168)
    ...  # every commbench_amd.ops call now runs the kernels compiled for that shape
    jit.deactivate()

Cache: $EP_JIT_CACHE_DIR, else commbench_amd/jit_cache next to the shipped library.
"""
import ctypes
import hashlib
import os
import shutil
import subprocess
from typing import Dict, Optional

from . import _lib
from . import build as hip_build

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
HEADERS = ["ep_device.h"]
SHAPE_MACROS = {
    "num_topk": "MI_EP_FIXED_TOPK",
    "num_experts": "MI_EP_FIXED_EXPERTS",
    "num_ranks": "MI_EP_FIXED_RANKS",
    "row_bytes": "MI_EP_FIXED_ROW_BYTES",
    "hidden": "MI_EP_FIXED_HIDDEN",
}

_config = {"overlay_root": None, "rocm_home": None, "cache_dir": None}


def init_jit(overlay_root: Optional[str] = None, rocm_home: Optional[str] = None,
             cache_dir: Optional[str] = None) -> None:
    """Sets where later compilations take their sources and compiler from.  A file of
    `overlay_root` named like a shipped kernel source (ep_layout.hip, ep_permute.hip, ep_combine.hip,
    ep_abi.hip, ep_host.hip, ep_device.h) replaces it, as the reference's overlay replaces one
    header; `rocm_home` is the toolchain root (hipcc under bin/)."""
    if overlay_root is not None and not os.path.isdir(overlay_root):
        raise ValueError(f"overlay_root {overlay_root!r} is not a folder")
    _config.update(overlay_root=overlay_root, rocm_home=rocm_home, cache_dir=cache_dir)


def cache_dir() -> str:
    return _config["cache_dir"] or os.environ.get("EP_JIT_CACHE_DIR") or os.path.join(PKG_DIR, "jit_cache")


def _hipcc() -> str:
    home = _config["rocm_home"] or os.environ.get("ROCM_HOME") or "/opt/rocm"
    return os.environ.get("HIPCC", os.path.join(home, "bin", "hipcc"))


def source_files() -> Dict[str, str]:
    """name -> path of every file of the build, the overlay's files first."""
    files = {}
    for name in hip_build.SOURCES + HEADERS:
        path = os.path.join(hip_build.CSRC_DIR, name)
        overlay = _config["overlay_root"]
        if overlay is not None and os.path.exists(os.path.join(overlay, name)):
            path = os.path.join(overlay, name)
        files[name] = path
    return files


def _defines(shapes: Dict[str, int]) -> Dict[str, int]:
    unknown = set(shapes) - set(SHAPE_MACROS)
    if unknown:
        raise ValueError(f"unknown shape name(s) {sorted(unknown)}; known: {sorted(SHAPE_MACROS)}")
    return {SHAPE_MACROS[k]: int(v) for k, v in sorted(shapes.items()) if v}


def library_path(**shapes: int) -> str:
    """Where the library for these fixed shapes lives in the cache: named by a hash of the sources
    (overlay applied), the public header, the flags and the shapes."""
    h = hashlib.sha256()
    for name, path in sorted(source_files().items()):
        h.update(name.encode())
        with open(path, "rb") as f:
            h.update(f.read())
    with open(os.path.join(ROOT, "include", "mi_ep.h"), "rb") as f:
        h.update(f.read())
    h.update(" ".join(hip_build.HIPCC_FLAGS).encode())
    h.update(repr(sorted(_defines(shapes).items())).encode())
    return os.path.join(cache_dir(), f"libmi_ep_{h.hexdigest()[:16]}.so")


def compile_library(**shapes: int) -> str:
    """Compiles (or finds in the cache) the library with the given shapes fixed; returns its path."""
    out = library_path(**shapes)
    if os.path.exists(out):
        return out
    os.makedirs(cache_dir(), exist_ok=True)
    # The sources include "../../include/mi_ep.h": stage them in a tree of the same shape.
    stage = out[:-3] + f"_src{os.getpid()}"          # per process: two may build the same library at once
    shutil.rmtree(stage, ignore_errors=True)
    csrc = os.path.join(stage, "commbench_amd", "csrc")
    os.makedirs(csrc)
    os.makedirs(os.path.join(stage, "include"))
    shutil.copy(os.path.join(ROOT, "include", "mi_ep.h"), os.path.join(stage, "include", "mi_ep.h"))
    for name, path in source_files().items():
        shutil.copy(path, os.path.join(csrc, name))
    cmd = [_hipcc(), *hip_build.HIPCC_FLAGS, *[f"-D{k}={v}" for k, v in _defines(shapes).items()],
           "-o", f"{out}.{os.getpid()}.tmp"] + [os.path.join(csrc, s) for s in hip_build.SOURCES]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    shutil.rmtree(stage, ignore_errors=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stdout + proc.stderr)
    os.replace(f"{out}.{os.getpid()}.tmp", out)     # atomic: a reader sees the old file or the whole new one
    return out


def load_library(**shapes: int) -> ctypes.CDLL:
    """The compiled library, loaded and bound to the prototypes of include/mi_ep.h."""
    return _lib.bind(ctypes.CDLL(compile_library(**shapes)))


def activate(**shapes: int) -> ctypes.CDLL:
    """Compiles, loads and installs the library for these shapes: commbench_amd.ops runs on it until
    deactivate().  Calls with other shapes then fail with MI_EP_EINVAL."""
    lib = load_library(**shapes)
    _lib.use(lib)
    return lib


def deactivate() -> None:
    """Back to the shipped library (every shape at run time)."""
    _lib.use(None)
