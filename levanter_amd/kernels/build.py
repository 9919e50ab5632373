"""Compiles the HIP sources under ``csrc/`` into one shared library for gfx950.

The library is built in the tree (``levanter_amd/kernels/liblevanter_amd_hip.so``); when the
tree cannot be written, in a per-user folder under the temporary directory. A build compiles
the sources in parallel and prints a line per file, so a first call in a fresh checkout
shows progress. ``ensure_built`` builds only when there is no library or its sources changed.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from typing import List, Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(_HERE), "csrc")
LIB_NAME = "liblevanter_amd_hip.so"
ARCH = "gfx950"

MFMA_ATTENTION_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128)

# (source, extra defines, object name)
SOURCES = [
    ("errors.hip", [], "errors.o"),
    ("elementwise.hip", [], "elementwise.o"),
    ("gemm_simple.hip", [], "gemm_simple.o"),
    ("attention_simple.hip", [], "attention_simple.o"),
    ("gemm_mfma.hip", [], "gemm_mfma.o"),
    ("attention_dispatch.hip", [], "attention_dispatch.o"),
] + [("attention_mfma.hip", [f"-DLEV_HD={hd}"], f"attention_mfma_hd{hd}.o") for hd in MFMA_ATTENTION_HEAD_DIMS]

# -packed-fp32-ops off: packed 32-bit float instructions are not to be generated on this hardware pool
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


def _log(msg: str) -> None:
    print(f"[levanter_amd build] {msg}", file=sys.stderr, flush=True)


def find_hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def source_hash() -> str:
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(CSRC, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()[:16]


def _writable(d: str) -> bool:
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".probe_{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def library_dir() -> str:
    if _writable(_HERE):
        return _HERE
    d = os.path.join(tempfile.gettempdir(), f"levanter_amd_{os.getuid()}")
    os.makedirs(d, exist_ok=True)
    return d


def library_path() -> str:
    return os.path.join(library_dir(), LIB_NAME)


def _stamp_path(lib: str) -> str:
    return lib + ".hash"


def is_current(lib: Optional[str] = None) -> bool:
    lib = lib or library_path()
    try:
        with open(_stamp_path(lib)) as f:
            return os.path.isfile(lib) and f.read().strip() == source_hash()
    except OSError:
        return False


def build(force: bool = True, jobs: Optional[int] = None) -> str:
    """Compile every source and link the library. Returns its path."""
    hipcc = find_hipcc()
    if hipcc is None:
        raise RuntimeError("hipcc not found: the HIP library of levanter_amd cannot be built (set HIPCC or install ROCm)")
    lib = library_path()
    if not force and is_current(lib):
        return lib
    obj_dir = os.path.join(library_dir(), "_build")
    os.makedirs(obj_dir, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1, len(SOURCES))
    env = dict(os.environ)
    home = env.get("HOME", "")
    if not home or not os.path.isdir(home) or not os.access(home, os.W_OK):
        env["HOME"] = tempfile.gettempdir()  # hipcc wants a HOME it can write its caches to
    t0 = time.time()
    _log(f"compiling {len(SOURCES)} HIP objects for {ARCH} with {jobs} jobs (first call only) ...")

    def compile_one(item) -> str:
        src, defines, obj_name = item
        obj = os.path.join(obj_dir, obj_name)
        cmd = [hipcc, *HIPCC_FLAGS, *defines, "-c", os.path.join(CSRC, src), "-o", obj]
        t = time.time()
        r = subprocess.run(cmd, capture_output=True, text=True, env=env)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src} {' '.join(defines)}:\n{_filter(r.stderr)}")
        _log(f"  {obj_name[:-2]} done in {time.time() - t:.0f}s")
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs: List[str] = list(pool.map(compile_one, SOURCES))
    tmp = lib + f".tmp{os.getpid()}"
    r = subprocess.run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs], capture_output=True, text=True, env=env)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed to link {LIB_NAME}:\n{_filter(r.stderr)}")
    os.replace(tmp, lib)
    with open(_stamp_path(lib), "w") as f:
        f.write(source_hash())
    _log(f"built {lib} in {time.time() - t0:.0f}s")
    return lib


def _filter(stderr: str) -> str:
    return "\n".join(l for l in stderr.splitlines() if "packed-fp32-ops" not in l)


def ensure_built() -> str:
    """The path of a library that matches the sources; builds it if there is none."""
    lib = library_path()
    if is_current(lib):
        return lib
    if os.path.isfile(lib) and find_hipcc() is None:
        _log(f"warning: {lib} is older than its sources and hipcc is not there to rebuild it")
        return lib
    return build(force=True)
