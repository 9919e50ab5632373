"""Compiles the HIP sources under ``csrc/`` into shared libraries for gfx950, one per unit:

* ``core``: errors, embedding / norms / KV write / sampling, the 32-bit GEMM and attention;
* ``gemm_mfma``: the bfloat16 GEMMs on the matrix cores;
* ``gemm_library``: the vendor library's GEMM (hipBLASLt) for prompt-sized row counts, where it is ahead;
* ``attn_hd<N>``: the bfloat16 attention on the matrix cores for head size N (16 .. 128 in steps of 16).

A model loads ``core`` and, in bfloat16, ``gemm_mfma`` and the attention unit of its own head size, so a first
call in a fresh checkout compiles what that model needs. The libraries are built in the tree
(``levanter_amd/kernels/``); when the tree cannot be written, in a per-user folder under the temporary
directory. A build compiles its sources in parallel and prints a line per file. ``ensure_built`` builds a
unit only when it has no library or the sources changed; ``build`` builds every unit.
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
from typing import Dict, Iterable, List, Optional, Tuple

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(_HERE), "csrc")
ARCH = "gfx950"

MFMA_ATTENTION_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128)

# unit -> [(source, extra defines, object name)]
UNITS: Dict[str, List[Tuple[str, List[str], str]]] = {
    "core": [
        ("errors.hip", [], "errors.o"),
        ("elementwise.hip", [], "elementwise.o"),
        ("gemm_simple.hip", [], "gemm_simple.o"),
        ("attention_simple.hip", [], "attention_simple.o"),
        ("attention_common.hip", [], "attention_common.o"),
    ],
    "gemm_mfma": [("gemm_mfma.hip", [], "gemm_mfma.o")],
    "gemm_library": [("gemm_library.hip", [], "gemm_library.o")],
}
# libraries a unit is linked against
UNIT_LINK_FLAGS: Dict[str, List[str]] = {"gemm_library": ["-lhipblaslt"]}
for _hd in MFMA_ATTENTION_HEAD_DIMS:
    UNITS[f"attn_hd{_hd}"] = [
        ("attention_mfma.hip", [f"-DLEV_HD={_hd}"], f"attention_mfma_hd{_hd}.o"),
        ("attention_dispatch.hip", [f"-DLEV_HD={_hd}"], f"attention_dispatch_hd{_hd}.o"),
    ]


def attention_unit(head_dim: int) -> str:
    return f"attn_hd{head_dim}"


def lib_name(unit: str) -> str:
    return f"liblevanter_amd_{unit}.so"


# -packed-fp32-ops off: no packed 32-bit float instructions (v_pk_*_f32) are generated; some forms have given wrong results on MI355X
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


def _with_includes(names: Iterable[str]) -> List[str]:
    """The given sources and every file of ``csrc/`` that they include with ``#include "..."``, directly or not."""
    seen, todo = set(), list(names)
    while todo:
        name = todo.pop()
        if name in seen:
            continue
        seen.add(name)
        with open(os.path.join(CSRC, name), encoding="utf-8") as f:
            for line in f:
                line = line.strip()
                if line.startswith("#include \""):
                    inc = line.split('"')[1]
                    if os.path.isfile(os.path.join(CSRC, inc)):
                        todo.append(inc)
    return sorted(seen)


def source_hash(unit: str = "core") -> str:
    """Hash of what a unit is built from: the flags, its own sources and defines, and the headers they include."""
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    names = _with_includes(src for src, _, _ in UNITS[unit])
    for name in names:
        h.update(name.encode())
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    for _, defines, obj in UNITS[unit]:
        h.update((" ".join(defines) + obj).encode())
    h.update(" ".join(UNIT_LINK_FLAGS.get(unit, [])).encode())
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


def library_path(unit: str = "core") -> str:
    return os.path.join(library_dir(), lib_name(unit))


def _stamp_path(lib: str) -> str:
    return lib + ".hash"


def is_current(unit: str = "core") -> bool:
    lib = library_path(unit)
    try:
        with open(_stamp_path(lib)) as f:
            return os.path.isfile(lib) and f.read().strip() == source_hash(unit)
    except OSError:
        return False


def build(force: bool = True, jobs: Optional[int] = None, units: Optional[Iterable[str]] = None) -> Dict[str, str]:
    """Compile and link the given units (all of them by default). Returns unit -> library path."""
    hipcc = find_hipcc()
    if hipcc is None:
        raise RuntimeError("hipcc not found: the HIP libraries of levanter_amd cannot be built (set HIPCC or install ROCm)")
    wanted = list(UNITS) if units is None else list(units)
    for u in wanted:
        if u not in UNITS:
            raise RuntimeError(f"unknown kernel unit {u!r}; known: {', '.join(UNITS)}")
    todo = [u for u in wanted if force or not is_current(u)]
    paths = {u: library_path(u) for u in wanted}
    if not todo:
        return paths
    obj_dir = os.path.join(library_dir(), "_build")
    os.makedirs(obj_dir, exist_ok=True)
    items = [item for u in todo for item in UNITS[u]]
    jobs = jobs or min(8, os.cpu_count() or 1, len(items))
    env = dict(os.environ)
    home = env.get("HOME", "")
    if not home or not os.path.isdir(home) or not os.access(home, os.W_OK):
        env["HOME"] = tempfile.gettempdir()  # hipcc wants a HOME it can write its caches to
    t0 = time.time()
    _log(f"compiling {len(items)} HIP objects ({', '.join(todo)}) for {ARCH} with {jobs} jobs ...")

    def compile_one(item) -> None:
        src, defines, obj_name = item
        obj = os.path.join(obj_dir, obj_name)
        cmd = [hipcc, *HIPCC_FLAGS, *defines, "-c", os.path.join(CSRC, src), "-o", obj]
        t = time.time()
        r = subprocess.run(cmd, capture_output=True, text=True, env=env)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src} {' '.join(defines)}:\n{_filter(r.stderr)}")
        _log(f"  {obj_name[:-2]} done in {time.time() - t:.0f}s")

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, items))
    for u in todo:
        lib = paths[u]
        objs = [os.path.join(obj_dir, obj_name) for _, _, obj_name in UNITS[u]]
        tmp = lib + f".tmp{os.getpid()}"
        r = subprocess.run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs, *UNIT_LINK_FLAGS.get(u, [])],
                           capture_output=True, text=True, env=env)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed to link {lib_name(u)}:\n{_filter(r.stderr)}")
        os.replace(tmp, lib)
        with open(_stamp_path(lib), "w") as f:
            f.write(source_hash(u))
    _log(f"built {', '.join(lib_name(u) for u in todo)} in {library_dir()} in {time.time() - t0:.0f}s")
    return paths


def _filter(stderr: str) -> str:
    return "\n".join(l for l in stderr.splitlines() if "packed-fp32-ops" not in l)


def ensure_built(unit: str = "core") -> str:
    """The path of a library of this unit that matches the sources; builds it if there is none."""
    lib = library_path(unit)
    if is_current(unit):
        return lib
    if os.path.isfile(lib) and find_hipcc() is None:
        _log(f"warning: {lib} is older than its sources and hipcc is not there to rebuild it")
        return lib
    return build(force=True, units=[unit])[unit]
