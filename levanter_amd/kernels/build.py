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

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from dataclasses import dataclass, field
from typing import Dict, Iterable, List, Optional, Tuple

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(_HERE), "csrc")
ARCH = "gfx950"

MFMA_ATTENTION_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128)


@dataclass
class KernelUnit:
    """One shared library: its sources, how they are compiled and linked, and the ``extern "C"`` entry points it offers.

    ``sources``: (file, extra defines, object name); a relative file lies in ``source_dir``. Sources may include the
    headers of ``csrc/`` (``common.h``: the error functions, dtype tags, reductions) wherever they lie themselves.
    ``signatures``: entry point -> ctypes argument types; the result is an int (0, or a negative code with a message in
    ``lev_last_error()``) unless the name ends in ``_workspace`` (a byte count). ``HipKernels`` sets them when it
    loads the library."""

    name: str
    sources: List[Tuple[str, List[str], str]]
    source_dir: str = CSRC
    link_flags: List[str] = field(default_factory=list)
    signatures: Dict[str, list] = field(default_factory=dict)

    def source_path(self, src: str) -> str:
        return src if os.path.isabs(src) else os.path.join(self.source_dir, src)


UNITS: Dict[str, KernelUnit] = {}


def register_unit(name: str, sources, *, source_dir: str = CSRC, link_flags: Iterable[str] = (), signatures: Optional[Dict[str, list]] = None,
                  replace: bool = False) -> KernelUnit:
    """Make a kernel library known: ``ensure_built(name)`` compiles it when it is missing or stale and
    ``HipKernels.call(name, entry, ...)`` loads it at its first use. A part that brings a kernel of its own registers a unit
    for it from its own module (its ``.hip`` may lie anywhere); nothing in this package has to change.
    ``sources``: file names, or (file, defines, object name) where one file is compiled several ways."""
    if name in UNITS and not replace:
        raise ValueError(f"kernel unit {name!r} is already registered")
    items = []
    for src in sources:
        if isinstance(src, str):
            src = (src, [], os.path.splitext(os.path.basename(src))[0] + ".o")
        items.append((src[0], list(src[1]), src[2]))
    unit = KernelUnit(name, items, source_dir, list(link_flags), dict(signatures or {}))
    UNITS[name] = unit
    return unit


def unregister_unit(name: str) -> None:
    UNITS.pop(name, None)


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


def _with_includes(unit: KernelUnit) -> List[str]:
    """The unit's sources and every file that they include with ``#include "..."``, directly or not: looked up beside the
    including file and in ``csrc/`` (the include path of every compilation)."""
    seen, todo = set(), [unit.source_path(src) for src, _, _ in unit.sources]
    while todo:
        path = todo.pop()
        if path in seen:
            continue
        seen.add(path)
        with open(path, encoding="utf-8") as f:
            for line in f:
                line = line.strip()
                if line.startswith("#include \""):
                    inc = line.split('"')[1]
                    for base in (os.path.dirname(path), CSRC):
                        if os.path.isfile(os.path.join(base, inc)):
                            todo.append(os.path.join(base, inc))
                            break
    return sorted(seen)


def source_hash(unit: str = "core") -> str:
    """Hash of what a unit is built from: the flags, its own sources and defines, and the headers they include."""
    u = UNITS[unit]
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    for path in _with_includes(u):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    for _, defines, obj in u.sources:
        h.update((" ".join(defines) + obj).encode())
    h.update(" ".join(u.link_flags).encode())
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
    items = [(UNITS[u], item) for u in todo for item in UNITS[u].sources]
    jobs = jobs or min(8, os.cpu_count() or 1, len(items))
    env = dict(os.environ)
    home = env.get("HOME", "")
    if not home or not os.path.isdir(home) or not os.access(home, os.W_OK):
        env["HOME"] = tempfile.gettempdir()  # hipcc wants a HOME it can write its caches to
    t0 = time.time()
    _log(f"compiling {len(items)} HIP objects ({', '.join(todo)}) for {ARCH} with {jobs} jobs ...")

    def compile_one(unit_item) -> None:
        unit, (src, defines, obj_name) = unit_item
        obj = os.path.join(obj_dir, _object_name(unit, obj_name))
        cmd = [hipcc, *HIPCC_FLAGS, f"-I{CSRC}", *defines, "-c", unit.source_path(src), "-o", obj]
        t = time.time()
        r = subprocess.run(cmd, capture_output=True, text=True, env=env)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src} {' '.join(defines)}:\n{_filter(r.stderr)}")
        _log(f"  {obj_name[:-2]} done in {time.time() - t:.0f}s")

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, items))
    for u in todo:
        lib = paths[u]
        objs = [os.path.join(obj_dir, _object_name(UNITS[u], obj_name)) for _, _, obj_name in UNITS[u].sources]
        tmp = lib + f".tmp{os.getpid()}"
        r = subprocess.run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs, *UNITS[u].link_flags],
                           capture_output=True, text=True, env=env)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed to link {lib_name(u)}:\n{_filter(r.stderr)}")
        os.replace(tmp, lib)
        with open(_stamp_path(lib), "w") as f:
            f.write(source_hash(u))
    _log(f"built {', '.join(lib_name(u) for u in todo)} in {library_dir()} in {time.time() - t0:.0f}s")
    return paths


def _object_name(unit: KernelUnit, obj_name: str) -> str:
    """Objects of units outside ``csrc/`` carry the unit's name: two units may both have a ``kernel.o``."""
    return obj_name if unit.source_dir == CSRC else f"{unit.name}__{obj_name}"


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


# ---- the units of this package --------------------------------------------------------------------------------
_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float

register_unit("core", ["errors.hip", "elementwise.hip", "gemm_simple.hip", "attention_simple.hip", "attention_common.hip"], signatures={
    "lev_embed": [_P] * 5 + [_I, _I, _I, _P],
    "lev_norm": [_P] * 5 + [_I, _I, _F, _I, _I, _P],
    "lev_norm_pending": [_P, _P, _I] + [_P] * 5 + [_I, _I, _I, _F, _I, _I, _P],
    "lev_kv_write": [_P, _P, _L, _L, _P, _P, _P] + [_I] * 5 + [_P],
    "lev_sample": [_P, _L, _P, _P, _P, _P, _P, _P, _I, _I, _P],
    "lev_sample_workspace": [_I],
    "lev_feed_tokens": [_P, _P, _P, _I, _P],
    "lev_linear_simple": [_P, _L, _P, _P, _P, _L, _P, _L] + [_I] * 6 + [_P],
    "lev_attention_simple": [_P, _L, _P, _L, _P, _P, _P, _P, _P] + [_I] * 6 + [_F, _I, _I, _F, _P, _I, _P],
    "lev_attention_mfma_workspace": [_I] * 5,
})
register_unit("gemm_mfma", ["gemm_mfma.hip"], signatures={
    "lev_linear_mfma": [_P, _L, _P, _P, _P, _L, _P, _L, _P] + [_I] * 6 + [_P],
    "lev_linear_mfma_workspace": [_I, _I, _I],
    "lev_linear_mfma_ranges": [_I, _I, _I],
    "lev_linear_mfma_force": [_I],
    "lev_linear_mfma_finish": [_P, _P, _P, _L, _P, _L] + [_I] * 5 + [_P],
})
# the vendor library's GEMM (hipBLASLt) behind the same interface
register_unit("gemm_library", ["gemm_library.hip"], link_flags=["-lhipblaslt"], signatures={
    "lev_linear_library": [_P, _L, _P, _P, _P, _L, _P, _L, _P, _L] + [_I] * 5 + [_P],
    "lev_linear_library_workspace": [],
})
for _hd in MFMA_ATTENTION_HEAD_DIMS:
    register_unit(attention_unit(_hd), [("attention_mfma.hip", [f"-DLEV_HD={_hd}"], f"attention_mfma_hd{_hd}.o"),
                                        ("attention_dispatch.hip", [f"-DLEV_HD={_hd}"], f"attention_dispatch_hd{_hd}.o")], signatures={
        "lev_attention_mfma": [_P, _L, _P, _L, _P, _P, _P, _P, _P, _I, _P, _I, _P, _I, _P, _P, _L, _P, _P] + [_I] * 5 + [_F, _I, _F, _P, _I, _P],
    })
