"""Reading and writing safetensors files without executing anything from them.

Format: 8 bytes little-endian header length N, N bytes of JSON
``{name: {"dtype": "BF16", "shape": [...], "data_offsets": [begin, end]}, "__metadata__": {...}}``,
then the raw little-endian tensor bytes. The reference reads the same files through the
safetensors package (src/levanter/compat/hf_checkpoints.py:209-217) and looks for an index
of shards first (hf_checkpoints.py:507-513,531-561).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import torch

_DTYPES = {
    "F64": torch.float64,
    "F32": torch.float32,
    "F16": torch.float16,
    "BF16": torch.bfloat16,
    "I64": torch.int64,
    "I32": torch.int32,
    "I16": torch.int16,
    "I8": torch.int8,
    "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One memory-mapped file. ``keys()``, ``info(name)`` and ``tensor(name)``; tensors are
    views into the mapping and must be copied (``.clone()``, ``.to(device)``) before ``close``."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: truncated file ({size} bytes, no header length)")
        self._f = open(path, "rb")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n <= 0 or 8 + n > size:
            raise SafetensorsError(f"{path}: truncated file (header of {n} bytes does not fit in {size})")
        try:
            header = json.loads(self._f.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON: {e}") from None
        self.metadata = header.pop("__metadata__", {}) or {}
        self._entries: Dict[str, dict] = header
        self._base = 8 + n
        data_len = size - self._base
        for name, e in header.items():
            if e.get("dtype") not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {e.get('dtype')!r}")
            b, en = e["data_offsets"]
            want = _numel(e["shape"]) * _DTYPES[e["dtype"]].itemsize
            if en - b != want:
                raise SafetensorsError(f"{path}: tensor {name!r} spans {en - b} bytes, its shape and dtype need {want}")
            if b < 0 or en > data_len:
                raise SafetensorsError(f"{path}: truncated file (tensor {name!r} ends at byte {en} of {data_len})")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def keys(self) -> List[str]:
        return list(self._entries)

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        e = self._entries[name]
        return _DTYPES[e["dtype"]], tuple(e["shape"])

    def tensor(self, name: str) -> torch.Tensor:
        e = self._entries[name]
        dtype = _DTYPES[e["dtype"]]
        b, en = e["data_offsets"]
        count = _numel(e["shape"])
        if count == 0:
            return torch.empty(tuple(e["shape"]), dtype=dtype)
        import warnings

        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the mapping is read-only; nobody writes through the view
            t = torch.frombuffer(self._mm, dtype=dtype, count=count, offset=self._base + b)
        return t.reshape(tuple(e["shape"]))

    def close(self) -> None:
        # tensors made by ``tensor`` keep the mapping alive through the buffer protocol; dropping
        # our handles is enough
        self._mm = None
        self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def _numel(shape: Iterable[int]) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n


def open_model_files(model_dir: str) -> List[SafetensorsFile]:
    """The safetensors files of a model folder: the shards an index names, else model.safetensors."""
    index = os.path.join(model_dir, "model.safetensors.index.json")
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.isfile(index):
        with open(index) as f:
            weight_map = json.load(f).get("weight_map", {})
        shards = sorted(set(weight_map.values()))
        missing = [s for s in shards if not os.path.isfile(os.path.join(model_dir, s))]
        if missing:
            raise FileNotFoundError(f"{model_dir}: the index names shards that are not there: {', '.join(missing)}")
        return [SafetensorsFile(os.path.join(model_dir, s)) for s in shards]
    if os.path.isfile(single):
        return [SafetensorsFile(single)]
    raise FileNotFoundError(f"{model_dir}: neither model.safetensors nor model.safetensors.index.json found")


def save_file(tensors: Dict[str, torch.Tensor], path: str, metadata: Dict[str, str] | None = None) -> None:
    """Write tensors (on the CPU) to one safetensors file, in the order of the dict."""
    header: Dict[str, dict] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    for name, t in tensors.items():
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, t in tensors.items():
            c = t.detach().contiguous().cpu()
            if c.numel():
                f.write(c.view(torch.uint8).numpy().tobytes() if c.dim() else c.reshape(1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
