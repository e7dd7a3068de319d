"""Reading and writing the safetensors container: an 8-byte little-endian header
length, a JSON header {name: {dtype, shape, data_offsets}}, then raw little-endian
data.  The reference maps the file into memory and converts tensor by tensor
(crates/denno-engine/src/load.rs:27-58, 81-147); so does this reader, so a large model
never lies in host memory twice.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
import warnings
from typing import Dict, Iterable, Tuple

import torch

_DTYPES = {
    "F32": (torch.float32, 4), "BF16": (torch.bfloat16, 2), "F16": (torch.float16, 2),
    "F64": (torch.float64, 8), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One mapped file.  `entries[name] = (dtype string, shape tuple)`; `tensor(name)` is a
    CPU tensor that views the mapping (read-only: copy or convert before writing)."""

    def __init__(self, path: str):
        self.path = path
        self._f = open(path, "rb")
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short for a safetensors file")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n > size - 8:
            raise SafetensorsError(f"{path}: header length {n} exceeds the file")
        try:
            header = json.loads(self._f.read(n).decode("utf-8"))
        except Exception as e:
            raise SafetensorsError(f"{path}: header is not JSON: {e}") from None
        self.metadata = header.pop("__metadata__", {})
        self._base = 8 + n
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        self.entries: Dict[str, Tuple[str, Tuple[int, ...]]] = {}
        self._offsets = {}
        for name, e in header.items():
            dt, shape = e["dtype"], tuple(e["shape"])
            b, end = e["data_offsets"]
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor '{name}' has unsupported dtype {dt}")
            numel = 1
            for s in shape:
                numel *= s
            if end - b != numel * _DTYPES[dt][1] or self._base + end > size:
                raise SafetensorsError(
                    f"{path}: tensor '{name}' {dt}{list(shape)} does not match its {end - b} bytes")
            self.entries[name] = (dt, shape)
            self._offsets[name] = (b, end)

    def tensor(self, name: str) -> torch.Tensor:
        dt, shape = self.entries[name]
        b, end = self._offsets[name]
        if end == b:
            return torch.empty(shape, dtype=_DTYPES[dt][0])
        buf = memoryview(self._mm)[self._base + b:self._base + end]
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)   # the mapping is read-only; callers copy
            return torch.frombuffer(buf, dtype=_DTYPES[dt][0]).reshape(shape)

    def close(self):
        # tensors handed out view the mapping; they must be dropped first
        try:
            self._mm.close()
        except BufferError:
            pass
        self._f.close()


def open_checkpoint(model_dir: str):
    """-> ({name: SafetensorsFile}, [files]) for `model.safetensors`, or for every shard
    that `model.safetensors.index.json` lists (crates/denno-engine/src/load.rs:81-125)."""
    single = os.path.join(model_dir, "model.safetensors")
    index = os.path.join(model_dir, "model.safetensors.index.json")
    files, where = [], {}
    if os.path.isfile(single):
        paths = [single]
    elif os.path.isfile(index):
        with open(index) as f:
            wm = json.load(f).get("weight_map")
        if not isinstance(wm, dict) or not wm:
            raise SafetensorsError(f"{index}: no 'weight_map', or an empty one")
        paths = [os.path.join(model_dir, p) for p in sorted(set(wm.values()))]
    else:
        raise SafetensorsError(f"{model_dir}: neither model.safetensors nor model.safetensors.index.json")
    for p in paths:
        sf = SafetensorsFile(p)
        files.append(sf)
        for name in sf.entries:
            where[name] = sf
    return where, files


def write_safetensors(path: str, layout: Iterable[Tuple[str, torch.dtype, Tuple[int, ...]]],
                      produce, metadata=None):
    """Writes tensors one at a time: `layout` gives (name, dtype, shape) in file order,
    `produce(name)` returns that tensor when its turn comes."""
    layout = list(layout)
    header, off = {}, 0
    for name, dtype, shape in layout:
        numel = 1
        for s in shape:
            numel *= s
        nbytes = numel * _DTYPES[_NAMES[dtype]][1]
        header[name] = {"dtype": _NAMES[dtype], "shape": list(shape), "data_offsets": [off, off + nbytes]}
        off += nbytes
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * ((8 - len(raw) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(raw)))
        f.write(raw)
        for name, dtype, shape in layout:
            t = produce(name)
            if t.dtype != dtype or tuple(t.shape) != tuple(shape):
                raise SafetensorsError(f"'{name}': produced {t.dtype}{list(t.shape)}, "
                                       f"layout says {dtype}{list(shape)}")
            t = t.contiguous().cpu()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
