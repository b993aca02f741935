"""Reader and writer of the safetensors container, from its public layout.

Layout: 8 bytes little-endian header length n, n bytes of JSON
`{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}`,
then the raw little-endian data.  The reader maps the file and hands out tensors by
name without copying; a folder may hold one `model.safetensors` or several shards
named by `model.safetensors.index.json` (crates/synaptix-models/llm/qwen3/src/loader.rs:87-115
of the reference resolves shards the same way).
"""
from __future__ import annotations

import json
import mmap
import os
import struct

import torch


class SafetensorsError(ValueError):
    pass


_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    """One mapped file: `names()`, `info(name)`, `tensor(name)`."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._f = open(path, "rb")
        except OSError as e:
            raise SafetensorsError(f"open {path}: {e}") from None
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: shorter than a header")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n > size - 8:
            raise SafetensorsError(f"{path}: header length {n} exceeds the file")
        try:
            header = json.loads(self._f.read(n))
        except json.JSONDecodeError as e:
            raise SafetensorsError(f"{path}: header is not JSON: {e}") from None
        self.metadata = header.pop("__metadata__", {}) or {}
        self._entries = header
        self._base = 8 + n
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size else None
        for name, e in header.items():
            b, en = e["data_offsets"]
            if not (0 <= b <= en <= size - self._base):
                raise SafetensorsError(f"{path}: tensor {name!r} lies outside the file")

    def names(self):
        return list(self._entries)

    def info(self, name: str):
        e = self._entries[name]
        return e["dtype"], tuple(e["shape"])

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that aliases the mapped file (read-only: copy before writing)."""
        if name not in self._entries:
            raise SafetensorsError(f"tensor not found: {name}")
        e = self._entries[name]
        if e["dtype"] not in _DTYPES:
            raise SafetensorsError(f"{self.path}: tensor {name!r}: unsupported dtype {e['dtype']}")
        dtype = _DTYPES[e["dtype"]]
        shape = tuple(e["shape"])
        b, en = e["data_offsets"]
        count = 1
        for s in shape:
            count *= s
        if (en - b) != count * torch.empty(0, dtype=dtype).element_size():
            raise SafetensorsError(f"{self.path}: tensor {name!r}: {en - b} bytes do not fill shape {shape}")
        if count == 0:
            return torch.empty(shape, dtype=dtype)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the map is read-only; tensors from it are never written
            t = torch.frombuffer(self._map, dtype=dtype, count=count, offset=self._base + b)
        return t.view(shape)


def resolve_shards(folder: str) -> list:
    single = os.path.join(folder, "model.safetensors")
    if os.path.isfile(single):
        return [single]
    index = os.path.join(folder, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index) as f:
            wm = json.load(f).get("weight_map", {})
        return [os.path.join(folder, n) for n in sorted(set(wm.values()))]
    raise SafetensorsError(f"no model.safetensors and no model.safetensors.index.json in {folder}")


def save_file(tensors: dict, path: str, metadata: dict | None = None) -> None:
    """Write `tensors` (name -> CPU tensor) as one safetensors file."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors)
    blobs = []
    for name in order:
        t = tensors[name].detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        blobs.append(t)
    raw = json.dumps(header, separators=(",", ":")).encode()
    raw += b" " * ((8 - len(raw) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(raw)))
        f.write(raw)
        for t in blobs:
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dtype != torch.bool
                        else t.to(torch.uint8).numpy().tobytes())
