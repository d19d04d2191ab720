"""Reading and writing the safetensors container: an 8-byte little-endian header length,
a JSON header {name: {dtype, shape, data_offsets}}, then the raw bytes.  Tensors are
read by name from a memory map; nothing in the file is executed.  It stands where the
reference has its GGUF parser with bounds-checked tensor data (include/gguf.h:120-134,
src/gguf.c): every offset is checked against the file before it is used.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, Tuple

import torch

_DTYPES = {
    "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16, "F64": torch.float64,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One .safetensors file, memory-mapped; `entries` maps a name to (dtype, shape)."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        self._f = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen <= 0 or 8 + hlen > size:
            raise SafetensorsError(f"{path}: header length {hlen} exceeds the file ({size} bytes)")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: the header is not JSON ({e})") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: the header is not a JSON object")
        self._base = 8 + hlen
        self._data_len = size - self._base
        # private (copy-on-write) rather than read-only: nothing writes to it, and a tensor can share its memory
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_COPY) if size else None
        self.entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...]]] = {}
        self._spans = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            try:
                dt = _DTYPES[info["dtype"]]
                shape = tuple(int(s) for s in info["shape"])
                a, b = (int(v) for v in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: malformed entry for tensor {name!r}") from None
            n = 1
            for s in shape:
                if s < 0:
                    raise SafetensorsError(f"{path}: tensor {name!r} has a negative dimension")
                n *= s
            nbytes = n * torch.empty((), dtype=dt).element_size()
            if a < 0 or b < a or b > self._data_len or b - a != nbytes:
                raise SafetensorsError(f"{path}: tensor {name!r} has data offsets [{a}, {b}) that do not fit "
                                       f"its shape {shape} / the file")
            self.entries[name] = (dt, shape)
            self._spans[name] = (a, b)

    def names(self) -> Iterable[str]:
        return self.entries.keys()

    def read(self, name: str) -> torch.Tensor:
        """A tensor that owns its memory (copied out of the map)."""
        dt, shape = self.entries[name]
        a, b = self._spans[name]
        if a == b:
            return torch.empty(shape, dtype=dt)
        owned = bytearray(self._mm[self._base + a:self._base + b])     # one copy out of the map
        return torch.frombuffer(owned, dtype=dt).reshape(shape)

    def view(self, name: str) -> torch.Tensor:
        """The tensor as it lies in the map: no copy, no memory of its own (the reference maps its file the same way
        and points its tensors into it, src/model.c:147).  The pages come in when they are touched; release()
        lets them go again.  Not to be written to; it keeps the map alive for as long as it lives."""
        dt, shape = self.entries[name]
        a, b = self._spans[name]
        if a == b:
            return torch.empty(shape, dtype=dt)
        if (self._base + a) % torch.empty((), dtype=dt).element_size():
            return self.read(name)                          # not aligned for its type in the file: a copy is
        return torch.frombuffer(self._mm, dtype=dt, count=(b - a) // torch.empty((), dtype=dt).element_size(),
                                offset=self._base + a).reshape(shape)

    def release(self, name: str) -> None:
        """Tells the system that the tensor's pages are not needed any more (they are read again from the file
        if they are): what was touched of it stops counting as this process's memory."""
        a, b = self._spans[name]
        ps = mmap.PAGESIZE
        lo = -(-(self._base + a) // ps) * ps               # whole pages inside the span only: neighbours may be in use
        hi = (self._base + b) // ps * ps
        if hi > lo and self._mm is not None and hasattr(self._mm, "madvise"):
            try:
                self._mm.madvise(mmap.MADV_DONTNEED, lo, hi - lo)
            except (OSError, ValueError, AttributeError):
                pass                                        # advice only

    def close(self) -> None:
        # The map is not unmapped here but when nothing refers to it any more: a tensor from view() shares its memory
        # and holds a reference to it, and unmapping under such a tensor would leave it pointing nowhere.
        self._mm = None
        self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def open_model_files(folder: str):
    """The safetensors files of a model folder: model.safetensors, or the shards that
    model.safetensors.index.json names."""
    single = os.path.join(folder, "model.safetensors")
    index = os.path.join(folder, "model.safetensors.index.json")
    if os.path.isfile(single):
        return [SafetensorsFile(single)]
    if os.path.isfile(index):
        with open(index) as f:
            idx = json.load(f)
        shards = sorted(set(idx.get("weight_map", {}).values()))
        if not shards:
            raise SafetensorsError(f"{index}: no weight_map")
        return [SafetensorsFile(os.path.join(folder, s)) for s in shards]
    raise SafetensorsError(f"{folder}: neither model.safetensors nor model.safetensors.index.json")


def write_file(path: str, tensors: Dict[str, torch.Tensor], metadata: dict | None = None) -> None:
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + n]}
        off += n
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)
