"""Reading and writing the safetensors container: 8 bytes little-endian header
length, a JSON header (name -> dtype, shape, data_offsets), then raw
little-endian data.  Tensors are memory-mapped and copied one at a time, so a
model never has to fit into host memory."""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Iterable

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    def __init__(self, path: str) -> None:
        self.path = path
        self._f = open(path, "rb")
        (n,) = struct.unpack("<Q", self._f.read(8))
        header = json.loads(self._f.read(n).decode("utf-8"))
        self.metadata = header.pop("__metadata__", None)
        self.entries = header
        self._base = 8 + n
        self._mm = None

    def names(self) -> list[str]:
        return list(self.entries)

    def shape(self, name: str) -> tuple[int, ...]:
        return tuple(self.entries[name]["shape"])

    def dtype(self, name: str) -> torch.dtype:
        code = self.entries[name]["dtype"]
        if code not in _DTYPES:
            raise ValueError(f"{self.path}: tensor {name!r} has unsupported dtype {code}")
        return _DTYPES[code]

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapped file (read-only: copy before writing)."""
        if self._mm is None:
            self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        e = self.entries[name]
        a, b = e["data_offsets"]
        dt = self.dtype(name)
        shape = tuple(e["shape"])
        count = 1
        for d in shape:
            count *= d
        if count == 0:
            return torch.empty(shape, dtype=dt)
        import warnings

        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the buffer is read-only; it is only ever copied from
            t = torch.frombuffer(self._mm, dtype=dt, count=count, offset=self._base + a)
        assert (b - a) == count * t.element_size(), f"{self.path}: {name!r} has inconsistent offsets"
        return t.reshape(shape)

    def close(self) -> None:
        self._mm = None
        self._f.close()


def write_safetensors(path: str, tensors: Iterable[tuple[str, torch.Tensor]], specs: list[tuple[str, torch.dtype, tuple]]):
    """Writes tensors in the order of ``specs`` (name, dtype, shape); ``tensors``
    yields them in the same order, one at a time, so that only one is in memory."""
    header = {}
    off = 0
    for name, dt, shape in specs:
        n = torch.empty((), dtype=dt).element_size()
        for d in shape:
            n *= d
        header[name] = {"dtype": _NAMES[dt], "shape": list(shape), "data_offsets": [off, off + n]}
        off += n
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * ((8 - len(raw) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(raw)))
        f.write(raw)
        for (name, t), (sname, dt, shape) in zip(tensors, specs):
            assert name == sname and t.dtype == dt and tuple(t.shape) == tuple(shape), (name, sname)
            t = t.contiguous().cpu()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)
