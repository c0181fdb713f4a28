"""Minimal safetensors reader and writer.

File layout: 8 bytes little-endian header length, a JSON header mapping each tensor
name to {"dtype", "shape", "data_offsets": [begin, end)} relative to the end of the
header, then the raw little-endian data.  The reader memory-maps the file, as the
reference does for all shards (/root/reference/src/models/layers/mod.rs:129-135).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch

_NP = {
    "F64": (np.float64, torch.float64), "F32": (np.float32, torch.float32),
    "F16": (np.float16, torch.float16), "BF16": (np.uint16, torch.bfloat16),
    "I64": (np.int64, torch.int64), "I32": (np.int32, torch.int32),
    "I16": (np.int16, torch.int16), "I8": (np.int8, torch.int8),
    "U8": (np.uint8, torch.uint8), "BOOL": (np.bool_, torch.bool),
}
_TAG = {torch.float64: "F64", torch.float32: "F32", torch.float16: "F16",
        torch.bfloat16: "BF16", torch.int64: "I64", torch.int32: "I32",
        torch.int16: "I16", torch.int8: "I8", torch.uint8: "U8", torch.bool: "BOOL"}


class SafetensorsFile:
    """One memory-mapped .safetensors file."""

    def __init__(self, path: str):
        self.path = path
        self._f = open(path, "rb")
        head = self._f.read(8)
        if len(head) != 8:
            raise ValueError(f"{path}: too short to be a safetensors file")
        (n,) = struct.unpack("<Q", head)
        size = os.fstat(self._f.fileno()).st_size
        if n <= 0 or 8 + n > size:
            raise ValueError(f"{path}: bad safetensors header length {n}")
        try:
            header = json.loads(self._f.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise ValueError(f"{path}: safetensors header is not JSON ({e})") from e
        header.pop("__metadata__", None)
        self._base = 8 + n
        self.entries: Dict[str, dict] = header
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        for name, e in header.items():
            b, end = e["data_offsets"]
            if e["dtype"] not in _NP:
                raise ValueError(f"{path}: tensor {name!r} has unsupported dtype {e['dtype']}")
            if self._base + end > size or b > end:
                raise ValueError(f"{path}: tensor {name!r} lies outside the file")

    def names(self) -> List[str]:
        return list(self.entries)

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self.entries[name]["shape"])

    def dtype(self, name: str) -> torch.dtype:
        return _NP[self.entries[name]["dtype"]][1]

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapped file (read-only memory: copy before writing)."""
        e = self.entries[name]
        np_t, torch_t = _NP[e["dtype"]]
        b, end = e["data_offsets"]
        shape = tuple(e["shape"])
        count = int(np.prod(shape, dtype=np.int64)) if shape else 1
        if (end - b) != count * np.dtype(np_t).itemsize:
            raise ValueError(f"{self.path}: tensor {name!r}: byte length does not match its shape")
        arr = np.frombuffer(self._mm, dtype=np_t, count=count, offset=self._base + b)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")          # read-only buffer; never written through
            t = torch.from_numpy(arr)
        if torch_t is torch.bfloat16:
            t = t.view(torch.bfloat16)
        return t.reshape(shape)

    def close(self) -> None:
        try:
            self._mm.close()
        except (BufferError, ValueError):
            pass                                      # tensors still view the map
        self._f.close()


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]]) -> None:
    """Write tensors in the order given.  `tensors` may be a generator, so that a large
    model is written one tensor at a time; the header needs shapes first, so the data is
    streamed to a temporary file beside the target and then joined."""
    tmp = path + ".data.tmp"
    header: Dict[str, dict] = {}
    offset = 0
    with open(tmp, "wb") as data:
        for name, t in tensors:
            if name in header:
                raise ValueError(f"duplicate tensor name {name!r}")
            t = t.detach().to("cpu").contiguous()
            if t.dtype not in _TAG:
                raise ValueError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
            raw = t.view(torch.int16).numpy() if t.dtype is torch.bfloat16 else t.numpy()
            buf = raw.tobytes()
            header[name] = {"dtype": _TAG[t.dtype], "shape": list(t.shape),
                            "data_offsets": [offset, offset + len(buf)]}
            data.write(buf)
            offset += len(buf)
    hb = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hb += b" " * ((8 - len(hb) % 8) % 8)
    with open(path, "wb") as out, open(tmp, "rb") as data:
        out.write(struct.pack("<Q", len(hb)))
        out.write(hb)
        while True:
            chunk = data.read(1 << 24)
            if not chunk:
                break
            out.write(chunk)
    os.remove(tmp)
