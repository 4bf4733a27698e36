"""Reader for safetensors files: an 8-byte little-endian header length, that many bytes of JSON (name -> dtype, shape, data_offsets),
then the tensors' bytes.  Nothing in the file is executed; tensors are memory-mapped and handed out as numpy views."""
from __future__ import annotations

import json
import struct

import numpy as np

_DTYPES = {"BF16": np.uint16, "F16": np.float16, "F32": np.float32, "F64": np.float64, "I32": np.int32, "I64": np.int64, "U8": np.uint8}


class SafeTensors:
    def __init__(self, path: str):
        self.path = path
        with open(path, "rb") as f:
            head = f.read(8)
            if len(head) != 8:
                raise ValueError(f"{path}: not a safetensors file")
            (n,) = struct.unpack("<Q", head)
            meta = json.loads(f.read(n).decode("utf-8"))
        self.base = 8 + n
        self.meta = {k: v for k, v in meta.items() if k != "__metadata__"}
        self._map = np.memmap(path, dtype=np.uint8, mode="r")

    def names(self):
        return list(self.meta)

    def __contains__(self, name: str) -> bool:
        return name in self.meta

    def shape(self, name: str) -> tuple:
        return tuple(self.meta[name]["shape"])

    def dtype(self, name: str) -> str:
        return self.meta[name]["dtype"]

    def raw(self, name: str) -> np.ndarray:
        """The tensor in its stored type; bfloat16 comes as its uint16 bit patterns."""
        m = self.meta[name]
        if m["dtype"] not in _DTYPES:
            raise ValueError(f"{self.path}: tensor {name} has unsupported dtype {m['dtype']}")
        a, b = m["data_offsets"]
        dt = np.dtype(_DTYPES[m["dtype"]])
        n = int(np.prod(m["shape"])) if m["shape"] else 1
        if b - a != n * dt.itemsize:
            raise ValueError(f"{self.path}: tensor {name}: {b - a} bytes for shape {m['shape']}")
        return self._map[self.base + a:self.base + b].view(dt).reshape(m["shape"])

    def f32(self, name: str) -> np.ndarray:
        r = self.raw(name)
        if self.meta[name]["dtype"] == "BF16":
            return (r.astype(np.uint32) << 16).view(np.float32)
        return np.asarray(r, dtype=np.float32)

    def bf16_bits(self, name: str) -> np.ndarray:
        """uint16 bit patterns of a matrix stored in bfloat16."""
        if self.meta[name]["dtype"] != "BF16":
            raise ValueError(f"{self.path}: tensor {name} is {self.meta[name]['dtype']}, the dense path takes bfloat16 matrices")
        return np.ascontiguousarray(self.raw(name))


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even bfloat16 bit patterns (writers of synthetic models use it)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return u.astype(np.uint16)


def write(path: str, tensors: dict) -> None:
    """tensors: name -> numpy array (float32 arrays are stored as bfloat16, int32 as they are)."""
    meta, blobs, off = {}, [], 0
    for name, a in tensors.items():
        a = np.asarray(a)
        if a.dtype == np.int32:
            raw, dt = np.ascontiguousarray(a).tobytes(), "I32"
        else:
            raw, dt = f32_to_bf16_bits(a).tobytes(), "BF16"
        meta[name] = {"dtype": dt, "shape": list(a.shape), "data_offsets": [off, off + len(raw)]}
        blobs.append(raw)
        off += len(raw)
    head = json.dumps(meta, separators=(",", ":")).encode()
    head += b" " * (-len(head) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(head)))
        f.write(head)
        for b in blobs:
            f.write(b)
