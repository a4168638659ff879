"""Reading and writing safetensors files.

Layout of a file: eight bytes holding the little-endian length N of the header,
N bytes of JSON ``{name: {"dtype", "shape", "data_offsets": [begin, end]}, ...}``
(plus an optional ``__metadata__`` entry), then the tensors' bytes, offsets
counted from the end of the header.  The reader maps the file and hands out
tensors that view the mapping, so a checkpoint larger than memory is never read
whole (the reference maps its files too: backends/vllm/src/models/llama.rs:84-93).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch

# safetensors dtype name -> (numpy dtype of the raw bytes, torch dtype to view them as)
_DTYPES = {
    "F64": (np.float64, torch.float64),
    "F32": (np.float32, torch.float32),
    "F16": (np.float16, torch.float16),
    "BF16": (np.uint16, torch.bfloat16),
    "I64": (np.int64, torch.int64),
    "I32": (np.int32, torch.int32),
    "I16": (np.int16, torch.int16),
    "I8": (np.int8, torch.int8),
    "U8": (np.uint8, torch.uint8),
    "BOOL": (np.bool_, torch.bool),
}
_NAMES = {torch.float64: "F64", torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16",
          torch.int64: "I64", torch.int32: "I32", torch.int16: "I16", torch.int8: "I8", torch.uint8: "U8",
          torch.bool: "BOOL"}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """A mapped safetensors file: names, shapes and dtypes without touching the data; tensors on request."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._fh = open(path, "rb")
        except OSError as e:
            raise SafetensorsError(f"cannot open {path}: {e}") from None
        size = os.fstat(self._fh.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        (n,) = struct.unpack("<Q", self._fh.read(8))
        if n > size - 8:
            raise SafetensorsError(f"{path}: header length {n} exceeds the file size {size}")
        try:
            header = json.loads(self._fh.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from None
        self.metadata = header.pop("__metadata__", None) or {}
        self._base = 8 + n
        self._entries: Dict[str, dict] = {}
        for name, e in header.items():
            dt, shape, (b, end) = e.get("dtype"), e.get("shape"), e.get("data_offsets", (None, None))
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor '{name}' has unsupported dtype {dt}")
            want = int(np.prod(shape, dtype=np.int64)) * np.dtype(_DTYPES[dt][0]).itemsize
            if b is None or end - b != want or self._base + end > size:
                raise SafetensorsError(f"{path}: tensor '{name}' has inconsistent offsets")
            self._entries[name] = {"dtype": dt, "shape": tuple(shape), "begin": b, "end": end}
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def names(self) -> List[str]:
        return list(self._entries)

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._entries[name]["shape"]

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self._entries[name]["dtype"]][1]

    def tensor(self, name: str) -> torch.Tensor:
        """A read-only CPU tensor viewing the mapped bytes (copy it before changing it)."""
        e = self._entries[name]
        np_dt, t_dt = _DTYPES[e["dtype"]]
        count = int(np.prod(e["shape"], dtype=np.int64))
        if count == 0:
            return torch.empty(e["shape"], dtype=t_dt)
        arr = np.frombuffer(self._map, dtype=np_dt, count=count, offset=self._base + e["begin"])
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # torch warns that the array is not writable
            t = torch.from_numpy(arr)
        if t_dt is torch.bfloat16:
            t = t.view(torch.bfloat16)
        return t.reshape(e["shape"])

    def close(self):
        # tensors handed out keep the mapping alive through numpy's buffer reference
        self._fh.close()


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata: Dict[str, str] = None,
                      ) -> None:
    """Write ``(name, tensor)`` pairs in the given order.  Tensors are consumed one at a time."""
    tensors = list(tensors)
    header: Dict[str, dict] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    for name, t in tensors:
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor '{name}': dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + nbytes]}
        off += nbytes
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * ((8 - len(raw) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(raw)))
        f.write(raw)
        for _, t in tensors:
            t = t.detach().contiguous().cpu()
            if t.dtype is torch.bfloat16:
                t = t.view(torch.int16)
            f.write(t.numpy().tobytes())
    os.replace(tmp, path)
