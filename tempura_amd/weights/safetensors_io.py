"""Minimal safetensors reader and writer (format only; no model knowledge).

A file is an 8-byte little-endian header length, a JSON header mapping tensor
names to ``{"dtype", "shape", "data_offsets"}``, and the raw little-endian data.
The reader maps the file and hands out tensors one by one, so a large checkpoint
never needs a second host copy (the reference maps its shards the same way,
/root/reference/engine/src/loader.rs:119-145).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch

# safetensors dtype tag -> (numpy dtype used to view the bytes, torch dtype of the result)
_DTYPES = {
    "F64": (np.float64, torch.float64),
    "F32": (np.float32, torch.float32),
    "F16": (np.float16, torch.float16),
    "BF16": (np.int16, torch.bfloat16),
    "I64": (np.int64, torch.int64),
    "I32": (np.int32, torch.int32),
    "I16": (np.int16, torch.int16),
    "I8": (np.int8, torch.int8),
    "U8": (np.uint8, torch.uint8),
    "BOOL": (np.bool_, torch.bool),
}
_TAG_OF = {torch.float64: "F64", torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16",
           torch.int64: "I64", torch.int32: "I32", torch.int16: "I16", torch.int8: "I8",
           torch.uint8: "U8", torch.bool: "BOOL"}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One mapped ``.safetensors`` file."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._f = open(path, "rb")
        except OSError as e:
            raise SafetensorsError(f"cannot open {path}: {e}") from e
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen <= 0 or 8 + hlen > size:
            raise SafetensorsError(f"{path}: header length {hlen} exceeds file size {size}")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from e
        self.metadata = header.pop("__metadata__", {}) or {}
        self._data_start = 8 + hlen
        self._entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        for name, info in header.items():
            tag = info.get("dtype")
            if tag not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {tag!r}")
            shape = tuple(int(s) for s in info["shape"])
            b, e = (int(x) for x in info["data_offsets"])
            n = int(np.prod(shape, dtype=np.int64)) if shape else 1
            if e - b != n * np.dtype(_DTYPES[tag][0]).itemsize or self._data_start + e > size or b < 0:
                raise SafetensorsError(f"{path}: tensor {name!r} has inconsistent offsets {b}:{e} for shape {shape}")
            self._entries[name] = (tag, shape, b, e)
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_COPY) if size > 0 else None

    def names(self) -> List[str]:
        return list(self._entries)

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._entries[name][1]

    def dtype_tag(self, name: str) -> str:
        return self._entries[name][0]

    def tensor(self, name: str) -> torch.Tensor:
        """The tensor as stored (a view of the mapping; copy before the file is closed)."""
        tag, shape, b, e = self._entries[name]
        np_dt, t_dt = _DTYPES[tag]
        n = int(np.prod(shape, dtype=np.int64)) if shape else 1
        arr = np.frombuffer(self._mm, dtype=np_dt, count=n, offset=self._data_start + b)
        t = torch.from_numpy(arr)
        if tag == "BF16":
            t = t.view(torch.bfloat16)
        return t.reshape(shape)

    def close(self) -> None:
        # numpy views may still reference the mapping; dropping our handles is enough.
        self._mm = None
        self._f.close()


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata=None) -> None:
    """Write ``(name, tensor)`` pairs to ``path``.

    ``tensors`` may be a generator called twice: it is given as a callable-free
    iterable of already materialised tensors, or as a list.  Tensors are written
    in name order of arrival; each is moved to host and made contiguous.
    """
    items = list(tensors)
    header = {}
    off = 0
    for name, t in items:
        if t.dtype not in _TAG_OF:
            raise SafetensorsError(f"cannot store dtype {t.dtype} for {name!r}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _TAG_OF[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + nbytes]}
        off += nbytes
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    hbytes = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hbytes += b" " * ((8 - len(hbytes) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hbytes)))
        f.write(hbytes)
        for name, t in items:
            t = t.detach().to("cpu").contiguous()
            if t.dtype == torch.bfloat16:
                f.write(t.view(torch.int16).numpy().tobytes())
            else:
                f.write(t.numpy().tobytes())
