"""safetensors container: reader over a memory map, and a writer.

Layout: 8-byte little-endian header length, a JSON object
``name -> {dtype, shape, data_offsets: [start, end)}`` with offsets relative to
the end of the header, then the data section. Checks follow the reference's
reader (crates/safetensors/src/lib.rs:70-124: header within file, start <= end,
end within the data section) and add ``end - start == prod(shape) * itemsize``.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Mapping, Tuple

import numpy as np
import torch


class SafetensorsError(ValueError):
    pass


# dtype tag -> (torch dtype, numpy carrier dtype, itemsize)
_DTYPES = {
    "F32": (torch.float32, np.dtype("<f4"), 4),
    "F16": (torch.float16, np.dtype("<f2"), 2),
    "BF16": (torch.bfloat16, np.dtype("<u2"), 2),     # numpy has no bfloat16: carried as bits
    "F64": (torch.float64, np.dtype("<f8"), 8),
    "I64": (torch.int64, np.dtype("<i8"), 8),
    "I32": (torch.int32, np.dtype("<i4"), 4),
    "I16": (torch.int16, np.dtype("<i2"), 2),
    "I8": (torch.int8, np.dtype("i1"), 1),
    "U8": (torch.uint8, np.dtype("u1"), 1),
    "BOOL": (torch.bool, np.dtype("?"), 1),
}
_TAG_OF = {torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16", torch.float64: "F64",
           torch.int64: "I64", torch.int32: "I32", torch.int16: "I16", torch.int8: "I8",
           torch.uint8: "U8", torch.bool: "BOOL"}


class SafetensorsFile:
    """Views of the tensors of one file, by name; nothing is copied until asked."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: truncated (no header length)")
        self._f = open(path, "rb")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        (hlen,) = struct.unpack("<Q", self._mm[:8])
        if 8 + hlen > size:
            raise SafetensorsError(f"{path}: truncated header ({hlen} bytes announced, file has {size})")
        try:
            header = json.loads(self._mm[8:8 + hlen].decode("utf-8"))
        except Exception as e:  # malformed JSON
            raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header is not a JSON object")
        self._data0 = 8 + hlen
        data_len = size - self._data0
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            try:
                tag = info["dtype"]
                shape = tuple(int(x) for x in info["shape"])
                s, e = (int(x) for x in info["data_offsets"])
            except Exception:
                raise SafetensorsError(f"{path}: entry {name!r} is malformed") from None
            if s > e or e > data_len:
                raise SafetensorsError(f"{path}: {name}: data offsets [{s}, {e}) outside the data section ({data_len} bytes)")
            if tag in _DTYPES:
                n = 1
                for d in shape:
                    n *= d
                if e - s != n * _DTYPES[tag][2]:
                    raise SafetensorsError(f"{path}: {name}: {e - s} bytes do not hold {tag}{list(shape)}")
            self.entries[name] = (tag, shape, s, e)

    def names(self) -> List[str]:
        return list(self.entries)

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name][1]

    def dtype_tag(self, name: str) -> str:
        return self.entries[name][0]

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor of the stored dtype (a copy; the map may be closed afterwards)."""
        if name not in self.entries:
            raise KeyError(name)
        tag, shape, s, e = self.entries[name]
        if tag not in _DTYPES:
            raise SafetensorsError(f"{self.path}: {name}: unsupported dtype {tag}")
        tdtype, ndtype, _ = _DTYPES[tag]
        arr = np.frombuffer(self._mm, dtype=ndtype, count=(e - s) // ndtype.itemsize,
                            offset=self._data0 + s).copy()
        t = torch.from_numpy(arr)
        if tag == "BF16":
            t = t.view(torch.bfloat16)
        return t.reshape(shape)

    def close(self) -> None:
        try:
            self._mm.close()
        finally:
            self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor], metadata: Mapping[str, str] = None) -> None:
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _TAG_OF:
            raise SafetensorsError(f"{name}: cannot store dtype {t.dtype}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _TAG_OF[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            if t.dtype == torch.bfloat16:
                t = t.view(torch.int16)
            f.write(t.numpy().tobytes())
    os.replace(tmp, path)
