"""Reading the safetensors container without copying it.

A file is: eight bytes (the header's length, little-endian), that many bytes of JSON
({tensor name: {"dtype", "shape", "data_offsets": [begin, end]}}, plus an optional
"__metadata__" entry), then the tensors' bytes; offsets count from the end of the header.
The file is mapped into memory and every tensor is a view of the mapping: nothing is read
until a tensor's bytes are touched (a copy to the GPU, a conversion), and the pages belong to
the file cache, not to the process.  A checkpoint of tens of gigabytes therefore never
stands in host memory as a whole; the model takes tensor after tensor to the device.
"""
from __future__ import annotations

import json
import mmap
import struct
from pathlib import Path
from typing import Dict, Iterator, Tuple

import torch

# container dtype -> (torch dtype, bytes per element)
_DTYPES = {
    "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_MAX_HEADER = 100 * 1024 * 1024


class SafetensorsFile:
    """One mapped file.  `names()`, `shape(name)`, `dtype(name)` read the header only;
    `tensor(name)` is a view of the mapping on the host, in the stored dtype."""

    def __init__(self, path):
        self.path = Path(path)
        with self.path.open("rb") as source:
            size = source.seek(0, 2)
            source.seek(0)
            prefix = source.read(8)
            if len(prefix) != 8:
                raise ValueError(f"{self.path}: too short to be a safetensors file")
            (header_bytes,) = struct.unpack("<Q", prefix)
            if header_bytes > min(_MAX_HEADER, size - 8):
                raise ValueError(f"{self.path}: the header claims {header_bytes} bytes, "
                                 f"the file has {size}")
            try:
                header = json.loads(source.read(header_bytes).decode("utf-8"))
            except (UnicodeDecodeError, json.JSONDecodeError) as error:
                raise ValueError(f"{self.path}: the header is not JSON: {error}") from None
            if not isinstance(header, dict):
                raise ValueError(f"{self.path}: the header must be a JSON object")
            self._data_start = 8 + header_bytes
            data_bytes = size - self._data_start
            # private copy-on-write mapping: the views are writable tensors, the file is not touched
            self._map = (mmap.mmap(source.fileno(), 0, access=mmap.ACCESS_COPY)
                         if size > 0 else None)
        self.metadata = header.pop("__metadata__", None)
        self._entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        for name, entry in header.items():
            try:
                dtype, itemsize = _DTYPES[entry["dtype"]]
                shape = tuple(int(extent) for extent in entry["shape"])
                begin, end = (int(offset) for offset in entry["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise ValueError(f"{self.path}: malformed or unsupported entry for tensor "
                                 f"'{name}': {entry!r}") from None
            count = 1
            for extent in shape:
                count *= extent
            if (min(shape, default=0) < 0 or not 0 <= begin <= end <= data_bytes
                    or end - begin != count * itemsize):
                raise ValueError(f"{self.path}: tensor '{name}' of shape {list(shape)} does not "
                                 f"fit its bytes [{begin}, {end}) of {data_bytes}")
            self._entries[name] = (dtype, shape, begin, count)

    def names(self) -> Iterator[str]:
        return iter(self._entries)

    def __contains__(self, name) -> bool:
        return name in self._entries

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._entries[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return self._entries[name][0]

    def tensor(self, name: str) -> torch.Tensor:
        dtype, shape, begin, count = self._entries[name]
        if count == 0:
            return torch.empty(shape, dtype=dtype)
        offset = self._data_start + begin
        if offset % dtype.itemsize:     # a writer that did not align the data: copy it out
            raw = bytearray(self._map[offset:offset + count * dtype.itemsize])
            return torch.frombuffer(raw, dtype=dtype, count=count).view(shape)
        return torch.frombuffer(self._map, dtype=dtype, count=count, offset=offset).view(shape)
