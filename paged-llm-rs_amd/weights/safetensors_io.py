"""Reading and writing the safetensors container.

The format: eight bytes of little-endian header length, a JSON header mapping
each tensor name to ``{"dtype", "shape", "data_offsets"}`` (offsets relative to
the end of the header), then the raw little-endian data.  The file is mapped,
not read: a tensor's bytes are touched when it is copied to the device.
"""

from __future__ import annotations

import json
import mmap
import struct
import warnings
from pathlib import Path

import torch

from ..errors import IoError, WeightError

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    """The header of one file and lazy access to its tensors."""

    def __init__(self, path):
        self.path = Path(path)
        try:
            self._file = open(self.path, "rb")
        except OSError as e:
            raise IoError(f"reading {self.path}: {e}") from e
        head = self._file.read(8)
        if len(head) != 8:
            raise WeightError(f"{self.path}: shorter than a safetensors header")
        (length,) = struct.unpack("<Q", head)
        size = self.path.stat().st_size
        if length > size - 8:
            raise WeightError(f"{self.path}: header of {length} bytes in a file of {size}")
        try:
            header = json.loads(self._file.read(length))
        except (json.JSONDecodeError, UnicodeDecodeError) as e:
            raise WeightError(f"{self.path}: header is not JSON: {e}") from e
        if not isinstance(header, dict):
            raise WeightError(f"{self.path}: header is not a JSON object")
        self.metadata = header.pop("__metadata__", {})
        self.entries = header
        self._base = 8 + length
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ) if size else None
        for name, e in self.entries.items():
            # (a file that was cut, or written by something else, is a wrong weight file and said to be one)
            whole = (lambda v: isinstance(v, int) and not isinstance(v, bool) and v >= 0)
            offsets = e.get("data_offsets") if isinstance(e, dict) else None
            if not (isinstance(e, dict) and isinstance(e.get("shape"), list) and all(whole(n) for n in e["shape"])
                    and isinstance(offsets, list) and len(offsets) == 2 and all(whole(n) for n in offsets)
                    and isinstance(e.get("dtype"), str)):
                raise WeightError(f"{self.path}: the entry of {name!r} is not a dtype, a shape and two data offsets")
            if e["dtype"] not in _DTYPES:
                raise WeightError(f"{self.path}: {name} has dtype {e['dtype']!r}, which is not read here")
            begin, end = offsets
            count = 1
            for n in e["shape"]:
                count *= n
            width = torch.empty((), dtype=_DTYPES[e["dtype"]]).element_size()
            if end < begin or end - begin != count * width or self._base + end > size:
                raise WeightError(f"{self.path}: {name} has the bytes {begin} to {end} for shape {e['shape']}, in a file "
                                  f"with {size - self._base} bytes of data")

    def names(self):
        return list(self.entries)

    def shape(self, name) -> tuple:
        return tuple(self.entries[name]["shape"])

    def dtype(self, name) -> torch.dtype:
        return _DTYPES[self.entries[name]["dtype"]]

    def tensor(self, name) -> torch.Tensor:
        """A CPU tensor viewing the mapped bytes (read-only; copy before writing)."""
        e = self.entries[name]
        begin, end = e["data_offsets"]
        shape = tuple(e["shape"])
        dtype = _DTYPES[e["dtype"]]
        if end == begin:
            return torch.empty(shape, dtype=dtype)
        view = memoryview(self._map)[self._base + begin:self._base + end]
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)   # the map is read-only, and only read
            return torch.frombuffer(view, dtype=dtype).reshape(shape)

    def close(self):
        # Tensors handed out may still view the map; it is closed with them.
        self._file.close()


def write_safetensors(path, tensors, metadata: dict | None = None) -> None:
    """Write ``tensors`` (an iterable of (name, make) where ``make()`` returns a
    CPU tensor, or a dict of tensors) one after the other, so that a large model
    never sits in memory twice.  ``make`` is called twice for a callable entry:
    once is avoided by passing ``(name, shape, dtype, make)``."""
    items = []
    if isinstance(tensors, dict):
        for name, t in tensors.items():
            items.append((name, tuple(t.shape), t.dtype, (lambda t=t: t)))
    else:
        items = list(tensors)
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    for name, shape, dtype, _ in items:
        if dtype not in _NAMES:
            raise WeightError(f"{name} has dtype {dtype}, which is not written here")
        count = 1
        for s in shape:
            count *= s
        size = count * torch.empty((), dtype=dtype).element_size()
        header[name] = {"dtype": _NAMES[dtype], "shape": list(shape), "data_offsets": [offset, offset + size]}
        offset += size
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * (-len(blob) % 8)
    path = Path(path)
    try:
        with open(path, "wb") as f:
            f.write(struct.pack("<Q", len(blob)))
            f.write(blob)
            for name, shape, dtype, make in items:
                t = make().contiguous()
                if tuple(t.shape) != tuple(shape) or t.dtype != dtype:
                    raise WeightError(f"{name}: made {tuple(t.shape)} {t.dtype}, declared {shape} {dtype}")
                f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    except OSError as e:
        raise IoError(f"writing {path}: {e}") from e
