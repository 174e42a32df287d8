"""Reading and writing the safetensors container: an 8-byte little-endian header
length, a JSON header (name -> dtype, shape, byte range), then the raw bytes.

Tensors are looked up by name, as the reference looks its tensors up in the map
that its container reader returns (J/core/model/GGUF.java:58-70,
J/model/loader/ModelLoader.java:285-303); the file is memory-mapped and a tensor
is a view until it is copied to the device.
"""
from __future__ import annotations

import json
import mmap
import os
import struct

import torch

_DTYPES = {
    "F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "F64": torch.float64,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One memory-mapped .safetensors file."""

    def __init__(self, path):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: {size} bytes is too short for a safetensors header")
        self._f = open(path, "rb")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n > size - 8:
            raise SafetensorsError(f"{path}: header says {n} bytes but the file has {size - 8} after the length")
        try:
            header = json.loads(self._f.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON ({e})") from None
        self.metadata = header.pop("__metadata__", {}) or {}
        self._base = 8 + n
        self.entries = {}
        for name, e in header.items():
            dt = e.get("dtype")
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dt!r}")
            shape = tuple(int(s) for s in e["shape"])
            b, end = (int(o) for o in e["data_offsets"])
            count = 1
            for s in shape:
                count *= s
            want = count * torch.empty((), dtype=_DTYPES[dt]).element_size()
            if b < 0 or end < b:
                raise SafetensorsError(f"{path}: tensor {name!r} has the byte range {b}..{end}, which is no range "
                                       "of the data that follows the header")
            if end - b != want:
                raise SafetensorsError(f"{path}: tensor {name!r} of shape {shape} {dt} needs {want} bytes, "
                                       f"its range holds {end - b}")
            if self._base + end > size:
                raise SafetensorsError(f"{path}: file is truncated: tensor {name!r} ends at byte "
                                       f"{self._base + end}, the file has {size}")
            self.entries[name] = (_DTYPES[dt], shape, b, count)
        # two tensors never share bytes: a header whose ranges overlap would load one tensor's values as another's
        last_end, last_name = 0, None
        for name, (dt, shape, b, count) in sorted(self.entries.items(), key=lambda kv: kv[1][2]):
            if count == 0:
                continue
            if b < last_end:
                raise SafetensorsError(f"{path}: tensors {last_name!r} and {name!r} overlap (byte {b} lies before {last_end})")
            last_end, last_name = b + count * torch.empty((), dtype=dt).element_size(), name
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def names(self):
        return list(self.entries)

    def shape(self, name):
        return self.entries[name][1]

    def dtype(self, name):
        return self.entries[name][0]

    def tensor(self, name):
        """A CPU tensor that views the mapped file (read-only: copy before writing)."""
        dtype, shape, begin, count = self.entries[name]
        if count == 0:
            return torch.empty(shape, dtype=dtype)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")   # the buffer is read-only; the view is never written
            t = torch.frombuffer(self._mm, dtype=dtype, count=count, offset=self._base + begin)
        return t.reshape(shape)

    def close(self):
        self._mm = None
        self._f.close()


def write_safetensors(path, tensors, metadata=None):
    """Write ``{name: CPU tensor}`` in name order. ``tensors`` may be an iterable of
    ``(name, shape, dtype, make)`` so that one tensor at a time is in memory."""
    items = []
    if isinstance(tensors, dict):
        for name in sorted(tensors):
            t = tensors[name]
            items.append((name, tuple(t.shape), t.dtype, (lambda t=t: t)))
    else:
        items = sorted(tensors, key=lambda it: it[0])
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    for name, shape, dtype, _ in items:
        n = 1
        for s in shape:
            n *= s
        nbytes = n * torch.empty((), dtype=dtype).element_size()
        header[name] = {"dtype": _NAMES[dtype], "shape": list(shape), "data_offsets": [off, off + nbytes]}
        off += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".part"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, shape, dtype, make in items:
            t = make().contiguous()
            if tuple(t.shape) != tuple(shape) or t.dtype != dtype:
                raise ValueError(f"{name}: made {tuple(t.shape)} {t.dtype}, declared {shape} {dtype}")
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)
