"""Reader and writer for the safetensors container: an 8-byte little-endian header length, a
JSON header {name: {dtype, shape, data_offsets}}, then the raw little-endian tensor bytes.
The reader maps the file and checks every tensor's byte range against the file before
anything is read, as the reference does for its own container
(src/minillm/gguf_model.cpp:110-127)."""
from __future__ import annotations

import json
import mmap
import os
import struct
import warnings

import torch

_DTYPES = {
    "F32": (torch.float32, 4), "BF16": (torch.bfloat16, 2), "F16": (torch.float16, 2),
    "F64": (torch.float64, 8), "I32": (torch.int32, 4), "I64": (torch.int64, 8),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """A mapped safetensors file: `entries` holds (dtype, shape) per name without touching
    the data; `tensor(name)` returns a CPU tensor that views the mapping."""

    def __init__(self, path):
        self.path = path
        if not os.path.isfile(path):
            raise SafetensorsError(f"{path}: no such file")
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: truncated (no header length)")
        self._file = open(path, "rb")
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        (header_len,) = struct.unpack("<Q", self._map[:8])
        if header_len > size - 8:
            raise SafetensorsError(f"{path}: header length {header_len} exceeds the file")
        try:
            header = json.loads(self._map[8:8 + header_len].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as err:
            raise SafetensorsError(f"{path}: header is not JSON ({err})") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header is not a JSON object")
        self._data_start = 8 + header_len
        data_bytes = size - self._data_start
        self.entries = {}
        self._ranges = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            try:
                dtype_name, shape, (begin, end) = info["dtype"], info["shape"], info["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: malformed header entry for {name}") from None
            if dtype_name not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name} has unsupported dtype {dtype_name}")
            dtype, width = _DTYPES[dtype_name]
            count = 1
            for extent in shape:
                count *= int(extent)
            if begin < 0 or end < begin or end > data_bytes or end - begin != count * width:
                raise SafetensorsError(f"{path}: tensor {name} has a byte range outside the file "
                                       f"or of the wrong size")
            self.entries[name] = (dtype, tuple(int(e) for e in shape))
            self._ranges[name] = (begin, count)

    def tensor(self, name):
        dtype, shape = self.entries[name]
        begin, count = self._ranges[name]
        if count == 0:
            return torch.empty(shape, dtype=dtype)
        start = self._data_start + begin
        width = _DTYPES[_NAMES[dtype]][1]
        if start % width == 0:
            with warnings.catch_warnings():
                warnings.simplefilter("ignore", UserWarning)      # the mapping is read-only; nobody writes
                flat = torch.frombuffer(self._map, dtype=dtype, count=count, offset=start)
        else:                                                     # misaligned in the file: copy out
            flat = torch.frombuffer(bytearray(self._map[start:start + count * width]), dtype=dtype, count=count)
        return flat.view(shape)

    def close(self):
        # tensors returned by `tensor` view the mapping: the caller copies before closing
        try:
            self._map.close()
        except BufferError:
            pass
        self._file.close()


def write_safetensors(path, tensors, metadata=None):
    """Write {name: CPU tensor}: widest element types first, then by name, bytes back to back
    (every tensor then starts at a multiple of its element size)."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for t in tensors.values():
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"cannot write dtype {t.dtype}")
    ordered = []
    for name in sorted(tensors, key=lambda n: (-tensors[n].element_size(), n)):
        t = tensors[name].detach().contiguous().cpu()
        size = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + size]}
        ordered.append(t)
        offset += size
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    text += b" " * ((-len(text)) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for t in ordered:                                  # (straight from the tensor's memory: no second copy)
            if t.numel():
                f.write(memoryview(t.view(torch.uint8).reshape(-1).numpy()))
