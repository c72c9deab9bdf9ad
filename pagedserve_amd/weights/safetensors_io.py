"""A small reader and writer for the safetensors file format.

Layout of a file: an unsigned 64-bit little-endian header length ``n``; ``n`` bytes
of JSON that map each tensor name to ``{"dtype", "shape", "data_offsets": [begin,
end]}`` (offsets relative to the end of the header; the key ``__metadata__`` holds
free-form strings); then the raw little-endian tensor bytes.

The reference delegates reading to ``transformers`` (src/model/gpt2.py:92-93); this
engine reads the file itself, by name, through a memory map, so that a tensor is
only paged in when it is converted.
"""

import json
import mmap
import os
import struct
from typing import Dict, Tuple

import torch

_DTYPES = {
    "F64": (torch.float64, 8),
    "F32": (torch.float32, 4),
    "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2),
    "I64": (torch.int64, 8),
    "I32": (torch.int32, 4),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {dtype: name for name, (dtype, _) in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """Header of one file plus lazy access to its tensors."""

    def __init__(self, path):
        self.path = path
        if not os.path.isfile(path):
            raise SafetensorsError(f"no such file: {path}")
        self._handle = open(path, "rb")
        size = os.fstat(self._handle.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        (header_len,) = struct.unpack("<Q", self._handle.read(8))
        if header_len > size - 8:
            raise SafetensorsError(f"{path}: header length {header_len} exceeds the file")
        try:
            header = json.loads(self._handle.read(header_len).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as error:
            raise SafetensorsError(f"{path}: header is not JSON ({error})") from error
        self.metadata = header.pop("__metadata__", {}) or {}
        self._data_start = 8 + header_len
        self._data_len = size - self._data_start
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        for name, info in header.items():
            dtype = info.get("dtype")
            if dtype not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unknown dtype {dtype!r}")
            shape = tuple(int(extent) for extent in info["shape"])
            begin, end = (int(offset) for offset in info["data_offsets"])
            count = 1
            for extent in shape:
                count *= extent
            if end - begin != count * _DTYPES[dtype][1] or begin < 0 or end > self._data_len:
                raise SafetensorsError(f"{path}: tensor {name!r} has inconsistent offsets")
            self.entries[name] = (dtype, shape, begin, end)
        self._map = None

    def names(self):
        return list(self.entries)

    def shape(self, name) -> Tuple[int, ...]:
        return self.entries[name][1]

    def dtype(self, name) -> torch.dtype:
        return _DTYPES[self.entries[name][0]][0]

    def tensor(self, name) -> torch.Tensor:
        """A CPU tensor that copies the bytes of ``name`` out of the map."""
        dtype_name, shape, begin, end = self.entries[name]
        dtype, _ = _DTYPES[dtype_name]
        if end == begin:
            return torch.empty(shape, dtype=dtype)
        if self._map is None:
            self._map = mmap.mmap(self._handle.fileno(), 0, access=mmap.ACCESS_READ)
        raw = bytearray(self._map[self._data_start + begin:self._data_start + end])
        return torch.frombuffer(raw, dtype=dtype).reshape(shape)

    def close(self):
        if self._map is not None:
            self._map.close()
            self._map = None
        self._handle.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def write_safetensors(path, tensors: Dict[str, torch.Tensor], metadata=None):
    """Write ``tensors`` (CPU, any supported dtype) under their names, sorted."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(key): str(value) for key, value in metadata.items()}
    offset = 0
    order = sorted(tensors)
    for name in order:
        tensor = tensors[name]
        if tensor.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name!r}: dtype {tensor.dtype} cannot be stored")
        nbytes = tensor.numel() * tensor.element_size()
        header[name] = {
            "dtype": _NAMES[tensor.dtype],
            "shape": list(tensor.shape),
            "data_offsets": [offset, offset + nbytes],
        }
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(blob)))
        handle.write(blob)
        for name in order:
            tensor = tensors[name].detach().cpu().contiguous()
            if tensor.numel() == 0:
                continue
            if tensor.dtype == torch.bool:
                tensor = tensor.to(torch.uint8)
            handle.write(tensor.reshape(-1).view(torch.uint8).numpy().tobytes())
