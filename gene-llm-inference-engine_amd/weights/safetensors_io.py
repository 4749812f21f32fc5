"""Reading and writing of single-file safetensors checkpoints.

Format as the reference reads it (src/loader/safetensors.cpp:25-88): eight bytes of
little-endian header length, a JSON object that maps tensor names to
{dtype, shape, data_offsets [begin, end)} with offsets relative to the end of the header, an
optional "__metadata__" entry, then the data.  The file is memory-mapped and tensors are views
into the mapping, so a large file is never read whole into host memory.
"""
from __future__ import annotations

import json
import mmap
import struct
import warnings
from dataclasses import dataclass
from pathlib import Path
from typing import Dict, Tuple

import torch


class SafetensorsError(ValueError):
    pass


_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}
_MAX_HEADER = 100 * 1024 * 1024      # src/loader/safetensors.cpp:37


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype_name: str
    shape: Tuple[int, ...]
    begin: int
    end: int

    @property
    def numel(self):
        n = 1
        for s in self.shape:
            n *= s
        return n


class SafetensorsFile:
    """Entries by name and zero-copy CPU tensors over the mapped file."""

    def __init__(self, path):
        self.path = str(path)
        self._file = open(path, "rb")
        size = Path(path).stat().st_size
        if size < 8:
            raise SafetensorsError(f"{self.path}: too small to be a safetensors file")
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        (hlen,) = struct.unpack("<Q", self._map[:8])
        if hlen > _MAX_HEADER or hlen > size - 8:
            raise SafetensorsError(f"{self.path}: header length {hlen} does not fit the file")
        try:
            header = json.loads(self._map[8:8 + hlen].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{self.path}: header is not valid JSON ({e})") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{self.path}: header is not a JSON object")
        self._data_start = 8 + hlen
        data_size = size - self._data_start
        self.metadata = header.get("__metadata__") or {}
        self.entries: Dict[str, TensorEntry] = {}
        for name, e in header.items():
            if name == "__metadata__":
                continue
            try:
                dtype_name, shape, (b, t) = e["dtype"], tuple(int(s) for s in e["shape"]), e["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{self.path}: entry '{name}' is malformed") from None
            if any(s < 0 for s in shape) or not 0 <= b <= t <= data_size:
                raise SafetensorsError(f"{self.path}: entry '{name}' has offsets or a shape outside the file")
            entry = TensorEntry(name, dtype_name, shape, int(b), int(t))
            if dtype_name in _DTYPES:
                want = entry.numel * torch.empty((), dtype=_DTYPES[dtype_name]).element_size()
                if want != t - b:
                    raise SafetensorsError(f"{self.path}: entry '{name}' holds {t - b} bytes, its shape needs {want}")
            self.entries[name] = entry

    def __contains__(self, name):
        return name in self.entries

    def tensor(self, name) -> torch.Tensor:
        """A read-only CPU view of the tensor's bytes (copy it before changing it)."""
        e = self.entries[name]
        if e.dtype_name not in _DTYPES:
            raise SafetensorsError(f"tensor '{name}' has unsupported dtype {e.dtype_name}")
        if e.numel == 0:
            return torch.empty(e.shape, dtype=_DTYPES[e.dtype_name])
        dtype = _DTYPES[e.dtype_name]
        start = self._data_start + e.begin
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")      # the mapping is read-only; nothing here writes to it
            if start % torch.empty((), dtype=dtype).element_size() == 0:
                flat = torch.frombuffer(self._map, dtype=dtype, count=e.numel, offset=start)
            else:                                # data at an odd address: an aligned copy
                flat = torch.frombuffer(bytearray(self._map[start:self._data_start + e.end]), dtype=dtype)
        return flat.reshape(e.shape)

    def close(self):
        """Closes the file.  The mapping itself lives as long as any tensor made from it (tensors keep
        a reference to it), so it is never unmapped under a tensor."""
        self._file.close()


def write_safetensors(path, tensors: Dict[str, torch.Tensor], metadata=None) -> None:
    """Writes CPU tensors under their names; data are 8-byte aligned behind a padded header."""
    header, offset, ordered = {}, 0, []
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor '{name}' has dtype {t.dtype}, which safetensors cannot hold")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        ordered.append(t)
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    text += b" " * (-(8 + len(text)) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for t in ordered:
            if t.numel():
                f.write(memoryview(t.reshape(-1).view(torch.uint8).numpy()))
