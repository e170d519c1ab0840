"""Read and write ``.safetensors`` files by tensor name, without the safetensors package.

Layout of a file: an unsigned 64-bit little-endian header length, that many bytes of JSON
mapping each tensor name to ``{"dtype", "shape", "data_offsets": [begin, end]}`` (offsets
relative to the end of the header; the key ``__metadata__`` holds free-form strings), then the
tensors' bytes.  The reader maps the file into memory and hands out tensors that view it, so a
checkpoint larger than host memory can be streamed to the GPU tensor by tensor.
"""

from __future__ import annotations

import json
import mmap
import struct
from pathlib import Path

import torch

_DTYPES = {
    "F64": torch.float64,
    "F32": torch.float32,
    "F16": torch.float16,
    "BF16": torch.bfloat16,
    "I64": torch.int64,
    "I32": torch.int32,
    "I16": torch.int16,
    "I8": torch.int8,
    "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One mapped file.  ``names()``, ``shape(name)``, ``dtype(name)``, ``tensor(name)``."""

    def __init__(self, path):
        self.path = Path(path)
        self._file = open(self.path, "rb")
        size = self.path.stat().st_size
        if size < 8:
            raise SafetensorsError(f"{self.path}: too short to be a safetensors file")
        (header_len,) = struct.unpack("<Q", self._file.read(8))
        if header_len <= 0 or 8 + header_len > size:
            raise SafetensorsError(f"{self.path}: header length {header_len} exceeds the file")
        try:
            header = json.loads(self._file.read(header_len))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{self.path}: header is not JSON: {e}") from e
        self.metadata = header.pop("__metadata__", {}) or {}
        self._entries = header
        self._data_start = 8 + header_len
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        data_len = size - self._data_start
        for name, entry in header.items():
            if entry["dtype"] not in _DTYPES:
                raise SafetensorsError(f"{self.path}: {name} has unknown dtype {entry['dtype']}")
            begin, end = entry["data_offsets"]
            count = 1
            for s in entry["shape"]:
                count *= s
            width = torch.empty((), dtype=_DTYPES[entry["dtype"]]).element_size()
            if not (0 <= begin <= end <= data_len) or end - begin != count * width:
                raise SafetensorsError(f"{self.path}: {name} has inconsistent offsets")

    def names(self) -> list:
        return list(self._entries)

    def __contains__(self, name: str) -> bool:
        return name in self._entries

    def shape(self, name: str) -> tuple:
        return tuple(self._entries[name]["shape"])

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self._entries[name]["dtype"]]

    def tensor(self, name: str) -> torch.Tensor:
        """A read-only view of the mapped bytes (copy or move it before the file closes)."""
        entry = self._entries[name]
        begin, end = entry["data_offsets"]
        shape = tuple(entry["shape"])
        dtype = _DTYPES[entry["dtype"]]
        if end == begin:
            return torch.empty(shape, dtype=dtype)
        import warnings

        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the map is read-only; the view is never written
            flat = torch.frombuffer(self._map, dtype=torch.uint8, count=end - begin,
                                    offset=self._data_start + begin)
        return flat.view(dtype).reshape(shape)

    def close(self) -> None:
        try:
            self._map.close()
        except BufferError:
            pass  # a tensor still views the map; it is released with the last view
        self._file.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def save_file(tensors: dict, path, metadata: dict | None = None) -> None:
    """Write ``tensors`` (name -> CPU tensor) in name order."""
    header, offset = {}, 0
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    ordered = sorted(tensors)
    for name in ordered:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"{name}: dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * (-len(blob) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in ordered:
            t = tensors[name].detach().cpu().contiguous()
            f.write(t.reshape(-1).view(torch.uint8).numpy().tobytes())


def weight_files(folder) -> list:
    """The checkpoint's files: those an index names, else ``model.safetensors``, else every
    ``*.safetensors`` in the folder (reference: mercury/model/loader.py:34-45)."""
    folder = Path(folder)
    index = folder / "model.safetensors.index.json"
    if index.exists():
        weight_map = json.loads(index.read_text())["weight_map"]
        return sorted({folder / name for name in weight_map.values()})
    single = folder / "model.safetensors"
    if single.exists():
        return [single]
    shards = sorted(folder.glob("*.safetensors"))
    if not shards:
        raise FileNotFoundError(f"no safetensors weights under {folder}")
    return shards
