"""Reading and writing safetensors files without any library.

Format (as the reference's reader parses it, models/qwen35.py:95-123): an 8-byte little-endian
header length, a JSON header that gives ``dtype``, ``shape`` and ``data_offsets`` (relative to the end
of the header) for each tensor, then the bytes.  The checks are those of the reference's streaming
index (models/safetensors_stream.py:71-118): header size, truncation, ``end >= begin``, byte size
equal to the product of the shape times the item size, known dtype.

Files are memory-mapped: a tensor is a view of the file until it is copied to the device.
"""
from __future__ import annotations

import json
import mmap
import struct
from pathlib import Path

import numpy as np
import torch

MAX_HEADER_BYTES = 1 << 30

_DTYPES = {
    "F32": (torch.float32, 4), "F16": (torch.float16, 2), "BF16": (torch.bfloat16, 2),
    "F64": (torch.float64, 8), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One memory-mapped file: ``entries[name] = (dtype name, shape, begin, end)``."""

    def __init__(self, path):
        self.path = Path(path)
        size = self.path.stat().st_size
        if size < 8:
            raise SafetensorsError(f"{self.path}: file of {size} bytes is too short for a safetensors header")
        self._fh = open(self.path, "rb")
        (hlen,) = struct.unpack("<Q", self._fh.read(8))
        if hlen > MAX_HEADER_BYTES:
            raise SafetensorsError(f"{self.path}: header length {hlen} exceeds {MAX_HEADER_BYTES}")
        if 8 + hlen > size:
            raise SafetensorsError(f"{self.path}: header of {hlen} bytes is cut off (file has {size})")
        try:
            header = json.loads(self._fh.read(hlen))
        except json.JSONDecodeError as e:
            raise SafetensorsError(f"{self.path}: header is not JSON: {e}") from None
        self._base = 8 + hlen
        self.entries: dict[str, tuple[str, tuple[int, ...], int, int]] = {}
        for name, meta in header.items():
            if name == "__metadata__":
                continue
            dt, shape = meta.get("dtype"), tuple(int(s) for s in meta.get("shape", ()))
            begin, end = (int(v) for v in meta["data_offsets"])
            if dt not in _DTYPES:
                raise SafetensorsError(f"{self.path}: tensor {name}: dtype {dt!r} is not supported")
            if end < begin or self._base + end > size:
                raise SafetensorsError(f"{self.path}: tensor {name}: bytes [{begin}, {end}) lie outside the file")
            want = int(np.prod(shape, dtype=np.int64)) * _DTYPES[dt][1]
            if end - begin != want:
                raise SafetensorsError(f"{self.path}: tensor {name}: {end - begin} bytes stored, "
                                       f"shape {list(shape)} of {dt} needs {want}")
            self.entries[name] = (dt, shape, begin, end)
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def tensor(self, name: str) -> torch.Tensor:
        """A read-only view of the file's bytes as a CPU tensor (not a copy)."""
        dt, shape, begin, end = self.entries[name]
        tdt, _ = _DTYPES[dt]
        if end == begin:
            return torch.empty(shape, dtype=tdt)
        buf = memoryview(self._map)[self._base + begin:self._base + end]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the buffer is read-only; nothing here writes to it
            flat = torch.frombuffer(buf, dtype=tdt)
        return flat.reshape(shape)


class ModelFiles:
    """All safetensors files of a model folder as one name -> tensor map.

    ``model.safetensors.index.json`` is followed if it is there (models/safetensors_stream.py:53-69);
    else the patterns of the reference (models/qwen3.py:39-54)."""

    def __init__(self, model_dir):
        model_dir = Path(model_dir)
        index = model_dir / "model.safetensors.index.json"
        if index.is_file():
            names = sorted(set(json.loads(index.read_text())["weight_map"].values()))
            paths = [model_dir / n for n in names]
        else:
            paths, seen = [], set()
            for pattern in ("model.safetensors", "model-*.safetensors", "model.safetensors-*.safetensors"):
                for p in sorted(model_dir.glob(pattern)):
                    if p not in seen:
                        seen.add(p)
                        paths.append(p)
        if not paths:
            raise FileNotFoundError(f"No safetensors file in {model_dir}")
        self.files = [SafetensorsFile(p) for p in paths]
        self._where: dict[str, SafetensorsFile] = {}
        for f in self.files:
            for name in f.entries:
                self._where[name] = f

    def names(self) -> list[str]:
        return list(self._where)

    def shape(self, name: str) -> tuple[int, ...]:
        return self._where[name].entries[name][1]

    def dtype_name(self, name: str) -> str:
        return self._where[name].entries[name][0]

    def tensor(self, name: str) -> torch.Tensor:
        return self._where[name].tensor(name)


def write_safetensors(path, tensors: dict[str, torch.Tensor], metadata: dict | None = None) -> None:
    """Write CPU tensors in the order given; offsets are contiguous and the header is padded with
    spaces to a multiple of 8 bytes."""
    header, offset, blobs = {}, 0, []
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    for name, t in tensors.items():
        t = t.detach().contiguous().cpu()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name}: dtype {t.dtype} cannot be written")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        blobs.append(t)
        offset += nbytes
    raw = json.dumps(header, separators=(",", ":")).encode()
    raw += b" " * (-len(raw) % 8)
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(raw)))
        fh.write(raw)
        for t in blobs:
            if t.numel():
                fh.write(t.reshape(-1).view(torch.uint8).numpy().tobytes())
