"""Reading and writing safetensors files (reference: src/safetensors.ts:16-106).

The reader memory-maps the file, checks the whole header before any tensor is
read, and hands tensors out in their stored dtype (no widening).  The checks
are the reference's: header length, dtype, shape, offsets inside the file,
and tensors that tile the data region without gaps or overlap.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass

import numpy as np
import torch


class SafetensorsError(ValueError):
    pass


_DTYPES = {
    "F32": (4, torch.float32, np.dtype("<f4")),
    "BF16": (2, torch.bfloat16, np.dtype("<i2")),
    "F16": (2, torch.float16, np.dtype("<f2")),
    "I32": (4, torch.int32, np.dtype("<i4")),
    "I64": (8, torch.int64, np.dtype("<i8")),
}
_NAMES = {torch.float32: "F32", torch.bfloat16: "BF16", torch.float16: "F16",
          torch.int32: "I32", torch.int64: "I64"}
MAX_HEADER = 16 * 1024 * 1024


def stored_dtype(name: str) -> torch.dtype:
    """The torch dtype of a safetensors dtype name."""
    return _DTYPES[name][1]


@dataclass(frozen=True)
class TensorInfo:
    dtype: str
    shape: tuple[int, ...]
    begin: int
    end: int


class SafetensorsFile:
    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        self._file = open(path, "rb")
        try:
            prefix = self._file.read(8)
            if len(prefix) < 8:
                raise SafetensorsError(f"{path}: truncated safetensors file.")
            (header_size,) = struct.unpack("<Q", prefix)
            if header_size <= 0 or header_size > MAX_HEADER or header_size + 8 > size:
                raise SafetensorsError(f"{path}: invalid safetensors header length {header_size}.")
            try:
                parsed = json.loads(self._file.read(header_size).decode("utf-8"))
            except (UnicodeDecodeError, json.JSONDecodeError):
                raise SafetensorsError(f"{path}: invalid safetensors header.") from None
            if not isinstance(parsed, dict):
                raise SafetensorsError(f"{path}: invalid safetensors header.")
            data_size = size - 8 - header_size
            entries: dict[str, TensorInfo] = {}
            for name, raw in parsed.items():
                if name == "__metadata__":
                    continue
                ok = (isinstance(raw, dict) and raw.get("dtype") in _DTYPES and isinstance(raw.get("shape"), list)
                      and all(isinstance(n, int) and not isinstance(n, bool) and n > 0 for n in raw["shape"])
                      and isinstance(raw.get("data_offsets"), list) and len(raw["data_offsets"]) == 2
                      and all(isinstance(n, int) and not isinstance(n, bool) for n in raw["data_offsets"]))
                if not ok:
                    raise SafetensorsError(f"{path}: unsupported or malformed tensor {name!r}.")
                begin, end = raw["data_offsets"]
                count = 1
                for n in raw["shape"]:
                    count *= n
                if begin < 0 or end - begin != count * _DTYPES[raw["dtype"]][0] or end > data_size:
                    raise SafetensorsError(f"{path}: invalid tensor offsets for {name!r}.")
                entries[name] = TensorInfo(raw["dtype"], tuple(raw["shape"]), begin, end)
            previous = 0
            for info in sorted(entries.values(), key=lambda e: e.begin):
                if info.begin != previous:
                    raise SafetensorsError(f"{path}: safetensors data contains gaps or overlapping tensors.")
                previous = info.end
            if previous != data_size:
                raise SafetensorsError(f"{path}: safetensors data size does not match its header.")
            self.entries = entries
            self._start = 8 + header_size
            # a private mapping: nothing is ever written to it, but tensors may then view its pages directly
            self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_COPY) if size else None
        except Exception:
            self._file.close()
            raise

    def names(self):
        return self.entries.keys()

    def info(self, name: str) -> TensorInfo:
        return self.entries[name]

    def read(self, name: str, copy: bool = True) -> torch.Tensor:
        """The tensor in its stored dtype.  `copy=False`: a view of the file's mapping (no host copy), which
        must be dropped before the file is closed; meant for `view.to(device)` right away."""
        info = self.entries[name]
        _, torch_dtype, np_dtype = _DTYPES[info.dtype]
        count = (info.end - info.begin) // np_dtype.itemsize
        array = np.frombuffer(self._map, dtype=np_dtype, count=count, offset=self._start + info.begin)
        tensor = torch.from_numpy(array.copy() if copy else array)
        if info.dtype == "BF16":
            tensor = tensor.view(torch.bfloat16)
        return tensor.reshape(info.shape)

    def close(self):
        if getattr(self, "_map", None) is not None:
            self._map.close()
            self._map = None
        self._file.close()


def write_safetensors(path: str, tensors: dict[str, torch.Tensor], metadata: dict[str, str] | None = None) -> None:
    """Write `tensors` (CPU, contiguous after .contiguous()) in name order, data packed without gaps."""
    header: dict = {}
    if metadata:
        header["__metadata__"] = metadata
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"Cannot store dtype {t.dtype} of {name!r}.")
        size = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + size]}
        offset += size
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            if t.dtype == torch.bfloat16:
                t = t.view(torch.int16)
            f.write(t.numpy().tobytes())
