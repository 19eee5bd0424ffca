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


def _is_count(value) -> bool:
    return isinstance(value, int) and not isinstance(value, bool)


def _parse_header(path: str, file, size: int) -> tuple[dict, int]:
    """The JSON header of a safetensors file and the number of bytes before the tensor data."""
    lead = file.read(8)
    if len(lead) != 8:
        raise SafetensorsError(f"{path}: {size} bytes are too few for a safetensors file (8 bytes of header length first).")
    (length,) = struct.unpack("<Q", lead)
    if not 0 < length <= MAX_HEADER:
        raise SafetensorsError(f"{path}: a header of {length} bytes is outside 1..{MAX_HEADER}.")
    if 8 + length > size:
        raise SafetensorsError(f"{path}: the header claims {length} bytes, the file has {size - 8} after its first 8.")
    try:
        header = json.loads(file.read(length).decode("utf-8"))
    except (UnicodeDecodeError, json.JSONDecodeError) as error:
        raise SafetensorsError(f"{path}: the header is not JSON ({error}).") from None
    if not isinstance(header, dict):
        raise SafetensorsError(f"{path}: the header is JSON but not an object of tensors.")
    return header, 8 + length


def _tensor_info(path: str, name: str, raw, data_size: int) -> TensorInfo:
    """One header entry, checked by itself: a known dtype, a shape of positive sizes, and a byte range that holds
    exactly that many elements inside the data."""
    if not isinstance(raw, dict):
        raise SafetensorsError(f"{path}: tensor {name!r} is described by {type(raw).__name__}, not by an object.")
    dtype, shape, offsets = raw.get("dtype"), raw.get("shape"), raw.get("data_offsets")
    if dtype not in _DTYPES:
        raise SafetensorsError(f"{path}: tensor {name!r} has dtype {dtype!r}; this reader takes {sorted(_DTYPES)}.")
    if not isinstance(shape, list) or not all(_is_count(n) and n > 0 for n in shape):
        raise SafetensorsError(f"{path}: tensor {name!r} has shape {shape!r}; sizes must be positive integers.")
    if not isinstance(offsets, list) or len(offsets) != 2 or not all(_is_count(n) for n in offsets):
        raise SafetensorsError(f"{path}: tensor {name!r} has data_offsets {offsets!r}; two integers are expected.")
    begin, end = offsets
    nbytes = _DTYPES[dtype][0]
    for n in shape:
        nbytes *= n
    if begin < 0 or end > data_size or end - begin != nbytes:
        raise SafetensorsError(f"{path}: tensor {name!r} ({dtype} {shape}) needs {nbytes} bytes, its range "
                               f"[{begin}, {end}) of {data_size} data bytes does not give them.")
    return TensorInfo(dtype, tuple(shape), begin, end)


def _check_tiling(path: str, entries: dict, data_size: int) -> None:
    """The tensors' ranges, in order, must tile the data: no byte twice, none unaccounted for."""
    at = 0
    for name, info in sorted(entries.items(), key=lambda item: item[1].begin):
        if info.begin != at:
            what = "overlaps its predecessor" if info.begin < at else f"leaves bytes {at}..{info.begin - 1} unused"
            raise SafetensorsError(f"{path}: tensor {name!r} begins at byte {info.begin} and {what}.")
        at = info.end
    if at != data_size:
        raise SafetensorsError(f"{path}: the tensors end at byte {at}, the data at {data_size}.")


class SafetensorsFile:
    """A safetensors file, memory-mapped.  What the header says is checked before any tensor is handed out
    (the checks of the reference's reader, src/safetensors.ts:26-66)."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        self._file = open(path, "rb")
        try:
            header, self._start = _parse_header(path, self._file, size)
            data_size = size - self._start
            self.entries = {name: _tensor_info(path, name, raw, data_size)
                            for name, raw in header.items() if name != "__metadata__"}
            _check_tiling(path, self.entries, data_size)
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
