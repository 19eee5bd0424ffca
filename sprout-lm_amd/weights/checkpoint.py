"""A model folder's tensors, in one file or in shards (reference: src/weight-files.ts:6-52)."""
from __future__ import annotations

import json
import os
import re
from collections import OrderedDict

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile, TensorInfo

_SHARD_NAME = re.compile(r"^[a-zA-Z0-9_-][a-zA-Z0-9_.-]*\.safetensors$")
MAX_OPEN_SHARDS = 8


class Checkpoint:
    """Name -> tensor lookup over `model.safetensors` or `model.safetensors.index.json`."""

    def __init__(self, folder: str):
        self.folder = os.path.abspath(folder)
        self._open: "OrderedDict[str, SafetensorsFile]" = OrderedDict()
        index_path = os.path.join(self.folder, "model.safetensors.index.json")
        self._infos: dict[str, tuple[str, TensorInfo]] = {}
        if os.path.exists(index_path):
            with open(index_path) as f:
                index = json.load(f)
            mapping = index.get("weight_map") if isinstance(index, dict) else None
            if not isinstance(mapping, dict) or not mapping:
                raise SafetensorsError("Invalid safetensors weight map.")
            for shard in mapping.values():
                if not isinstance(shard, str) or not _SHARD_NAME.match(shard):
                    raise SafetensorsError(f"Invalid checkpoint shard filename {shard!r}.")
            for shard in sorted(set(mapping.values())):
                file = self._file(shard)
                for name in file.names():
                    if mapping.get(name) == shard:
                        self._infos[name] = (shard, file.info(name))
            absent = sorted(n for n in mapping if n not in self._infos)
            if absent:
                raise SafetensorsError(f"The shard index of {self.folder!r} names {len(absent)} tensors that their shards "
                                       f"do not hold: " + ", ".join(absent[:8]) + (" ..." if len(absent) > 8 else ""))
        else:
            single = os.path.join(self.folder, "model.safetensors")
            if not os.path.exists(single):
                raise SafetensorsError(f"No model.safetensors or model.safetensors.index.json in {self.folder!r}.")
            file = self._file("model.safetensors")
            for name in file.names():
                self._infos[name] = ("model.safetensors", file.info(name))

    def _file(self, shard: str) -> SafetensorsFile:
        file = self._open.get(shard)
        if file is not None:
            self._open.move_to_end(shard)
            return file
        if len(self._open) >= MAX_OPEN_SHARDS:
            _, oldest = self._open.popitem(last=False)
            oldest.close()
        file = SafetensorsFile(os.path.join(self.folder, shard))
        self._open[shard] = file
        return file

    def names(self):
        return self._infos.keys()

    def info(self, name: str) -> TensorInfo:
        return self._infos[name][1]

    def dtype(self, name: str) -> torch.dtype:
        """The torch dtype `name` is stored in."""
        from .safetensors_io import stored_dtype
        return stored_dtype(self._infos[name][1].dtype)

    def read(self, name: str, copy: bool = True) -> torch.Tensor:
        """`copy=False`: a view of the file's mapping, to be used before the next tensor is read."""
        shard, _ = self._infos[name]
        return self._file(shard).read(name, copy)

    def close(self):
        for file in self._open.values():
            file.close()
        self._open.clear()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
