"""Seeded random weights for a model, and writing them as a model folder.

Values come from a counter generator keyed by (seed, tensor name, element index): element i of a tensor is a
function of those three alone, so a tensor is the same whether it is drawn on the host or on the GPU, whole or in
pieces, and the plain implementation of the tests, which reads the folder, sees what an engine that draws its
weights on the device computes with.  (The reference draws random weights only for its offline fixture,
scripts/reference.py:17,55-62.)

    h_j = mix(key + (3 i + j) * 0x9E3779B97F4A7C15), j = 0, 1, 2      key: 64 bits of sha256("seed:name")
    s   = the sum of the twelve 16-bit fields of h_0, h_1, h_2       (mean 6 * 65535, deviation 65536)
    x   = float32(s - 393210) * float32(std / 65536) (+ 1 for norm weights)

The device twin of `fill_numpy` is csrc/random_fill.hip; a GPU test holds the two to bit equality.
"""
from __future__ import annotations

import hashlib
import json
import os

import numpy as np
import torch

from .loader import TensorSpec
from .safetensors_io import write_safetensors

INIT_STD = 0.02
_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1, _M2 = np.uint64(0xBF58476D1CE4E5B9), np.uint64(0x94D049BB133111EB)
_CHUNK = 1 << 22


def key_for(seed: int, name: str) -> int:
    """The 64-bit key of tensor `name` under `seed`."""
    return int.from_bytes(hashlib.sha256(f"{seed}:{name}".encode()).digest()[:8], "little")


def _mix(x: np.ndarray) -> np.ndarray:
    x ^= x >> np.uint64(30); x *= _M1
    x ^= x >> np.uint64(27); x *= _M2
    x ^= x >> np.uint64(31)
    return x


def fill_numpy(key: int, n: int, scale: float, offset: float | None = None, first: int = 0) -> np.ndarray:
    """float32 values of elements first .. first + n - 1 of the tensor keyed `key`."""
    out = np.empty(n, dtype=np.float32)
    scale32 = np.float32(scale)
    with np.errstate(over="ignore"):
        for start in range(0, n, _CHUNK):
            count = min(_CHUNK, n - start)
            base = np.uint64(3) * (np.arange(count, dtype=np.uint64) + np.uint64(first + start))
            total = np.zeros(count, dtype=np.int64)
            for j in range(3):
                h = _mix(np.uint64(key) + (base + np.uint64(j)) * _GOLDEN)
                for shift in (0, 16, 32, 48):
                    total += ((h >> np.uint64(shift)) & np.uint64(0xFFFF)).astype(np.int64)
            x = (total - 393210).astype(np.float32) * scale32
            if offset is not None:
                x = x + np.float32(offset)
            out[start:start + count] = x
    return out


def random_tensors(expected: dict[str, TensorSpec], seed: int, dtype: torch.dtype = torch.float32,
                   device="cpu", std: float = INIT_STD) -> dict[str, torch.Tensor]:
    """One tensor per name from the counter generator keyed by (seed, name): the same values on every device.

    Matrices and biases are near N(0, std); norm weights are 1 + that; integer tables are not
    random-initialised by any part here and raise.  Values are float32, then rounded to `dtype`.
    """
    on_gpu = torch.device(device).type == "cuda"
    if on_gpu:
        from .. import ops
    out = {}
    scale = np.float32(std / 65536.0)
    for name, spec in expected.items():
        if spec.kind == "int_table":
            raise ValueError(f"No random initialisation for integer table {name!r}.")
        offset = 1.0 if spec.init == "one_plus_normal" else None
        if on_gpu:
            t = torch.empty(spec.shape, dtype=dtype, device=device)
            ops.random_fill(t, key_for(seed, name), float(scale), offset)
        else:
            n = int(np.prod(spec.shape, dtype=np.int64))
            t = torch.from_numpy(fill_numpy(key_for(seed, name), n, float(scale), offset)).reshape(spec.shape).to(dtype)
        out[name] = t
    return out


def write_model_folder(folder: str, config, seed: int, dtype: torch.dtype = torch.bfloat16,
                       std: float = INIT_STD, device=None) -> None:
    """Write config.json and model.safetensors of a randomly initialised model of `config`.  `device`: where the
    values are drawn (the same values either way; a GPU draws a large model in a moment, and is taken when there
    is one)."""
    from ..registry import build_model_plan
    if device is None:
        device = torch.device("cuda", torch.cuda.current_device()) if torch.cuda.is_available() else "cpu"
    os.makedirs(folder, exist_ok=True)
    plan = build_model_plan(config)
    tensors = random_tensors(plan.expected_tensors(), seed, dtype=dtype, std=std, device=device)
    tensors = {name: t.cpu() for name, t in tensors.items()}
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=2)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": str(seed)})
