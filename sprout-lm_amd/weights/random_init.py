"""Seeded random weights for a model, and writing them as a model folder."""
from __future__ import annotations

import hashlib
import json
import os

import torch

from .loader import TensorSpec
from .safetensors_io import write_safetensors

INIT_STD = 0.02


def _seed_for(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") >> 1


def random_tensors(expected: dict[str, TensorSpec], seed: int, dtype: torch.dtype = torch.float32,
                   device="cpu", std: float = INIT_STD) -> dict[str, torch.Tensor]:
    """One tensor per name, each from its own generator keyed by (seed, name).

    Matrices and biases are N(0, std); norm weights are 1 + N(0, std); integer
    tables are not random-initialised by any part here and raise.
    Values are drawn in float32 and then rounded to `dtype`.
    """
    out = {}
    for name, spec in expected.items():
        if spec.kind == "int_table":
            raise ValueError(f"No random initialisation for integer table {name!r}.")
        gen = torch.Generator(device=device)
        gen.manual_seed(_seed_for(seed, name))
        t = torch.empty(spec.shape, dtype=torch.float32, device=device).normal_(0.0, std, generator=gen)
        if spec.init == "one_plus_normal":
            t += 1.0
        out[name] = t.to(dtype)
    return out


def write_model_folder(folder: str, config, seed: int, dtype: torch.dtype = torch.bfloat16,
                       std: float = INIT_STD) -> None:
    """Write config.json and model.safetensors of a randomly initialised model of `config`."""
    from ..registry import build_model_plan
    os.makedirs(folder, exist_ok=True)
    plan = build_model_plan(config)
    tensors = random_tensors(plan.expected_tensors(), seed, dtype=dtype, std=std)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=2)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": str(seed)})
