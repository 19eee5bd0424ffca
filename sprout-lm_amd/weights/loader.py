"""Loading a model's tensors by name, with one error that names everything wrong."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .checkpoint import Checkpoint


class WeightError(ValueError):
    """Lists missing tensors, unexpected tensors and wrong shapes of a checkpoint together."""

    def __init__(self, folder, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.wrong_dtype = list(wrong_shape), list(wrong_dtype)
        lines = [f"Checkpoint {folder!r} does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, want, got in self.wrong_shape:
            lines.append(f"  shape mismatch for {name}: expected {list(want)}, got {list(got)}")
        for name, got in self.wrong_dtype:
            lines.append(f"  unsupported dtype for {name}: {got}")
        super().__init__("\n".join(lines))


@dataclass(frozen=True)
class TensorSpec:
    """What a part expects of one tensor.

    kind: "matrix" (a contraction operand), "vector" (norm weights, biases) or
    "int_table" (integer tables, kept as int32).
    """

    shape: tuple[int, ...]
    kind: str = "matrix"
    init: str = "normal"  # random-weights mode: "normal" = N(0, std), "one_plus_normal" = 1 + N(0, std)


def target_dtype(stored: torch.dtype, kind: str, compute: torch.dtype) -> torch.dtype:
    """The dtype a tensor is kept in on the device.

    float32 compute widens everything to float32 (exactly).  bfloat16 compute
    keeps 16-bit tensors in bfloat16 and leaves a tensor stored in 32-bit as
    it is; integer tables become int32.
    """
    if kind == "int_table":
        return torch.int32
    if compute == torch.float32:
        return torch.float32
    if stored == torch.float32:
        return torch.float32
    return torch.bfloat16


def load_named_tensors(folder: str, expected: dict[str, TensorSpec], ignorable: set[str],
                       compute: torch.dtype, device) -> dict[str, torch.Tensor]:
    """Read exactly the tensors in `expected`; anything else in the checkpoint must be in `ignorable`."""
    with Checkpoint(folder) as ckpt:
        present = set(ckpt.names())
        missing = sorted(n for n in expected if n not in present)
        unexpected = sorted(n for n in present if n not in expected and n not in ignorable)
        wrong_shape, wrong_dtype = [], []
        for name, spec in expected.items():
            if name not in present:
                continue
            info = ckpt.info(name)
            if tuple(info.shape) != tuple(spec.shape):
                wrong_shape.append((name, spec.shape, info.shape))
            is_int = info.dtype in ("I32", "I64")
            if is_int != (spec.kind == "int_table"):
                wrong_dtype.append((name, info.dtype))
        if missing or unexpected or wrong_shape or wrong_dtype:
            raise WeightError(folder, missing, unexpected, wrong_shape, wrong_dtype)
        out = {}
        for name, spec in expected.items():
            t = ckpt.read(name)
            out[name] = t.to(device=device, dtype=target_dtype(t.dtype, spec.kind, compute)).contiguous()
        return out
