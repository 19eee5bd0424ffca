"""Loading a model's tensors by name, with one error that names everything wrong."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .checkpoint import Checkpoint


class WeightError(ValueError):
    """Lists missing tensors, unexpected tensors and wrong shapes of a checkpoint together.

    Tensors that nobody asked for are no error by themselves (the reference reads what it asks for and
    nothing else, src/safetensors.ts:70-83); they are listed when something else is wrong, because a tensor
    that is "missing" and one that is "unexpected" are often the same tensor under two names, and they are
    an error of their own only for a strict load.
    """

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
                       compute: torch.dtype, device, strict: bool = False, notes: list | None = None,
                       before_read=None) -> dict[str, torch.Tensor]:
    """Read exactly the tensors in `expected`, by name, each with the shape its part expects.

    Other tensors in the checkpoint are left unread (a line in `notes` names them); with `strict` they are
    an error unless `ignorable` lists them.  Everything wrong with the checkpoint is reported in one
    WeightError.  `before_read(stored)`: called once the header has been checked and before any tensor is
    read, with the dtype each expected tensor is stored in (the place to count memory)."""
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
        if missing or wrong_shape or wrong_dtype or (strict and unexpected):
            raise WeightError(folder, missing, unexpected, wrong_shape, wrong_dtype)
        if unexpected and notes is not None:
            notes.append(f"{len(unexpected)} tensors of the checkpoint are not part of the model and were left "
                         f"unread: " + ", ".join(unexpected[:8]) + (" ..." if len(unexpected) > 8 else ""))
        stored = {name: ckpt.dtype(name) for name in expected}
        rounded = sorted(n for n, d in stored.items() if d == torch.float16 and compute == torch.bfloat16
                         and expected[n].kind != "int_table")
        if rounded and notes is not None:
            # float32 compute widens float16 exactly (reference: src/safetensors.ts:91-101); bfloat16 compute keeps
            # 16-bit tensors in bfloat16, which has three mantissa bits fewer than float16
            notes.append(f"{len(rounded)} tensors stored in float16 were rounded to bfloat16 for bfloat16 compute: "
                         + ", ".join(rounded[:8]) + (" ..." if len(rounded) > 8 else ""))
        if before_read is not None:
            before_read(stored)
        out = {}
        for name, spec in expected.items():
            # straight from the file's mapping to the device: no copy on the host in between
            view = ckpt.read(name, copy=False)
            kept = view.to(device=device, dtype=target_dtype(view.dtype, spec.kind, compute)).contiguous()
            if kept.data_ptr() == view.data_ptr():
                kept = kept.clone()       # a host tensor of the stored dtype: it must not live in the mapping
            out[name] = kept
            del view
        return out
