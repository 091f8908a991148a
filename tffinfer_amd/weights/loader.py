"""Matching the tensors of a file against what a model expects."""
from __future__ import annotations

import torch

from ..parts.base import WeightSpec


class WeightError(ValueError):
    """The tensors found do not fit the model: lists every missing tensor,
    every unexpected one and every wrong shape or type in one message."""

    def __init__(self, missing, unexpected, wrong_shape, wrong_dtype, where=""):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = [f"weights{' in ' + where if where else ''} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, want, got in self.wrong_shape:
            lines.append(f"  wrong shape: {name}: expected {list(want)}, found {list(got)}")
        for name, got in self.wrong_dtype:
            lines.append(f"  unsupported type: {name}: {got} (float32, bfloat16 or float16)")
        super().__init__("\n".join(lines))


_FLOATS = (torch.float32, torch.bfloat16, torch.float16)


def check_weights(expected: dict[str, WeightSpec], found: dict[str, torch.Tensor],
                  ignorable: set[str] = frozenset(), where: str = "") -> None:
    """Raises one WeightError naming everything that is wrong."""
    missing = [n for n in expected if n not in found]
    unexpected = [n for n in found if n not in expected and n not in ignorable]
    wrong_shape = [(n, expected[n].shape, tuple(found[n].shape)) for n in expected
                   if n in found and tuple(found[n].shape) != tuple(expected[n].shape)]
    wrong_dtype = [(n, found[n].dtype) for n in expected if n in found and found[n].dtype not in _FLOATS]
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightError(sorted(missing), sorted(unexpected), wrong_shape, wrong_dtype, where)


def normalize_stored(t: torch.Tensor) -> torch.Tensor:
    """The type a tensor is kept in on the host: bfloat16, except that a tensor
    stored in 32 bits stays so (float16 is widened to float32 rather than
    re-rounded to bfloat16's shorter mantissa); integer tables become int32."""
    if t.dtype in (torch.bfloat16, torch.float32):
        return t
    if t.dtype == torch.float16:
        return t.to(torch.float32)
    if t.dtype in (torch.int64, torch.int16, torch.int8, torch.uint8, torch.int32):
        return t.to(torch.int32)
    return t
