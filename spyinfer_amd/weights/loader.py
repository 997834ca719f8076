"""Weights by tensor name.

A model lists the tensors it needs as ``WeightSpec``s (full safetensors name,
shape, role).  ``load_weights`` reads exactly those from a model folder, checks
every one, and raises ONE error that lists all missing tensors, all unexpected
ones and all wrong shapes.  (The reference fails on the first missing name with
an anonymous ``out_of_range`` from ``map.at``, src/utils/weight_reader.hpp:19-22,
ignores extra tensors and checks no shape.)

Storage policy: floating tensors are kept in bfloat16 for a bfloat16 run and
widened (exactly) to float32 for a float32 run; a tensor stored in 32-bit float
stays float32 in both; integer tables become int32.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, Iterable, List, Optional, Tuple

import torch

from .safetensors_io import open_folder


@dataclasses.dataclass(frozen=True)
class WeightSpec:
    name: str
    shape: Tuple[int, ...]
    #: "matrix" (projection / embedding), "norm" (scale vector centred on 1), "bias" (vector centred on 0),
    #: "table" (integer table); the role decides how the random-weights mode draws the tensor
    role: str = "matrix"
    #: names whose presence is tolerated but not read (a tied head stored again)
    optional: bool = False


class WeightError(ValueError):
    """Lists every problem found in a model folder at once."""

    def __init__(self, folder, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = ["weights in %s do not fit the model:" % folder]
        if self.missing:
            lines.append("  missing tensors (%d): %s" % (len(self.missing), ", ".join(self.missing)))
        if self.unexpected:
            lines.append("  unexpected tensors (%d): %s" % (len(self.unexpected), ", ".join(self.unexpected)))
        for name, want, got in self.wrong_shape:
            lines.append("  wrong shape: %s expected %s, found %s" % (name, list(want), list(got)))
        for name, got in self.wrong_dtype:
            lines.append("  wrong dtype: %s is stored as %s" % (name, got))
        super().__init__("\n".join(lines))


def storage_dtype(stored: torch.dtype, run_dtype: torch.dtype, role: str) -> torch.dtype:
    if role == "table":
        return torch.int32
    if stored == torch.float32 or run_dtype == torch.float32:
        return torch.float32
    return torch.bfloat16


def load_weights(folder: str, specs: Iterable[WeightSpec], run_dtype: torch.dtype,
                 device: Optional[torch.device] = None) -> Dict[str, torch.Tensor]:
    specs = list(specs)
    files = open_folder(folder)
    where = {}
    for f in files:
        for name in f.names():
            where[name] = f
    want = {s.name: s for s in specs}
    missing = [s.name for s in specs if s.name not in where and not s.optional]
    unexpected = sorted(n for n in where if n not in want)
    wrong_shape, wrong_dtype = [], []
    for s in specs:
        if s.name not in where:
            continue
        dt, shape = where[s.name].info(s.name)
        if tuple(shape) != tuple(s.shape):
            wrong_shape.append((s.name, s.shape, shape))
        if s.role == "table":
            if dt.is_floating_point or dt == torch.bool:
                wrong_dtype.append((s.name, str(dt)))
        elif not dt.is_floating_point:
            wrong_dtype.append((s.name, str(dt)))
    if missing or unexpected or wrong_shape or wrong_dtype:
        for f in files:
            f.close()
        raise WeightError(folder, missing, unexpected, wrong_shape, wrong_dtype)
    out = {}
    for s in specs:
        if s.name not in where or s.optional:
            continue
        t = where[s.name].tensor(s.name)
        target = storage_dtype(t.dtype, run_dtype, s.role)
        if device is not None and torch.device(device).type != "cpu":
            t = t.to(device=device, dtype=target, non_blocking=False)
        else:
            t = t.to(dtype=target).clone() if t.dtype == target else t.to(dtype=target)
        out[s.name] = t.contiguous()
    for f in files:
        f.close()
    return out
