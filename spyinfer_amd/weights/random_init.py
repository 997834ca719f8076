"""Random-weights mode: write a model folder (config.json, model.safetensors)
from a configuration and a seed.

Every tensor is drawn from its own stream keyed by (seed, tensor name), so the
values do not depend on the order of tensors or on other tensors' shapes:
matrices ~ N(0, matrix_std), norm scales ~ norm_mean + N(0, norm_std), biases and
other vectors centred on zero ~ N(0, bias_std), integer tables uniform.  The folder is then read back by name like any other model.
The reference has no such mode.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Iterable

import torch

from .loader import WeightSpec
from .safetensors_io import write_file


ROLES = ("matrix", "norm", "bias", "table")


def _stream(seed: int, name: str) -> torch.Generator:
    digest = hashlib.sha256(("%d:%s" % (seed, name)).encode()).digest()
    g = torch.Generator(device="cpu")
    g.manual_seed(int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF)
    return g


def random_tensors(specs: Iterable[WeightSpec], seed: int, dtype: torch.dtype = torch.bfloat16,
                   matrix_std: float = 0.02, norm_mean: float = 1.0, norm_std: float = 0.01,
                   table_range: int = 2, bias_std: float = 0.02) -> Dict[str, torch.Tensor]:
    out = {}
    for s in specs:
        if s.optional:
            continue
        if s.role not in ROLES:
            raise ValueError("tensor %s has the role %r; known roles: %s" % (s.name, s.role, ", ".join(ROLES)))
        g = _stream(seed, s.name)
        if s.role == "table":
            out[s.name] = torch.randint(0, table_range, s.shape, generator=g, dtype=torch.int32)
        elif s.role == "norm":
            out[s.name] = (norm_mean + norm_std * torch.randn(s.shape, generator=g, dtype=torch.float32)).to(dtype)
        elif s.role == "bias":
            out[s.name] = (bias_std * torch.randn(s.shape, generator=g, dtype=torch.float32)).to(dtype)
        else:
            # big matrices are filled in row blocks to bound the float32 staging memory
            t = torch.empty(s.shape, dtype=dtype)
            rows = s.shape[0] if len(s.shape) > 1 else 1
            flat = t.view(rows, -1)
            step = max(1, (1 << 24) // max(1, flat.shape[1]))
            for r in range(0, rows, step):
                n = min(step, rows - r)
                flat[r:r + n] = (matrix_std * torch.randn((n, flat.shape[1]), generator=g, dtype=torch.float32)).to(dtype)
            out[s.name] = t
    return out


def random_tensors_on_device(specs: Iterable[WeightSpec], seed: int, dtype: torch.dtype, device,
                             matrix_std: float = 0.02, norm_mean: float = 1.0, norm_std: float = 0.0,
                             bias_std: float = 0.02) -> Dict[str, torch.Tensor]:
    """Random weights made on the device itself, for measurements at sizes whose files would take
    minutes to write and read.  Same distributions as ``random_tensors``, other values."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    out = {}
    for s in specs:
        if s.optional:
            continue
        if s.role == "table":
            out[s.name] = torch.randint(0, 2, s.shape, generator=g, dtype=torch.int32, device=device)
        elif s.role == "norm":
            out[s.name] = (norm_mean + norm_std * torch.randn(s.shape, generator=g, dtype=torch.float32, device=device)).to(dtype)
        elif s.role == "bias":
            out[s.name] = (bias_std * torch.randn(s.shape, generator=g, dtype=torch.float32, device=device)).to(dtype)
        else:
            t = torch.empty(s.shape, dtype=dtype, device=device)
            t.normal_(0.0, matrix_std, generator=g)
            out[s.name] = t
    return out


def write_random_model(folder: str, config: dict, seed: int, dtype: torch.dtype = torch.bfloat16, **init) -> str:
    """``config`` is the config.json content (with ``architectures``).  Returns ``folder``."""
    from ..config.registry import architecture_of

    arch = architecture_of(config)
    cfg = arch.config_cls.from_dict(config)
    model = arch.build(cfg)
    os.makedirs(folder, exist_ok=True)
    tensors = random_tensors(model.weight_specs(), seed, dtype, **init)
    write_file(os.path.join(folder, "model.safetensors"), tensors, {"format": "pt", "seed": str(seed)})
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f, indent=1)
    return folder
