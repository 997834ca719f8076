"""RMS norm.  y = x / sqrt(mean(x^2) + eps) * w, sums and scale in float32, eps inside the
root, the weight multiplies as it is (src/backends/cpu/x64/kernels.cpp:168-180;
src/backends/cuda/native/common.cuh:57-188)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Norm


class RMSNorm(Norm):
    def __init__(self, size: int, eps: float):
        self.size = size
        self.eps = float(eps)
        self.weight = None

    def weight_specs(self, prefix):
        return [WeightSpec(prefix + ".weight", (self.size,), "norm")]

    def bind(self, prefix, weights):
        self.weight = weights[prefix + ".weight"]

    def capturable(self, batch):
        return True

    def add_norm(self, resid, delta, out_dtype, rows=None):
        return ops.add_rms_norm(resid, delta, self.weight, self.eps, out_dtype, rows)

    def foldable(self, out_dtype):
        if out_dtype == torch.bfloat16 and self.weight is not None and self.weight.dtype == torch.bfloat16:
            return self.weight, self.eps
        return None
