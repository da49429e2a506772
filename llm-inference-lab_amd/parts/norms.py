"""Norms."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..weights.loader import TensorSpec, VECTOR, INIT_NORM
from .base import Norm
from .registry import register_part


class RMSNorm(Norm):
    """``y = x * rsqrt(mean(x^2) + eps) * w`` with the square, mean, rsqrt and
    both products in float32 and one rounding to the compute dtype at the end.

    Formula: rust/engine/src/runner/model/qwen2/kernels.rs:546-582 (the
    reference rounds once more, before the weight product; in float32 the two
    are the same).  ``size`` and ``eps`` come from the caller."""

    folds_pending = True
    keeps_launches = True

    def __init__(self, size: int, eps: float, tensors: Dict[str, str]):
        super().__init__(tensors)
        self.size = int(size)
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self):
        return {self.tensor_names["weight"]: TensorSpec((self.size,), VECTOR, INIT_NORM)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        self.weight = tensors[self.tensor_names["weight"]].contiguous()

    def forward(self, x, out, rows=None, pending=None):
        if pending is None:
            self.ops.rmsnorm(x, self.weight, self.eps, out, rows)
        else:
            self.ops.rmsnorm(x, self.weight, self.eps, out, rows, pending=pending)

    def rms_params(self):
        return self.weight, self.eps

    def weight_bytes(self):
        return self.weight.numel() * self.weight.element_size()


register_part("norm", "rmsnorm", RMSNorm)
