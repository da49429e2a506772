"""Position encodings."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import PositionEncoding
from .registry import register_part


class RotaryEmbedding(PositionEncoding):
    """Split-half rotation: with ``lo = x[:d/2]``, ``hi = x[d/2:]`` and
    ``angle_i = position * theta^(-2i/d)``, the result is ``[lo*cos - hi*sin,
    hi*cos + lo*sin]``; angles, sines and cosines in float32.

    Formula: rust/engine/src/runner/model/qwen2/kernels.rs:587-631; frequency
    table: rust/engine/src/runner/model/qwen2/engine.rs:304-306."""

    def __init__(self, dim: int, theta: float, tensors: Optional[Dict[str, str]] = None):
        super().__init__(tensors)
        if dim % 2:
            raise ValueError(f"rotary dimension {dim} must be even")
        self.dim = int(dim)
        self.theta = float(theta)
        self.inv_freq: Optional[torch.Tensor] = None

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        exponent = torch.arange(0, self.dim, 2, dtype=torch.float64) / self.dim
        self.inv_freq = (1.0 / (torch.tensor(self.theta, dtype=torch.float64) ** exponent)
                         ).to(torch.float32).to(ops.device)

    keeps_launches = True      # (the frequency table goes to the kernels; ``apply`` depends on the rows only)

    def rotary_table(self):
        return self.inv_freq

    def apply(self, q, k, positions):
        self.ops.rope_inplace(q, positions, self.inv_freq)
        self.ops.rope_inplace(k, positions, self.inv_freq)


class NoPosition(PositionEncoding):
    """No position encoding: queries and keys are used as projected."""

    keeps_launches = True

    def __init__(self, tensors: Optional[Dict[str, str]] = None, **_):
        super().__init__(tensors)

    def apply(self, q, k, positions):
        return None


register_part("position", "rope", RotaryEmbedding)
register_part("position", "none", NoPosition)
