"""Feed-forward parts."""
from __future__ import annotations

from typing import Dict

import torch

from ..weights.loader import TensorSpec, MATRIX
from .base import FeedForward, NormedInput
from .registry import register_part

PAIR = 16   # rows of the gate matrix and of the up matrix alternate in runs of 16


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Stack gate ``[I, K]`` and up ``[I, K]`` as ``[2*ceil16(I), K]``: rows
    ``32b .. 32b+15`` are gate rows ``16b .. 16b+15`` and rows ``32b+16 ..
    32b+31`` the up rows of the same outputs, so one 16-column tile of the
    product holds gate and the next one up for the same 16 outputs (rows past
    ``I`` are zero)."""
    inter, k = gate.shape
    padded = (inter + PAIR - 1) // PAIR * PAIR
    out = torch.zeros((2 * padded, k), dtype=gate.dtype, device=gate.device)
    view = out.view(padded // PAIR, 2, PAIR, k)
    g = torch.zeros((padded, k), dtype=gate.dtype, device=gate.device)
    u = torch.zeros((padded, k), dtype=gate.dtype, device=gate.device)
    g[:inter] = gate
    u[:inter] = up
    view[:, 0] = g.view(padded // PAIR, PAIR, k)
    view[:, 1] = u.view(padded // PAIR, PAIR, k)
    return out


class SwiGLU(FeedForward):
    """``residual += (silu(h Wg^T) * (h Wu^T)) Wd^T`` with ``silu(z) = z / (1 +
    exp(-z))``; accumulators, the sigmoid and the product in float32.

    Formula: rust/engine/src/runner/model/qwen2/engine.rs:1234-1294,
    rust/engine/src/runner/model/qwen2/kernels.rs:1469-1486."""

    def __init__(self, hidden_size: int, intermediate_size: int, tensors: Dict[str, str],
                 activation: str = "silu"):
        super().__init__(tensors)
        if activation != "silu":
            raise ValueError(f"SwiGLU supports activation 'silu', got '{activation}'")
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.w_gate_up = self.w_down = None

    def tensor_specs(self):
        t, h, i = self.tensor_names, self.hidden_size, self.intermediate_size
        return {
            t["gate_weight"]: TensorSpec((i, h), MATRIX),
            t["up_weight"]: TensorSpec((i, h), MATRIX),
            t["down_weight"]: TensorSpec((h, i), MATRIX),
        }

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "feed-forward (hidden size)")
        ops.check_product_sizes(self.intermediate_size, dtype, "feed-forward (intermediate size)")
        t = self.tensor_names
        self.w_gate_up = ops.prepare_weight(
            interleave_gate_up(tensors[t["gate_weight"]], tensors[t["up_weight"]]))
        self.w_down = ops.prepare_weight(tensors[t["down_weight"]].contiguous())

    takes_normed_input = True
    keeps_launches = True

    def forward(self, h, residual, ctx):
        rows = h.shape[0]
        act = ctx.scratch("swiglu.act", (rows, self.intermediate_size), self.dtype)
        fuse = isinstance(h, NormedInput) and self.ops.can_fuse(rows, self.dtype, self.hidden_size,
                                                                 self.w_gate_up.shape[0])
        rms = h.rms() if fuse else None      # (folds pieces still owed to the stream; else the norm does)
        if rms is not None:
            self.ops.fused_norm_swiglu(rms[0], rms[2], rms[3], self.w_gate_up, act)
        else:
            if isinstance(h, NormedInput):
                h = h.tensor()
            self.ops.linear_swiglu(h, self.w_gate_up, act)
        splits = self.ops.split_count(rows, self.dtype, self.hidden_size, self.intermediate_size)
        if splits > 1 and hasattr(ctx, "pending") and ctx.pending is None:
            # a narrow output: the product is cut along the inner size so that it spreads
            # over the chip, and its pieces are left for the next reader of the stream
            parts = ctx.scratch("swiglu.pieces", (splits, rows, self.hidden_size), torch.float32)
            ctx.pending = self.ops.linear_partials(act, self.w_down, parts, splits)
        else:
            self.ops.linear_residual(act, self.w_down, residual, None)

    def weight_bytes(self):
        return sum(w.numel() * w.element_size() for w in (self.w_gate_up, self.w_down))


register_part("feed_forward", "swiglu", SwiGLU)
