"""Arrangements of parts in a layer, the embedding and the output head."""
from __future__ import annotations

from typing import Dict

import torch

from ..config.spec import PartSpec
from ..weights.loader import TensorSpec, MATRIX
from .base import Block, Part, NormedInput
from .registry import register_part, build_part


class PreNormBlock(Block):
    """``x += mixer(norm1(x)); x += feed_forward(norm2(x))``; the sums are taken
    in float32 on the float32 residual stream.

    Arrangement: rust/engine/src/runner/model/qwen2/engine.rs:1065-1122 (layer
    loop), 1140-1147 and 1234-1241 (norm before each sublayer)."""

    def __init__(self, hidden_size: int, norm1: PartSpec, mixer: PartSpec, norm2: PartSpec,
                 feed_forward: PartSpec, tensors: Dict[str, str] = None):
        super().__init__(tensors)
        self.hidden_size = int(hidden_size)
        self.norm1 = build_part("norm", norm1)
        self.mixer = build_part("mixer", mixer)
        self.norm2 = build_part("norm", norm2)
        self.feed_forward = build_part("feed_forward", feed_forward)

    def parts(self):
        return [self.norm1, self.mixer, self.norm2, self.feed_forward]

    def mixer_part(self):
        return self.mixer

    def tensor_specs(self):
        specs = {}
        for p in self.parts():
            specs.update(p.tensor_specs())
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        for p in self.parts():
            p.bind(tensors, ops, dtype)

    def forward(self, residual, ctx, entry):
        h = NormedInput(self.norm1, residual, ctx, "block.normed", self.dtype)
        self.mixer.forward(h if self.mixer.takes_normed_input else h.tensor(), residual, ctx, entry)
        h = NormedInput(self.norm2, residual, ctx, "block.normed", self.dtype)
        self.feed_forward.forward(h if self.feed_forward.takes_normed_input else h.tensor(),
                                  residual, ctx)

    def weight_bytes(self):
        return sum(p.weight_bytes() for p in self.parts())


class TokenEmbedding(Part):
    """``x[r] = table[id_r]`` into the float32 residual stream
    (rust/engine/src/runner/model/qwen2/kernels.rs:46-57)."""

    def __init__(self, vocab_size: int, hidden_size: int, tensors: Dict[str, str]):
        super().__init__(tensors)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.table = None

    def tensor_specs(self):
        return {self.tensor_names["weight"]: TensorSpec((self.vocab_size, self.hidden_size), MATRIX)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "embedding (hidden size)")
        # in the order the product kernels read, so that a tied output head shares it
        self.table = ops.prepare_weight(tensors[self.tensor_names["weight"]], shared=True)

    def forward(self, ids, out, ctx=None):
        """``ctx``: the step's batch description, for embeddings that need more than the
        ids (positions, say); this one does not."""
        self.ops.embed(self.table, ids, out)

    def weight_bytes(self):
        return 0     # a step reads one row per token, not the table


class LinearHead(Part):
    """``logits = h W^T`` in float32; ``W`` is the embedding table when the
    names coincide (tied), as in rust/engine/src/runner/model/qwen2/engine.rs:299-303
    and 1312-1319."""

    def __init__(self, vocab_size: int, hidden_size: int, tensors: Dict[str, str]):
        super().__init__(tensors)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight = None

    def tensor_specs(self):
        return {self.tensor_names["weight"]: TensorSpec((self.vocab_size, self.hidden_size), MATRIX)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "output head (hidden size)")
        self.weight = ops.prepare_weight(tensors[self.tensor_names["weight"]], shared=True)

    takes_normed_input = True

    def forward(self, h, out):
        fuse = (isinstance(h, NormedInput) and self.ops.can_fuse(out.shape[0], self.dtype, self.hidden_size, out.shape[1])
                and not self.ops.pieces_too_large_to_read_per_block(getattr(h.ctx, "pending", None)))
        rms = h.rms(accept_pending=True) if fuse else None
        if rms is not None:
            # the last reader of the stream: pieces still owed to it are added on the fly
            pending = getattr(h.ctx, "pending", None)
            self.ops.fused_norm_logits(rms[0], rms[1], rms[2], rms[3], self.weight, out, pending=pending)
            h.ctx.pending = None
        else:
            if isinstance(h, NormedInput):
                h = h.tensor()
            self.ops.linear_logits(h, self.weight, out)

    def weight_bytes(self):
        return self.weight.numel() * self.weight.element_size()


register_part("block", "prenorm", PreNormBlock)
register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
