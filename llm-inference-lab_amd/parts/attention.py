"""Attention mixers."""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..config.spec import PartSpec
from ..weights.loader import TensorSpec, MATRIX, VECTOR
from .base import Mixer, KVCacheSpec, NormedInput
from .registry import register_part, build_part


class GQAAttention(Mixer):
    """Grouped-query attention over a paged cache.

    ``q = h Wq^T + bq`` (and k, v alike; float32 accumulate, bias added in
    float32), position encoding on q and k, keys and values of the new
    positions written to the cache before the scores are taken, so a step's
    tokens see themselves and each other causally; head ``h`` reads kv head
    ``h // (num_heads / num_kv_heads)``; scores ``q.k * scale`` over the keys
    ``max(0, p - window + 1) .. p`` of the query at position ``p``, softmax and
    the weighted sum of values in float32; then ``residual += attn Wo^T``.

    Formulas: projections rust/engine/src/runner/model/qwen2/engine.rs:1133-1210,
    cache write engine.rs:1072-1082, scores/softmax
    rust/engine/src/runner/model/qwen2/kernels.rs:702-853, output projection and
    residual engine.rs:1225-1233.  The window is not in the reference (it
    rejects ``use_sliding_window``, engine.rs:262)."""

    takes_normed_input = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[PartSpec], tensors: Dict[str, str], qkv_bias: bool = True,
                 out_bias: bool = False, window: Optional[int] = None,
                 scale: Optional[float] = None):
        super().__init__(tensors)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.qkv_bias = bool(qkv_bias)
        self.out_bias = bool(out_bias)
        self.window = None if window is None else int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.position = build_part("position", position) if position is not None else None
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None

    # sizes
    @property
    def q_size(self):
        return self.num_heads * self.head_dim

    @property
    def kv_size(self):
        return self.num_kv_heads * self.head_dim

    def tensor_specs(self):
        t, h = self.tensor_names, self.hidden_size
        specs = {
            t["q_weight"]: TensorSpec((self.q_size, h), MATRIX),
            t["k_weight"]: TensorSpec((self.kv_size, h), MATRIX),
            t["v_weight"]: TensorSpec((self.kv_size, h), MATRIX),
            t["o_weight"]: TensorSpec((h, self.q_size), MATRIX),
        }
        if self.qkv_bias:
            specs[t["q_bias"]] = TensorSpec((self.q_size,), VECTOR)
            specs[t["k_bias"]] = TensorSpec((self.kv_size,), VECTOR)
            specs[t["v_bias"]] = TensorSpec((self.kv_size,), VECTOR)
        if self.out_bias:
            specs[t["o_bias"]] = TensorSpec((h,), VECTOR)
        if self.position is not None:
            specs.update(self.position.tensor_specs())
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_attention_sizes(self.num_heads, self.num_kv_heads, self.head_dim, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "attention projections (hidden size)")
        ops.check_product_sizes(self.q_size, dtype, "attention output projection (heads * head size)")
        t = self.tensor_names
        # One projection instead of three: the rows of Wq, Wk, Wv stacked.
        self.w_qkv = ops.prepare_weight(torch.cat([tensors[t["q_weight"]], tensors[t["k_weight"]],
                                                   tensors[t["v_weight"]]], dim=0).contiguous())
        if self.qkv_bias:
            parts = [tensors[t["q_bias"]], tensors[t["k_bias"]], tensors[t["v_bias"]]]
            kept = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
            self.b_qkv = torch.cat([p.to(kept) for p in parts]).contiguous()
        self.w_o = ops.prepare_weight(tensors[t["o_weight"]].contiguous())
        self.b_o = tensors[t["o_bias"]].contiguous() if self.out_bias else None
        if self.position is not None:
            self.position.bind(tensors, ops, dtype)

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window)

    def forward(self, h, residual, ctx, entry):
        ops = self.ops
        rows = h.shape[0]
        table = self.position.rotary_table() if self.position is not None else None
        group = ctx.group(entry.group)
        k_cache = entry.k_cache if entry.writes_cache else None
        v_cache = entry.v_cache if entry.writes_cache else None
        fuse = (isinstance(h, NormedInput) and ops.can_fuse(rows, self.dtype, self.hidden_size, self.q_size + 2 * self.kv_size)
                and (self.position is None or table is not None)
                and not ops.pieces_too_large_to_read_per_block(getattr(ctx, "pending", None)))
        rms = h.rms(accept_pending=True) if fuse else None
        pending = None
        if rms is not None:
            # few rows: norm, the three projections, bias, rotation and the cache
            # write are one kernel
            q = ctx.scratch("attention.q", (rows, self.q_size), self.dtype)
            # pieces still owed to the stream are added as its rows are read, and folded
            # in by the output projection below
            pending = getattr(ctx, "pending", None)
            ops.fused_norm_qkv(rms[0], rms[2], rms[3], self.w_qkv, self.b_qkv, self.num_heads,
                               self.num_kv_heads, self.head_dim, table, ctx.positions, ctx.row_req,
                               group.block_table, group.page_size, k_cache, v_cache, q, pending=pending)
        elif (ops.can_fuse_qkv_rope(rows, self.dtype, self.head_dim, self.q_size + 2 * self.kv_size,
                                    self.hidden_size)
              and (self.position is None or table is not None)):
            # more rows: the norm on its own, then one kernel for the rest
            if isinstance(h, NormedInput):
                h = h.tensor()
            q = ctx.scratch("attention.q", (rows, self.q_size), self.dtype)
            ops.qkv_rope_cache(h, self.w_qkv, self.b_qkv, self.num_heads, self.num_kv_heads,
                               self.head_dim, table, ctx.positions, ctx.row_req, group.block_table,
                               group.page_size, k_cache, v_cache, q)
        else:
            if isinstance(h, NormedInput):
                h = h.tensor()
            q = ctx.scratch("attention.qkv", (rows, self.q_size + 2 * self.kv_size), self.dtype)
            ops.linear(h, self.w_qkv, q, self.b_qkv)
            if self.position is not None and table is None:
                qv = q[:, :self.q_size].unflatten(1, (self.num_heads, self.head_dim))
                kv = q[:, self.q_size:self.q_size + self.kv_size].unflatten(
                    1, (self.num_kv_heads, self.head_dim))
                self.position.apply(qv, kv, ctx.positions[:rows])
            ops.rope_kv_write(q, self.num_heads, self.num_kv_heads, self.head_dim, table,
                              ctx.positions, ctx.row_req, group.block_table, group.page_size,
                              k_cache, v_cache)
        out = ctx.scratch("attention.out", (rows, self.q_size), self.dtype)

        prepare = getattr(ops, "prepare_attention", None)
        prepared = []

        def attend():
            # (how many requests, how long their portions and their histories are: read from
            # the step's description when the launch is made, also when it is made again
            # from a kept sequence of calls; what stays the same then is checked once)
            if prepare is None:
                ops.paged_attention(
                    q, self.num_heads, self.num_kv_heads, self.head_dim,
                    entry.k_cache, entry.v_cache, group.block_table, group.page_size,
                    ctx.q_start, ctx.start_pos, ctx.n_reqs, ctx.max_q_len, ctx.max_ctx_len,
                    self.window, self.scale, out, self._short_requests(ctx))
                return
            if not prepared:
                prepared.append(prepare(
                    q, self.num_heads, self.num_kv_heads, self.head_dim, entry.k_cache, entry.v_cache,
                    group.block_table, group.page_size, getattr(ctx, "all_q_start", ctx.q_start),
                    getattr(ctx, "all_start_pos", ctx.start_pos), self.window, self.scale, out, ctx.row_req))
            prepared[0].launch(ctx.n_reqs, ctx.max_q_len, ctx.max_ctx_len, self._short_requests(ctx))
        live = getattr(ops, "live", None)
        if live is not None:
            live(attend)
        else:
            attend()
        if pending is not None:
            ops.linear_residual(out, self.w_o, residual, self.b_o, pending=pending)
            ctx.pending = None
            return
        splits = 1
        if getattr(ctx, "pending", 0) is None and ops.pieces_by_tiles(rows, self.hidden_size, self.q_size):
            splits = ops.split_count(rows, self.dtype, self.hidden_size, self.q_size)
        if splits > 1:
            # some rows of a large matrix: cut along the inner size, the pieces left for the
            # norm that reads the stream next
            parts = ctx.scratch("attention.pieces", (splits, rows, self.hidden_size), torch.float32)
            ctx.pending = ops.linear_partials(out, self.w_o, parts, splits, self.b_o)
        else:
            ops.linear_residual(out, self.w_o, residual, self.b_o)

    def _short_requests(self, ctx):
        """Which of the step's requests bring only a few tokens (the kernels serve those by
        another launch than the portions of prompts); worked out once per step, kept in
        the step's notes for the other layers."""
        limit = self.ops.attention_short_limit(self.num_heads, self.num_kv_heads, self.dtype, ctx.max_q_len)
        if limit <= 0:
            return None
        key = ("attention.short", limit)
        if key not in ctx.memo:
            count = longest = 0
            for b in range(ctx.n_reqs):
                n = ctx.host_q_start[b + 1] - ctx.host_q_start[b]
                if n <= limit:
                    count += 1
                    longest = max(longest, ctx.host_start_pos[b] + n)
            ctx.memo[key] = (ctx.row_req, limit, count, longest) if 0 < count < ctx.n_reqs else None
        return ctx.memo[key]

    @property
    def keeps_launches(self):
        return self.position is None or self.position.keeps_launches

    def kernel_libraries(self):
        return [("attention", self.head_dim)]

    def weight_bytes(self):
        total = 0
        for w in (self.w_qkv, self.b_qkv, self.w_o, self.b_o):
            if w is not None:
                total += w.numel() * w.element_size()
        return total


register_part("mixer", "gqa_attention", GQAAttention)
