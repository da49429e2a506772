"""A causal language model put together from a ``ModelSpec``.

Nothing here names an architecture: the embedding, the blocks, the final norm
and the head are built from the spec's records through the parts registry, and
the blocks run in the order of ``spec.schedule``.  The reference's counterpart
is a struct written for one architecture
(rust/engine/src/runner/model/qwen2/engine.rs:235-252) whose forward body is
``submit_forward_kernels`` (engine.rs:916-1130).
"""
from __future__ import annotations

import dataclasses
import os
from typing import Dict, List, Optional, Tuple

import torch

from ..cache.manager import CacheManager, GroupLayout
from ..config.spec import ModelSpec
from ..parts.base import NormedInput
from ..parts.registry import build_part, part_class
from ..weights.loader import TensorSpec


@dataclasses.dataclass
class EntryView:
    """What one run of a block sees of the cache manager."""

    index: int                      # position in the schedule
    block: int
    group: Optional[int] = None     # cache group, None if the mixer keeps no cache
    slot: Optional[int] = None      # which of the group's layers
    writes_cache: bool = False
    cache: Dict[str, torch.Tensor] = dataclasses.field(default_factory=dict)   # name -> [pages, *page_shape]
    state: Dict[str, torch.Tensor] = dataclasses.field(default_factory=dict)

    @property
    def k_cache(self) -> Optional[torch.Tensor]:
        """Attention's keys, ``[pages, kv_heads, page_size, head_dim]``."""
        return self.cache.get("k")

    @property
    def v_cache(self) -> Optional[torch.Tensor]:
        """Attention's values, ``[pages, kv_heads, head_dim, page_size]``."""
        return self.cache.get("v")


def _same_pending(a, b) -> bool:
    if a is None or b is None:
        return a is b
    return a.parts.data_ptr() == b.parts.data_ptr() and a.splits == b.splits and a.parts.shape == b.parts.shape


class CausalLM:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.embedding = build_part("embedding", spec.embedding)
        self.blocks = [part_class("block", b.kind)(**dict(b.parts), **dict(b.params)) for b in spec.blocks]
        self.final_norm = build_part("norm", spec.final_norm)
        self.head = build_part("head", spec.head)
        self.entries: List[EntryView] = [EntryView(i, e.block) for i, e in enumerate(spec.schedule)]
        self.ops = None
        self.dtype = None
        self._weight_bytes = None          # worked out when first asked for, after the weights are bound
        self._graph_safe = None
        self.ranges = None         # profiler ranges (engine/profiling.py), off by default
        # Launch sequences of the scheduled runs, kept by the shape of the step: see _run_block.
        self.keep_launches = os.environ.get("LLMLAB_KEEP_LAUNCHES", "1") not in ("0", "")
        self.verify_launches = os.environ.get("LLMLAB_VERIFY_LAUNCHES", "") not in ("0", "")
        self._launches: List[Dict[tuple, object]] = [dict() for _ in self.entries]
        self._launches_version = None      # the scratch buffers' version the kept sequences belong to
        self.launches_recorded = 0
        self.launches_replayed = 0

    def parts(self):
        return [self.embedding, *self.blocks, self.final_norm, self.head]

    @property
    def graph_safe(self) -> bool:
        """Whether a decode step of this model may be replayed from a captured graph."""
        if self._graph_safe is None:            # (asked at every step; the parts say it once)
            self._graph_safe = all(p.graph_safe for p in self.parts())
        return self._graph_safe

    def kernel_libraries(self):
        """What the parts want compiled before they are bound, each once."""
        seen = []
        for p in self.parts():
            for lib in p.kernel_libraries():
                if lib not in seen:
                    seen.append(lib)
        return seen

    # ---------------------------------------------------------------- weights
    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}

        def add(new):
            for name, s in new.items():
                if name in specs and specs[name] != s:
                    raise ValueError(f"tensor '{name}' is asked for with two shapes: "
                                     f"{specs[name]} and {s}")
                specs[name] = s
        add(self.embedding.tensor_specs())
        for b in self.blocks:
            add(b.tensor_specs())
        add(self.final_norm.tensor_specs())
        add(self.head.tensor_specs())
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor], ops, dtype: torch.dtype) -> None:
        self.ops, self.dtype = ops, dtype
        self._weight_bytes = self._graph_safe = None
        self.embedding.bind(tensors, ops, dtype)
        for b in self.blocks:
            b.bind(tensors, ops, dtype)
        self.final_norm.bind(tensors, ops, dtype)
        self.head.bind(tensors, ops, dtype)
        ops.release_shared()

    def weight_bytes_per_step(self) -> int:
        """Bytes of weights that one step reads once (every run of a block reads
        its block's weights; the embedding table is read by rows only)."""
        if self._weight_bytes is None:          # (asked at every decode step: the weights do not change once bound)
            total = sum(self.blocks[e.block].weight_bytes() for e in self.entries)
            self._weight_bytes = total + self.final_norm.weight_bytes() + self.head.weight_bytes()
        return self._weight_bytes

    # ------------------------------------------------------------------ cache
    def cache_layout(self) -> Tuple[List[GroupLayout], Dict[int, dict]]:
        """Groups of cache-owning runs by equal need, and per-run state specs."""
        groups: List[GroupLayout] = []
        by_spec: Dict[object, int] = {}
        state_specs: Dict[int, dict] = {}
        for view, entry in zip(self.entries, self.spec.schedule):
            mixer = self.blocks[entry.block].mixer_part()
            need = mixer.cache_spec()
            if need is not None:
                if entry.cache_of is None:
                    if need not in by_spec:
                        by_spec[need] = len(groups)
                        groups.append(GroupLayout(need, []))
                    view.group = by_spec[need]
                    view.slot = len(groups[view.group].entries)
                    view.writes_cache = True
                    groups[view.group].entries.append(view.index)
                else:
                    owner = self.entries[entry.cache_of]
                    owner_need = self.blocks[self.spec.schedule[entry.cache_of].block].mixer_part().cache_spec()
                    if owner_need != need:
                        raise ValueError(
                            f"schedule[{view.index}] reads the cache of schedule[{entry.cache_of}], "
                            f"whose need {owner_need} differs from its own {need}")
                    view.group, view.slot, view.writes_cache = owner.group, owner.slot, False
            elif entry.cache_of is not None:
                raise ValueError(f"schedule[{view.index}] names a cache but its mixer keeps none")
            st = mixer.state_spec()
            if st:
                state_specs[view.index] = dict(st)
        return groups, state_specs

    def attach_cache(self, cache: CacheManager) -> None:
        for view in self.entries:
            if view.group is not None:
                view.cache = {name: t[view.slot] for name, t in cache.storage[view.group].items()}
            view.state = cache.state.get(view.index, {})

    # ---------------------------------------------------------------- forward
    def forward(self, ctx) -> Optional[torch.Tensor]:
        """Run this step's rows through every scheduled block; returns float32
        logits ``[wanted, vocab]`` for ``ctx.want_rows`` (None if none wanted)."""
        rows, hidden = ctx.n_rows, self.spec.hidden_size
        x = ctx.scratch("model.residual", (rows, hidden), torch.float32)
        ctx.pending = None         # sums a product leaves in pieces for the next reader of x
        if self.ranges is not None:
            return self._forward_with_ranges(x, ctx)
        self.embedding.forward(ctx.token_ids, x, ctx)
        if self._launches_usable(ctx):
            stamp = self._launch_stamp(ctx)
            for view in self.entries:
                self._run_block(self.blocks[view.block], x, ctx, view, stamp)
        else:
            for view in self.entries:
                self.blocks[view.block].forward(x, ctx, view)
        return self._head(x, ctx)

    MAX_KEPT_LAUNCHES = 256       # per scheduled run

    def _launch_stamp(self, ctx) -> tuple:
        """What the kept sequences of this step are filed under, beside the sums owed to the
        stream.  Sequences written down before a scratch buffer moved hold pointers into
        (and keep alive) the buffers of before: they are dropped as soon as that shows."""
        if ctx.scratch_version != self._launches_version:
            for kept in self._launches:
                kept.clear()
            self._launches_version = ctx.scratch_version
        return (ctx.n_rows, ctx.scratch_version, self.ops.fingerprint())

    def _launches_usable(self, ctx) -> bool:
        return (self.keep_launches and hasattr(self.ops, "begin_recording") and hasattr(ctx, "scratch_version")
                and hasattr(ctx, "pending"))

    def _run_block(self, block, x, ctx, view, stamp) -> None:
        """One scheduled run of a block.  Between the host's decision what to launch and the
        launch itself lie shape checks, scratch lookups and argument marshalling that cost
        the host more than the GPU needs for a small model's step.  A block whose parts all
        say ``keeps_launches`` makes the same calls into the kernel libraries whenever the
        step has the same number of rows, the scratch buffers have not moved, the sums
        owed to the stream arrive in the same form and the kernel set's rules are the same;
        so the calls of its first such run are written down (``HipOps.begin_recording``)
        and made again from the list from then on.  Calls that depend on the step's data
        (attention: requests, lengths) are kept as closures and evaluated anew
        (``HipOps.live``).  ``LLMLAB_VERIFY_LAUNCHES=1``: at every replay the block's
        Python code is run as well, without launching, and must make the very same calls.
        The reference's host does this work in compiled code
        (rust/engine/src/runner/model/qwen2/engine.rs:916-1130)."""
        if not block.keeps_launches:
            block.forward(x, ctx, view)
            return
        owed = ctx.pending
        key = stamp + ((owed.parts.data_ptr(), owed.splits, tuple(owed.parts.shape)) if owed is not None else None,)
        kept = self._launches[view.index]
        hit = kept.get(key)
        ops = self.ops
        if hit is not None:
            record, owed_after = hit
            if self.verify_launches:
                again = ops.begin_recording(dry=True)
                try:
                    block.forward(x, ctx, view)
                finally:
                    ops.end_recording()
                if not again.same_as(record) or not _same_pending(ctx.pending, owed_after):
                    raise AssertionError(f"schedule[{view.index}]: the calls kept for steps of {ctx.n_rows} rows "
                                         f"are not the calls its parts would make now")
            ops.replay(record)
            ctx.pending = owed_after
            self.launches_replayed += 1
            return
        record = ops.begin_recording()
        try:
            block.forward(x, ctx, view)
        finally:
            ops.end_recording()
        if ctx.scratch_version == stamp[1]:        # (buffers that moved meanwhile: written down next time)
            if len(kept) >= self.MAX_KEPT_LAUNCHES:
                kept.clear()
            kept[key] = (record, ctx.pending)
            self.launches_recorded += 1

    def _head(self, x, ctx) -> Optional[torch.Tensor]:
        if ctx.n_want == 0:
            ctx.pending = None
            return None
        h = NormedInput(self.final_norm, x, ctx, "model.final_normed", self.dtype,
                        rows=ctx.want_rows, n_rows=ctx.n_want)
        logits = ctx.scratch("model.logits", (ctx.n_want, self.spec.vocab_size), torch.float32)
        self.head.forward(h if getattr(self.head, "takes_normed_input", False) else h.tensor(), logits)
        return logits

    def _forward_with_ranges(self, x, ctx) -> Optional[torch.Tensor]:
        """The same forward with a named range around every part's launches."""
        r = self.ranges
        with r.range("embedding"):
            self.embedding.forward(ctx.token_ids, x, ctx)
        usable = self._launches_usable(ctx)
        stamp = self._launch_stamp(ctx) if usable else None
        for view in self.entries:
            with r.range(f"block {view.index}"):
                if usable:
                    self._run_block(self.blocks[view.block], x, ctx, view, stamp)
                else:
                    self.blocks[view.block].forward(x, ctx, view)
        with r.range("final norm + head"):
            return self._head(x, ctx)
