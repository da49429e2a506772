"""Interfaces of the parts.

Data flow through a block: the residual stream ``x`` is a float32 tensor
``[rows, hidden]`` (rows = all tokens of the step, packed); a norm reads it and
writes activations in the compute dtype; a mixer or feed-forward reads those
activations and ADDS its result into the residual stream in float32.

Every part states which tensors of the model file it needs (``tensor_specs``),
receives them in ``bind``, and takes its sizes and constants as constructor
arguments.  No part knows which model it is in.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, Optional, Tuple

import torch

from ..weights.loader import TensorSpec


@dataclasses.dataclass(frozen=True)
class PageTensor:
    """One named tensor of a mixer's per-token cache.  ``token_shape`` is what one token
    keeps in it; a page of ``P`` tokens is a tensor of that shape with an axis of length
    ``P`` put in at ``token_axis``.  Keys of ``G`` heads of width ``d`` with
    ``token_axis=1``: pages ``[G, P, d]``; values with ``token_axis=2``: pages ``[G, d, P]``;
    one latent vector of width ``r`` per token with ``token_axis=0``: pages ``[P, r]``.
    ``dtype`` None means the engine's compute dtype."""

    token_shape: Tuple[int, ...]
    token_axis: int = 0
    dtype: Optional[torch.dtype] = None

    def page_shape(self, page_size: int) -> Tuple[int, ...]:
        shape = list(self.token_shape)
        if not 0 <= self.token_axis <= len(shape):
            raise ValueError(f"token_axis {self.token_axis} does not fit the shape {self.token_shape}")
        shape.insert(self.token_axis, int(page_size))
        return tuple(shape)

    def token_elements(self) -> int:
        n = 1
        for s in self.token_shape:
            n *= int(s)
        return n


@dataclasses.dataclass(frozen=True)
class CacheSpec:
    """What a mixer keeps for each token: named tensors in pages.  ``window``: how many
    of the latest positions (the current one included) it ever reads, or ``None`` for
    all.  Mixers with equal specs share one group of pages and one block table; the cache
    manager allocates ``[runs, pages, *page_shape]`` per name and a run of the mixer finds
    its slices in ``entry.cache[name]``."""

    tensors: Tuple[Tuple[str, PageTensor], ...]
    window: Optional[int] = None

    def __post_init__(self):
        names = [n for n, _ in self.tensors]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"a cache spec names at least one tensor, each once: {names}")
        if self.window is not None and self.window <= 0:
            raise ValueError(f"a window holds at least the current position, got {self.window}")

    def bytes_per_token(self, dtype: torch.dtype) -> int:
        return sum(t.token_elements() * torch.empty((), dtype=t.dtype or dtype).element_size()
                   for _, t in self.tensors)


def KVCacheSpec(num_kv_heads: int, head_dim: int, window: Optional[int] = None) -> CacheSpec:
    """The cache of an attention mixer: ``k`` in pages ``[kv_heads, P, head_dim]`` and ``v``
    in pages ``[kv_heads, head_dim, P]`` (values transposed, so that the probability-value
    product reads runs of tokens)."""
    return CacheSpec((("k", PageTensor((int(num_kv_heads), int(head_dim)), 1)),
                      ("v", PageTensor((int(num_kv_heads), int(head_dim)), 2))), window)


class Part:
    """Common base: tensors by role, bound after loading."""

    def __init__(self, tensors: Optional[Dict[str, str]] = None):
        self.tensor_names: Dict[str, str] = dict(tensors or {})
        self.ops = None
        self.dtype = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        """Tensor name in the model file -> expected shape and kind."""
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor], ops, dtype: torch.dtype) -> None:
        """Receive the loaded tensors (by file name), the kernel set and the
        compute dtype.  A part may rearrange its tensors here (fuse, interleave)."""
        self.ops = ops
        self.dtype = dtype

    def weight_bytes(self) -> int:
        """Bytes of weights one forward reads (for roofline accounting)."""
        return 0

    # False: ``forward`` decides something on the host from this step's data (indexes a
    # tensor with a host list, branches on a value) that a replayed graph would freeze.
    # A model with such a part runs its decode steps eagerly even when graphs are asked for.
    graph_safe = True

    def kernel_libraries(self):
        """Kernel libraries to have compiled before the model is bound, as ``(kind,
        parameter)`` pairs that ``kernels.build.library`` knows (``("attention",
        head_dim)``)."""
        return []

    # True: everything ``forward`` does on the GPU goes through the kernel set's entry points,
    # with arguments that depend on nothing but the number of rows of the step, the scratch
    # buffers and the sums owed to the stream; what depends on the step's data beyond that
    # is wrapped in ``ops.live(...)``.  The model may then write the calls of a run down and
    # make them again without running ``forward`` (``CausalLM._run_block``).  False (the
    # default, and right for any part that calls PyTorch or decides on the host from the
    # step's data): ``forward`` runs every time.
    keeps_launches = False


class Norm(Part):
    # True: ``forward(x, out, None, pending=p)`` first makes the stream whole,
    # ``x += sum_s p.parts[s]``, in the same pass (all rows in order only).
    folds_pending = False

    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        """``out[i] = norm(x[rows[i]])`` (all rows in order when ``rows`` is None).
        ``x`` float32, ``out`` compute dtype."""
        raise NotImplementedError

    def rms_params(self):
        """``(weight, eps)`` if this norm is a plain RMSNorm that a following matrix
        product may fold into itself; None otherwise."""
        return None


class PendingSums:
    """Sums that a product left in pieces instead of adding them into the float32
    residual stream: ``parts[s, r, :]`` for ``s < splits`` belongs to row ``r``.
    Whoever reads the stream next adds them on the fly, whoever adds into it next
    folds them in (``HipOps.add_pending`` does it on its own)."""

    __slots__ = ("parts", "splits")

    def __init__(self, parts: torch.Tensor, splits: int):
        self.parts, self.splits = parts, int(splits)


class NormedInput:
    """The input of a mixer, feed-forward or head whose norm has not run yet.

    A consumer that sets ``takes_normed_input = True`` is handed this object
    instead of a tensor.  It may fold the norm into its first kernel
    (``rms()`` gives what that kernel needs) or ask for the normed activations
    with ``tensor()``, which runs the norm once."""

    def __init__(self, norm: Norm, x: torch.Tensor, ctx, name: str, dtype: torch.dtype,
                 rows: Optional[torch.Tensor] = None, n_rows: Optional[int] = None):
        self.norm, self.x, self.ctx, self.name, self.dtype = norm, x, ctx, name, dtype
        self.rows = rows
        self.n_rows = int(n_rows if n_rows is not None else x.shape[0])
        self._tensor: Optional[torch.Tensor] = None

    @property
    def shape(self):
        return (self.n_rows, self.x.shape[1])

    def rms(self, accept_pending: bool = False):
        """``(x, rows, weight, eps)`` for a fused kernel, or None.

        The stream ``x`` may still be owed sums that a former product left in pieces
        (``ctx.pending``).  A caller that passes ``accept_pending=True`` takes that on:
        it hands ``ctx.pending`` to its kernels (which add the pieces while they read
        ``x``, and fold them in where they add into ``x``) and clears it once they
        are folded.  For every other caller the pieces are folded in here."""
        params = self.norm.rms_params()
        if params is None:
            return None
        if not accept_pending:
            self._fold_pending()
        return self.x, self.rows, params[0], params[1]

    def _fold_pending(self) -> None:
        pending = getattr(self.ctx, "pending", None)
        if pending is not None:
            self.norm.ops.add_pending(self.x, pending)
            self.ctx.pending = None

    def tensor(self) -> torch.Tensor:
        if self._tensor is None:
            out = self.ctx.scratch(self.name, (self.n_rows, self.x.shape[1]), self.dtype)
            pending = getattr(self.ctx, "pending", None)
            if pending is not None and self.rows is None and self.norm.folds_pending:
                self.norm.forward(self.x, out, None, pending=pending)     # folded in by the norm itself
                self.ctx.pending = None
            else:
                self._fold_pending()
                self.norm.forward(self.x, out, self.rows)
            self._tensor = out
        return self._tensor


class PositionEncoding(Part):
    def rotary_table(self) -> Optional[torch.Tensor]:
        """``inv_freq [rotary_dim/2]`` float32 if this is a split-half rotation
        that the fused projection epilogue can apply; None otherwise."""
        return None

    def apply(self, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor) -> None:
        """Encode positions into ``q [rows, heads, dim]`` and ``k`` in place."""
        raise NotImplementedError


class Mixer(Part):
    takes_normed_input = False     # True: ``forward`` gets a ``NormedInput`` and may fuse the norm

    def cache_spec(self) -> Optional[CacheSpec]:
        """Per-token cache need (``KVCacheSpec(...)`` for keys and values, or any
        ``CacheSpec`` of named page tensors), or None."""
        return None

    def state_spec(self) -> Dict[str, Tuple[Tuple[int, ...], torch.dtype]]:
        """Fixed-size per-request state: name -> (shape, dtype).  The cache
        manager keeps ``[max_requests, *shape]`` per name, zeroed at admission."""
        return {}

    def forward(self, h: torch.Tensor, residual: torch.Tensor, ctx, entry) -> None:
        """``residual += mixer(h)``; ``h`` are the normed activations of this
        step's rows, ``ctx`` the step's batch description, ``entry`` this run's
        cache and state (``EntryView``)."""
        raise NotImplementedError


class FeedForward(Part):
    takes_normed_input = False

    def forward(self, h: torch.Tensor, residual: torch.Tensor, ctx) -> None:
        """``residual += feed_forward(h)``."""
        raise NotImplementedError


class Block(Part):
    def parts(self):
        """The parts this block is made of (for tensor lists and binding)."""
        raise NotImplementedError

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self.parts())

    @property
    def keeps_launches(self):
        return all(p.keeps_launches for p in self.parts())

    def kernel_libraries(self):
        return [lib for p in self.parts() for lib in p.kernel_libraries()]

    def mixer_part(self) -> Mixer:
        raise NotImplementedError

    def forward(self, residual: torch.Tensor, ctx, entry) -> None:
        raise NotImplementedError
