"""The debug interface of the kernel set: the one place through which a choice that the
kernels make for themselves can be fixed from outside.

The product never calls it.  Tests do, to reach every kernel variant at small sizes (the
chooser would pick one tile per size, tiny matrices would never be cut along their inner
size), and measurements do, to compare variants.

Two kinds of choices:

* ``DispatchRules`` (``HipOps.rules``): the measured thresholds by which ``HipOps`` picks a
  path from the shape of a product.  One object, every field with its product value and
  what it was measured on.
* forced kernel shapes (``HipOps.debug.force(...)``, a context manager that restores on
  exit): the tile of the tiled products, the block shape of the few-row products, the
  number of key splits of decode attention, the number of pieces of a product cut by the
  tiled kernel.  These are process-wide switches inside the kernel libraries
  (``llmlab_debug_*`` entry points), so two ``HipOps`` in one process share them.
"""
from __future__ import annotations

import contextlib
import dataclasses
from typing import Optional, Tuple


@dataclasses.dataclass
class DispatchRules:
    # Fused norm + product kernels beyond one tile of 16 rows: only while the matrix, read
    # once per tile of rows, stays below this many bytes in all (else norm + tiled product
    # wins: 64 rows of a 55 MB matrix take 38 us fused, 26 us in two kernels).
    fuse_read_bytes: float = 128e6
    # Beyond 64 rows the few-row kernels (tiles of 16 rows, a block per tile and set of columns)
    # still take a product, up to this many rows, while the matrix times the tiles stays below
    # so many bytes: every tile streams the matrix for itself, and the tiles of a step that run
    # at the same time miss the caches together.  Measured inside decode steps of 96 / 128 /
    # 192 / 256 / 320 requests of the 0.5B shape (q/k/v and output product, 2 MB each): 1.88 ->
    # 1.64, 1.98 -> 1.76, 2.23 -> 2.14, 2.48 -> 2.41 ms, no difference from 320 on; of the 1.5B
    # shape (6 MB) 3.04 -> 2.80 and 3.29 -> 3.06 at 96 and 128; 2560 x 2048 (10 MB) at 128 rows
    # takes 23 us so and 17 through pieces.  Steps of 512-token portions beside decoding
    # requests lose 7 % with a limit of 1024 rows and nothing with 256.
    few_rows_max: int = 256
    few_rows_read_bytes: float = 64e6
    # From 17 rows on, a matrix of this many bytes that adds into the stream is cut along its
    # inner size by the tiled kernel: the few-row kernel reads it once per tile of 16 rows
    # (64 rows of 3584 x 18944: 89 us against 34; of 1536 x 8960: 25 against 13).
    tiled_pieces_bytes: float = 16e6
    # Pieces beyond this many bytes are folded once by a kernel of their own instead of being
    # added on the fly by every block of a fused kernel (32 rows of width 3584 in 7 pieces,
    # 3.2 MB: 12 us a layer more in the fused kernels; 8 rows of width 5120 in 3 pieces, 491 KB:
    # a decode step of the 14B shape 7.82 -> 7.56 ms folded once, of the 32B shape 16.03 ->
    # 15.97; 4 rows of the same, 246 KB: 6.70 -> 6.83, and the 115 to 131 KB of the 0.5B to 3B
    # shapes at 8 rows 3 to 7 % slower folded once).
    pieces_per_block_bytes: int = 400_000
    # A piece of a few-row product has at least this many K steps of 32 ...
    min_steps_per_split: int = 8
    # ... and of a many-row product this many K tiles of 64.
    min_tiles_per_split: int = 8
    # A few-row product of more strips than compute units is cut along its inner size when
    # the last round of its blocks would leave the chip this much slower than even rounds
    # (1.25 rounds of blocks take the time of 2: a waste of 1.6).
    uneven_rounds_waste: float = 1.3
    # q/k/v of this many rows up to 64 goes through pieces when the matrix is a large one
    # (64 rows of 7168 x 5120: 26 us against 52 with a head per block; slower below 24 rows).
    qkv_pieces_min_rows: int = 24
    # Debug only: a product that the tiled kernel cuts gets this many pieces whatever the
    # estimate says (0: the estimate decides).
    forced_tiled_pieces: int = 0
    # ``graph="auto"`` (engine/step.py): what one call into the kernel libraries costs the
    # host that makes it through ctypes, and the rate at which a decode step streams its
    # weights and its cache.  A decode step replayed from a HIP graph costs the host
    # nothing, but the GPU about a microsecond more at every kernel boundary than kernels
    # launched one by one by a host that runs ahead (measured: 4.05 against 3.90 ms a step
    # at the 7B shape, 17.3 against 16.9 at the 32B shape; 0.97 against 1.7 at the 0.5B
    # shape, where the host cannot keep up).
    host_seconds_per_call: float = 12e-6
    streamed_bytes_per_second: float = 4.2e12
    # the graph is taken unless the GPU's time outlasts the host's by this factor
    graph_host_margin: float = 1.25

    def graph_pays(self, calls: int, weight_bytes: float, cache_bytes: float) -> bool:
        """Whether a decode step of ``calls`` library calls that reads ``weight_bytes`` of
        weights and ``cache_bytes`` of cache should be replayed from a graph: yes, unless
        the GPU's streaming clearly outlasts the host's making of the calls."""
        host = calls * self.host_seconds_per_call
        gpu = (weight_bytes + cache_bytes) / self.streamed_bytes_per_second
        return gpu < self.graph_host_margin * host


class KernelDebug:
    def __init__(self, ops):
        self._ops = ops

    @contextlib.contextmanager
    def force(self, *, gemm_tile: Optional[int] = None,
              skinny_shape: Optional[Tuple[int, int, int, int]] = None,
              skinny_epilogue: Optional[int] = None,
              attention_splits: Optional[Tuple[int, int]] = None,
              attention_path: Optional[Tuple[int, int]] = None,
              attention_merge_kernel: Optional[int] = None,
              attention_merge_in_place: Optional[int] = None, attention_two_launches: Optional[int] = None,
              attention_one_launch: Optional[int] = None,
              f32_fma: Optional[bool] = None, **rules):
        """``gemm_tile``: 64 (64 x 64), 130 (64 x 128), 129 (128 x 128), 131 (128 x 256), 132 (256 x
        256) or 133 (192 x 256); -131: the choice among the first three; -256 and below: the
        tiles of two groups of waves (132, 133) from so many rows on.  ``skinny_shape``:
        (strips per block, K slices, staged rows 0/1 or -1, rows per tile) of the few-row
        product kernel, 0 = chosen by the kernel.  ``skinny_epilogue``: the force holds for
        this epilogue only.  ``attention_splits``: (head size, key splits of the decode
        launch).  ``attention_path``: (head size, launch of a step of many rows: 1 = the waves of a
        block split the keys of a tile of 32 rows, 2 = tiles of 32 rows per wave, 3 = late and
        early tiles in pairs, 4 = tiles of 16 rows per wave, 5 and 6 = 3 and 4 with two groups of
        waves that take the staged keys in turn; heads above 128 have no 5 and 6 and choose
        for themselves).  ``attention_merge_kernel`` / ``attention_merge_in_place``: a head size; the
        key splits of decode attention are merged there by the kernel of its own, or by the
        last block to arrive, whatever their number.  ``attention_two_launches`` / ``attention_one_launch``:
        a head size; a mixed step's decoding requests and its portions get a launch each also
        where one launch would serve both, or one launch wherever there is a kernel for both.
        ``f32_fma``: float32 products of many rows by the plain FMA kernel instead of the
        matrix cores.  Other keywords: fields of ``DispatchRules`` for the time of the block."""
        ops = self._ops
        core = ops._core
        saved = dataclasses.replace(ops.rules)
        for key, value in rules.items():
            if not hasattr(ops.rules, key):
                raise TypeError(f"no dispatch rule named '{key}'")
            setattr(ops.rules, key, value)
        lib = plib = mlib = tlib = None
        ops.debug_epoch += 1
        try:
            if attention_merge_kernel is not None:
                mlib = ops._attention_lib(int(attention_merge_kernel))
                mlib.llmlab_debug_attention_merge_kernel(1)
            elif attention_merge_in_place is not None:
                mlib = ops._attention_lib(int(attention_merge_in_place))
                mlib.llmlab_debug_attention_merge_kernel(-1)
            if attention_two_launches is not None:
                tlib = ops._attention_lib(int(attention_two_launches))
                tlib.llmlab_debug_attention_two_launches(1)
            elif attention_one_launch is not None:
                tlib = ops._attention_lib(int(attention_one_launch))
                tlib.llmlab_debug_attention_two_launches(-1)
            if attention_path is not None:
                plib = ops._attention_lib(int(attention_path[0]))
                plib.llmlab_debug_attention_path(int(attention_path[1]))
            if gemm_tile is not None:
                core.llmlab_debug_gemm_tile(int(gemm_tile))
            if f32_fma is not None:
                core.llmlab_debug_f32_fma(1 if f32_fma else 0)
            if skinny_shape is not None:
                core.llmlab_debug_skinny_shape(*[int(v) for v in skinny_shape])
            if skinny_epilogue is not None:
                core.llmlab_debug_skinny_epilogue(int(skinny_epilogue))
            if attention_splits is not None:
                lib = ops._attention_lib(int(attention_splits[0]))
                lib.llmlab_debug_attention_splits(int(attention_splits[1]))
            yield ops
        finally:
            ops.debug_epoch += 1
            ops.rules = saved
            if gemm_tile is not None:
                core.llmlab_debug_gemm_tile(0)
            if f32_fma is not None:
                core.llmlab_debug_f32_fma(0)
            if skinny_shape is not None:
                core.llmlab_debug_skinny_shape(0, 0, -1, 0)
            if skinny_epilogue is not None:
                core.llmlab_debug_skinny_epilogue(-1)
            if lib is not None:
                lib.llmlab_debug_attention_splits(0)
            if plib is not None:
                plib.llmlab_debug_attention_path(0)
            if mlib is not None:
                mlib.llmlab_debug_attention_merge_kernel(0)
            if tlib is not None:
                tlib.llmlab_debug_attention_two_launches(0)
