"""The host-side choices of the matrix products (which tile, how many pieces along the inner
size, which block shape for few rows) are plain functions of the sizes: they run here without
a GPU, over sizes drawn at random, against what every choice must satisfy, and a few
measured decisions are pinned so that a change of a constant shows."""
import ctypes
import random
import shutil

import pytest

from llm_inference_lab_amd.kernels import build

CUS = 256
KINDS = {0: (64, 64), 1: (64, 128), 2: (128, 128), 3: (128, 256), 4: (256, 256), 5: (192, 256)}


@pytest.fixture(scope="module")
def core():
    if shutil.which("hipcc") is None and not build.hipcc_path():
        pytest.skip("no hipcc to build the library with")
    try:
        lib = ctypes.CDLL(build.core_library())
    except (OSError, RuntimeError) as err:
        pytest.skip(f"the core library does not load here: {err}")
    lib.llmlab_linear_tile.restype = ctypes.c_int
    lib.llmlab_linear_plan.restype = None
    lib.llmlab_skinny_shape.restype = None
    return lib


def plan(core, m, n, k, max_pieces=16, min_tiles=8):
    out = (ctypes.c_int * 2)()
    core.llmlab_linear_plan(m, n, k, CUS, max_pieces, min_tiles, out)
    return out[0], out[1]


def test_tile_and_pieces_of_products_of_many_rows(core):
    rng = random.Random(5)
    for _ in range(3000):
        m = rng.choice([rng.randint(1, 64), rng.randint(65, 600), rng.randint(601, 9000)])
        n = rng.randint(1, 60000)
        k = 8 * rng.randint(1, 4000)
        width = core.llmlab_linear_tile(m, n, k, CUS)
        assert width in (64, 128, 256), (m, n, k, width)
        # the tiles of 256 columns are for steps of many rows, and inner sizes they were measured at
        if width == 256:
            assert m >= 512 and k >= 896, (m, n, k)
        pieces, kind = plan(core, m, n, k)
        assert 1 <= pieces <= 16 and kind in KINDS, (m, n, k, pieces, kind)
        if pieces > 1:
            tiles = (k + 63) // 64
            assert (tiles + pieces - 1) // pieces >= 8, (m, n, k, pieces)      # whole K tiles, enough of them
            assert kind != 3, "the 128 x 256 tile of eight waves makes no pieces"
        if kind in (4, 5):
            assert m >= 512 and k >= 896, (m, n, k, kind)


def test_limits_of_the_plan_are_kept(core):
    for max_pieces, min_tiles in ((1, 8), (3, 8), (16, 100), (16, 1)):
        for (m, n, k) in ((40, 3584, 18944), (576, 3584, 18944), (2048, 5120, 27648), (100, 896, 4864)):
            pieces, _ = plan(core, m, n, k, max_pieces, min_tiles)
            assert pieces <= max_pieces
            assert pieces == 1 or ((k + 63) // 64 + pieces - 1) // pieces >= min_tiles


@pytest.mark.parametrize("m,n,k,want", [
    # (measured: see the comments in csrc/gemm.hip)
    (2048, 37888, 3584, (1, 4)),      # gate/up of a 2,048-token step, 7B shape: 256 x 256, two groups of waves
    (2048, 55296, 5120, (1, 4)),
    (576, 3584, 18944, (6, 5)),       # down product of a mixed step: six pieces with the 192 x 256 tile
    (2048, 3584, 18944, (2, 4)),
    (576, 37888, 3584, (1, 5)),       # three tiles of 192 rows
    (2048, 4608, 3584, (1, 5)),
    (576, 1152, 896, (1, 0)),         # a small product: 64 x 64
    (2048, 9728, 896, (1, 5)),        # gate/up of the 0.5B shape
    (2048, 9728, 512, (1, 2)),        # an inner size shorter than any measured: no tile of two groups of waves
])
def test_measured_decisions(core, m, n, k, want):
    assert plan(core, m, n, k) == want


def test_block_shapes_of_products_of_few_rows(core):
    rng = random.Random(6)
    out = (ctypes.c_int * 5)()
    for _ in range(2000):
        epilogue = rng.choice([0, 1, 2, 3, 5])
        m = rng.randint(1, 64)
        n = 16 * rng.randint(1, 9500)
        if epilogue == 3:
            n = 32 * rng.randint(1, 3000)
        k = 8 * rng.randint(1, 3500)
        ksplit = rng.randint(2, 8) if epilogue == 5 else 1
        core.llmlab_skinny_shape(epilogue, int(epilogue in (2, 3) and rng.random() < 0.5), m, n, k, 0, CUS, ksplit, out)
        nsb, kw, stage, qsplit, mb = list(out)
        if nsb == 0:
            continue                                        # no shape fits: the caller takes another kernel
        assert nsb in (1, 2, 4, 8, 16) and kw >= 1 and nsb * kw <= 16, (epilogue, m, n, k, list(out))
        assert mb in (1, 2, 4) and 16 * mb <= max(16, 2 * m), (m, mb)
        assert stage in (0, 1) and qsplit == 1
