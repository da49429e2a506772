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
        # the tiles of 256 columns are for steps of many rows (of a wide matrix: from 129 on),
        # and inner sizes they were measured at
        if width == 256:
            one_tile = 64 < m <= 128 and 32768 <= n <= 65536 and k >= 1024      # (the 128 x 256 tile of eight waves)
            assert ((m >= 512 or (m > 128 and n >= 16384)) and k >= 896) or one_tile, (m, n, k)
        pieces, kind = plan(core, m, n, k)
        assert 1 <= pieces <= 16 and kind in KINDS, (m, n, k, pieces, kind)
        if pieces > 1:
            tiles = (k + 63) // 64
            assert (tiles + pieces - 1) // pieces >= 8, (m, n, k, pieces)      # whole K tiles, enough of them
            assert kind != 3, "the 128 x 256 tile of eight waves makes no pieces"
        if kind in (4, 5):
            assert (m >= 512 or (m > 128 and n >= 16384 and pieces == 1)) and k >= 896, (m, n, k, kind)


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
    (192, 55296, 5120, (1, 5)),       # one or two tiles of rows of a wide matrix already fill the chip:
    (256, 55296, 5120, (1, 4)),       # the tiles of two groups of waves (153 / 171 us against 187 / 199)
    (384, 27648, 5120, (1, 5)),
    (192, 27648, 5120, (1, 1)),       # ... not where half the units would stay idle
    (192, 4608, 3584, (1, 0)),        # 216 blocks of 64 x 64 are one round (26 us against 29 with 64 x 128),
    (1536, 896, 896, (1, 1)),         # 336 are two: 64 x 128 (11.5 us against 13.3)
    (384, 5120, 27648, (4, 2)),       # three tiles of 128 rows in four pieces (150 us against 183 in two of 64 x 128)
    (256, 8192, 8192, (4, 2)),
    (192, 5120, 27648, (4, 1)),       # ... from 256 rows on (a step of 192 requests of the 32B shape loses 5 % with them)
    (272, 5120, 27648, (2, 1)),       # ... and only well-filled tiles
])
def test_measured_decisions(core, m, n, k, want):
    assert plan(core, m, n, k) == want


def test_one_tile_of_rows_of_a_wide_matrix(core):
    """65 to 128 rows: the tile of a product that does not add into the stream (gate and up, the
    logits), measured inside decode steps of 96 and 128 requests."""
    assert core.llmlab_linear_tile(128, 37888, 3584, CUS) == 256      # 128 x 256: 77 us against 84
    assert core.llmlab_linear_tile(96, 55296, 5120, CUS) == 256
    assert core.llmlab_linear_tile(128, 152064, 3584, CUS) == 128     # a vocabulary gains nothing from it
    assert core.llmlab_linear_tile(128, 27648, 5120, CUS) == 128
    assert core.llmlab_linear_tile(64, 37888, 3584, CUS) == 128       # (64 x 128)


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


def test_when_a_decode_graph_pays():
    """``graph="auto"``: the rule on measured cases.  At the 0.5B shape (151 calls a step, 1 GB
    of weights) the host cannot keep up and the graph is taken, also with 3.2 GB of cache
    behind 64 requests; at the 7B and 32B shapes the step streams for longer than the host
    needs and is launched call by call; a small model behind a very long context is no
    longer misjudged by its weights alone."""
    from llm_inference_lab_amd.kernels.debug import DispatchRules
    rules = DispatchRules()
    assert rules.graph_pays(151, 0.988e9, 0.4e9)
    assert rules.graph_pays(151, 0.988e9, 3.2e9)
    assert not rules.graph_pays(171, 14.1e9, 1.9e9)
    assert not rules.graph_pays(387, 64.0e9, 17e9)
    assert rules.graph_pays(151, 0.988e9, 0.0) and not rules.graph_pays(151, 0.988e9, 12e9)


def test_the_engine_counts_a_decode_step_and_decides_step_by_step():
    """Over the kernel references on the CPU: the first decode step of ``graph="auto"`` runs
    eagerly and its calls are counted; what the rules are asked is the number of calls, the
    weights of one step and the cache that the step's requests hold at that moment, at
    every decode step anew.  (The rules here always say no: a CPU has no graphs.)"""
    import helpers as H
    import llm_inference_lab_amd as lab
    from emu_ops import EmuOps
    from llm_inference_lab_amd.kernels.debug import DispatchRules

    class Asked(DispatchRules):
        def __init__(self):
            super().__init__()
            self.questions = []

        def graph_pays(self, calls, weight_bytes, cache_bytes):
            self.questions.append((calls, weight_bytes, cache_bytes))
            return False

    ops = EmuOps()
    ops.rules = Asked()
    engine = H.make_engine("B", 1, "f32", ops=ops, device="cpu", graph="auto", num_pages=24)
    cfg = H.config_of("B")
    a, b = engine.open("a"), engine.open("b")
    engine.step([lab.StepEntry(a, H.random_ids(cfg, 30, 1), [29]), lab.StepEntry(b, H.random_ids(cfg, 7, 2), [6])])
    assert engine.step_fn.decode_calls is None and ops.rules.questions == []      # a prefill step decides nothing
    before = ops.calls_made
    engine.step([lab.StepEntry(a, [1], [0]), lab.StepEntry(b, [2], [0])])
    calls = ops.calls_made - before
    assert engine.step_fn.decode_calls == calls > 0 and engine.step_fn.use_graph is False
    engine.step([lab.StepEntry(a, [3], [0]), lab.StepEntry(b, [4], [0])])
    engine.step([lab.StepEntry(a, [5], [0])])
    assert [q[0] for q in ops.rules.questions] == [calls] * 3
    assert all(q[1] == engine.model.weight_bytes_per_step() for q in ops.rules.questions)
    # config B: one layer sees everything, two see the last 24 positions; 1 kv head of 32, float32
    per_token = 2 * 32 * 4
    seen = lambda n: per_token * (n + 2 * min(n, 24))
    assert [q[2] for q in ops.rules.questions] == [seen(31) + seen(8), seen(32) + seen(9), seen(33)]


# ----------------------------------------------------------------- attention
def attention_library(head_dim):
    if shutil.which("hipcc") is None and not build.hipcc_path():
        pytest.skip("no hipcc to build the library with")
    try:
        lib = ctypes.CDLL(build.attention_library(head_dim))
    except (OSError, RuntimeError) as err:
        pytest.skip(f"the attention library does not load here: {err}")
    lib.llmlab_attention_launch.restype = ctypes.c_int
    return lib


BF16, F32 = 1, 0        # (the dtype codes of the libraries)


@pytest.mark.parametrize("head_dim,nq,nkv", [(64, 14, 2), (128, 28, 4), (256, 8, 8)])
def test_attention_launch_is_one_the_head_size_has(head_dim, nq, nkv):
    """Over steps drawn at random: a decode step is told apart, the launches with two groups of
    waves and with 32 rows a wave only where the head size has them, pairs of tiles only at the
    start of prompts without a window."""
    lib = attention_library(head_dim)
    rng = random.Random(head_dim)
    group = nq // nkv
    for _ in range(3000):
        reqs = rng.choice([1, 2, 4, 8, 16, 64])
        q = rng.choice([1, 2, 3, rng.randint(4, 64), rng.randint(65, 4096)])
        ctx = q + rng.choice([0, rng.randint(0, 300), rng.randint(0, 9000)])
        window = rng.choice([0, 0, 0, 128, 4096])
        for dtype in (BF16, F32):
            path = lib.llmlab_attention_launch(dtype, nq, nkv, reqs, q, ctx, window, CUS)
            if q * group <= 16:
                assert path == 0, (q, path)
                continue
            if dtype == F32:
                assert path in (1, 2), (reqs, q, ctx, path)
                continue
            assert path in (1, 2, 3, 4, 6), (reqs, q, ctx, path)
            if head_dim > 128:
                assert path in (1, 3, 4)
            if path == 3:
                assert window == 0 and 16 * (ctx - q) <= q
            if path == 1:
                assert -(-q * group // 64) * nkv * reqs <= CUS // 2       # few tiles of rows only


@pytest.mark.parametrize("head_dim,nq,nkv,dtype,reqs,q,behind,want", [
    # (measured: see the comments in csrc/attention.hip; 1 = a block's waves split the keys of a tile of
    # rows, 2 = 32 rows a wave, 4 = 16 rows a wave, 6 = 4 with two groups of waves a block)
    (64, 14, 2, BF16, 1, 512, 1536, 1),      # a portion behind a history: 19 us against 32
    (64, 14, 2, BF16, 1, 512, 256, 6),
    (64, 14, 2, BF16, 1, 2048, 0, 6),        # a prompt from its start: 32 us against 38
    (64, 14, 2, BF16, 1, 8192, 0, 2),        # a long one: 221 against 235
    (64, 14, 2, BF16, 16, 64, 0, 4),         # many short prompts: 6.8 us against 8.0
    (64, 14, 2, BF16, 8, 512, 2048, 2),      # 75 us against 83
    (64, 14, 2, BF16, 2, 4096, 0, 4),        # 132 us against 161
    (128, 28, 4, BF16, 1, 128, 1024, 6),     # 25 us against 29 with the key split
    (128, 28, 4, BF16, 1, 128, 2560, 1),
    (128, 28, 4, BF16, 8, 128, 0, 2),        # 14 us against 19
    (128, 28, 4, BF16, 1, 64, 0, 4),         # 8.4 us against 9.8
    (128, 28, 4, BF16, 1, 2048, 4096, 6),    # 313 us against 374 to 470
    (64, 14, 2, F32, 1, 512, 1024, 1),       # 43 us against 162
    (64, 14, 2, F32, 1, 2048, 0, 1),         # 117 against 217
    (64, 14, 2, F32, 16, 512, 0, 2),         # 137 against 187
    (128, 28, 4, F32, 4, 256, 0, 2),         # 58 against 81
    (128, 28, 4, F32, 1, 256, 1024, 1),      # 77 against 226
    (128, 28, 4, F32, 1, 1024, 0, 1),        # a long portion's tiles are uneven: 148 against 184
    (128, 28, 4, F32, 2, 1024, 1024, 1),     # 620 against 656
    (128, 28, 4, F32, 4, 1024, 0, 2),        # 501 against 562
])
def test_measured_attention_launches(head_dim, nq, nkv, dtype, reqs, q, behind, want):
    lib = attention_library(head_dim)
    assert lib.llmlab_attention_launch(dtype, nq, nkv, reqs, q, behind + q, 0, CUS) == want


@pytest.mark.parametrize("head_dim,nq,nkv,portion,behind,decoding,their_keys,want", [
    # (measured, one launch against two: see the comment in llmlab_paged_attention)
    (64, 14, 2, 128, 2048, 63, 2048, 1),     # 28 us against 38
    (64, 14, 2, 256, 1024, 31, 1024, 1),     # 21 against 27
    (64, 14, 2, 512, 1536, 31, 1024, 1),     # 31 against 34
    (64, 14, 2, 512, 1536, 127, 1024, 2),    # 70 against 63
    (64, 14, 2, 512, 1536, 63, 512, 2),      # 43 against 40
    (128, 28, 4, 128, 2048, 63, 2048, 1),    # 75 against 88
    (128, 40, 8, 128, 2048, 127, 1024, 1),   # 145 against 164
    (128, 28, 4, 512, 512, 63, 2048, 2),     # (the portion's launch is not the one with the key split)
])
def test_measured_launches_of_a_mixed_step(head_dim, nq, nkv, portion, behind, decoding, their_keys, want):
    lib = attention_library(head_dim)
    lib.llmlab_attention_mixed_launches.restype = ctypes.c_int
    got = lib.llmlab_attention_mixed_launches(nq, nkv, decoding + 1, decoding, portion, behind + portion,
                                              their_keys, 0, CUS)
    assert got == want
    # not a mixed step: nobody decodes, or everybody
    assert lib.llmlab_attention_mixed_launches(nq, nkv, 4, 0, portion, behind + portion, 0, 0, CUS) == 0
    assert lib.llmlab_attention_mixed_launches(nq, nkv, 4, 4, portion, behind + portion, their_keys, 0, CUS) == 0
