"""Logits at real shapes with every dispatch rule at its product value: the whole
Qwen2.5-0.5B shape (24 layers, the real vocabulary), and one layer each at the widths of
Qwen2.5-7B (3584, 28/4 heads of 128, 18944) and Qwen2.5-32B (5120, 40/8, 27648), where the
rules for large matrices decide which kernels run (products cut along the inner size by
the tiled kernel, pieces folded by the norm, q/k/v through pieces, four waves per decode
block at head size 128).  No threshold is touched; the tests assert through the kernel
set's own predicates that those rules fire at these sizes.

The reference checks a real checkpoint whole against chunked below 1e-3 and 64
teacher-forced steps split against unsplit (rust/engine/src/runner/model/qwen2/engine.rs:
4359-4442, 4444-4758).

Tolerances, set before the first run on the GPU.  float32: 1e-3 against the float64 plain
implementation.  bfloat16: half as much again as the floor that rounding at the engine's
own rounding points sets at each shape, measured on the CPU with the emulation of the
kernels (tests/emu_ops.py: float32 arithmetic, the same roundings) on these sequences:
24 layers of the 0.5B shape 0.227 at most and 0.0335 in the root mean square (logits of
root mean square 1.6); one layer at the 7B widths 0.071 / 0.0112; at the 32B widths
0.078 / 0.0135."""
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

TOL = {"F": {"f32": (1e-3, 1e-3), "bf16": (0.34, 0.050)},
       "W7": {"f32": (1e-3, 1e-3), "bf16": (0.107, 0.0168)},
       "W32": {"f32": (1e-3, 1e-3), "bf16": (0.117, 0.0203)}}
CUTS = {"whole": H.steps_whole, "decode": H.steps_prefill_then_decode, "portions": H.steps_portions,
        "mixed": H.steps_mixed}
LENGTHS = {"F": ([44, 61, 80, 52], 1200), "W7": ([3, 75, 140, 330, 512], 1300),
           "W32": ([3, 75, 140, 330, 512], 1400)}


def sequences_of(name):
    cfg = H.config_of(name)
    lengths, seed = LENGTHS[name]
    return {f"r{i}": H.random_ids(cfg, n, seed + i) for i, n in enumerate(lengths)}


def check(name, dtype, got, want, seqs):
    worst, rms_limit = TOL[name][dtype]
    bad = H.first_wrong(got, want, worst)
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
    err = torch.cat([(got[r].double() - want[r])[~torch.isnan(got[r]).any(1)].flatten() for r in seqs])
    rms = float((err ** 2).mean().sqrt())
    assert rms <= rms_limit, f"root mean square error {rms} > {rms_limit}"


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("cut", ["whole", "mixed"])
def test_full_depth_at_the_half_billion_shape(dtype, cut):
    seqs = sequences_of("F")
    want = {rid: H.plain_logits("F", 1, ids) for rid, ids in seqs.items()}
    engine = H.make_engine("F", 1, dtype, page_size=64, num_pages=7, max_requests=4, max_batch_tokens=512)
    got = H.run_trace(engine, seqs, CUTS[cut](seqs))
    check("F", dtype, got, want, seqs)
    engine.cache.check()


def assert_large_matrix_rules_fire(ops, cfg):
    """At these widths the rules that the tiny and the 0.5B-wide tests can only force."""
    bf = torch.bfloat16
    h, inter = cfg.hidden_size, cfg.intermediate_size
    q = cfg.num_attention_heads * cfg.head_dim
    qkv = q + 2 * cfg.num_key_value_heads * cfg.head_dim
    # some rows of a large matrix: the product into the stream is cut by the tiled kernel ...
    assert ops.pieces_by_tiles(26, h, inter) and ops.pieces_by_tiles(64, h, q) and not ops.pieces_by_tiles(8, h, inter)
    assert ops.split_count(26, bf, h, inter) > 1 and ops.split_count(64, bf, h, q) > 1
    # ... while a step of one tile of rows has strips enough for the chip: 224 strips on 256
    # units are not cut, 320 strips (1.25 rounds of blocks) are cut in three (3.75 rounds) ...
    assert ops.split_count(8, bf, h, inter) == {3584: 1, 5120: 3}[h]
    # ... the fused norm + product kernels stop at one tile of rows ...
    assert ops.can_fuse(8, bf, h, qkv) and not ops.can_fuse(26, bf, h, 2 * inter) and not ops.can_fuse(64, bf, h, qkv)
    # ... q/k/v of 24 to 384 rows goes through pieces (two at least beyond 64 rows), of more
    # rows through the tiled epilogue, and never through the few-row kernels beyond 64 rows
    assert ops.rules.qkv_pieces_min_rows <= 26 <= ops.QKV_ROPE_MAX_ROWS and ops.pieces_by_tiles(26, qkv, h)
    assert ops._linear_plan(26, qkv, h)[0] > 1 and ops._linear_plan(64, qkv, h)[0] > 1
    assert ops._qkv_pieces_plan(140, qkv, h) is not None and ops._qkv_pieces_plan(256, qkv, h)[0] >= 2
    assert ops._qkv_pieces_plan(512, qkv, h) is None and not ops.few_rows_take(140, qkv, h)
    assert ops.can_fuse_qkv_rope(512, bf, cfg.head_dim, qkv, h) and ops.can_fuse_qkv_rope(140, bf, cfg.head_dim, qkv, h)
    # ... and pieces of many rows are too large for a fused kernel to read in every block
    from llm_inference_lab_amd.parts import PendingSums
    pieces = PendingSums(torch.empty((ops.split_count(64, bf, h, inter), 64, h), device="meta"),
                         ops.split_count(64, bf, h, inter))
    assert ops.pieces_too_large_to_read_per_block(pieces)


@pytest.mark.parametrize("name", ["W7", "W32"])
@pytest.mark.parametrize("dtype,cut", [("bf16", "whole"), ("bf16", "decode"), ("bf16", "portions"),
                                       ("bf16", "mixed"), ("f32", "mixed")])
def test_one_layer_at_the_widths_of_larger_models(name, dtype, cut):
    cfg = H.config_of(name)
    seqs = sequences_of(name)
    want = {rid: H.plain_logits(name, 1, ids) for rid, ids in seqs.items()}
    engine = H.make_engine(name, 1, dtype, page_size=64, num_pages=19, max_requests=4, max_batch_tokens=512)
    if dtype == "bf16":
        assert_large_matrix_rules_fire(engine.ops, cfg)
    got = H.run_trace(engine, seqs, CUTS[cut](seqs))
    check(name, dtype, got, want, seqs)
    engine.cache.check()


@pytest.mark.parametrize("name", ["W7", "W32"])
@pytest.mark.parametrize("cut", ["whole", "mixed"])
def test_one_layer_with_the_tiles_of_large_steps(name, cut):
    """The tiles that only steps of a thousand rows and more get by themselves (128 x 256,
    and 256 x 256 and 192 x 256 with their two groups of waves), forced on every product of more than 64
    rows of these shorter steps: q/k/v with rotation and cache write, both products into the
    stream, gate/up with SwiGLU and the logits."""
    seqs = sequences_of(name)
    want = {rid: H.plain_logits(name, 1, ids) for rid, ids in seqs.items()}
    for tile in (131, 132, 133):
        engine = H.make_engine(name, 1, "bf16", page_size=64, num_pages=19, max_requests=4, max_batch_tokens=512)
        with engine.ops.debug.force(gemm_tile=tile):
            got = H.run_trace(engine, seqs, CUTS[cut](seqs))
        check(name, "bf16", got, want, seqs)
        engine.cache.check()


@pytest.mark.parametrize("name", ["W7", "W32"])
@pytest.mark.parametrize("graph", [False, True])
def test_steps_of_many_decoding_requests_at_the_widths_of_larger_models(name, graph):
    """8, 26 and 64 requests decode together (one tile of rows; q/k/v and the products
    into the stream in pieces; four tiles), eagerly and from replayed graphs, after a
    first step that brings their prompts of 19 tokens as one batch of many rows."""
    cfg = H.config_of(name)
    seqs = {f"r{i:02d}": H.random_ids(cfg, 19 + 10, 2000 + i) for i in range(64)}
    want = {rid: H.plain_logits(name, 1, ids) for rid, ids in seqs.items()}
    engine = H.make_engine(name, 1, "bf16", page_size=64, num_pages=64, max_requests=64,
                           max_batch_tokens=2048, graph=graph)
    assert_large_matrix_rules_fire(engine.ops, cfg)
    for count in (8, 26, 64):
        some = {rid: seqs[rid] for rid in list(seqs)[:count]}
        steps = [([(rid, 19, True) for rid in some], [])]
        steps += [([(rid, 1, True) for rid in some], []) for _ in range(10)]
        replays = engine.step_fn.graph_replays
        got = H.run_trace(engine, some, steps)
        if graph:       # (a key is captured when it comes the second time, after the buffers have settled)
            assert engine.step_fn.graph_replays - replays >= 6
        check(name, "bf16", got, want, some)
    engine.cache.check()
