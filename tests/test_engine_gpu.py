"""The engine on the GPU against the plain implementation, in 32-bit and in
bfloat16: every request alone and whole; most of it in one step and the last 32
tokens one by one; portions of changing size down to two tokens; mixed batches
with so few pages that they are used again; long decoding; the first tokens of a
sequence; greedy generation through the entry point; the decode graph; and the
trace replay program."""
import json
import os
import subprocess
import sys

import pytest
import torch

import helpers as H
import plain_qwen2

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [1, 7, 29, 70, 130], "B": [5, 40, 61, 90, 200], "C": [3, 50, 97]}
CUTS = {"whole": H.steps_whole, "decode": H.steps_prefill_then_decode, "portions": H.steps_portions,
        "mixed": H.steps_mixed}


TOL_REAL = H.TOL_REAL


def sequences_of(name, seed=0):
    cfg = H.config_of(name)
    return {f"r{i}": H.random_ids(cfg, n, 100 * seed + i) for i, n in enumerate(LENGTHS[name])}


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("page_size", [16, 64])
def test_every_cut_matches_plain(dtype, name, cut, page_size):
    seqs = sequences_of(name)
    want = {rid: H.plain_logits(name, 1, ids) for rid, ids in seqs.items()}
    # pages for the four longest requests only: what one request gives back another takes
    longest = sorted((len(v) for v in seqs.values()), reverse=True)[:4]
    num_pages = sum((n + page_size - 1) // page_size for n in longest)
    engine = H.make_engine(name, 1, dtype, page_size=page_size, num_pages=num_pages, max_requests=4)
    got = H.run_trace(engine, seqs, CUTS[cut](seqs))
    bad = H.first_wrong(got, want, H.TOL[dtype])
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
    engine.cache.check()
    m = engine.cache.metrics()
    assert m["rows_used"] == 0 and all(g["pages_used"] == 0 for g in m["groups"])


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("cut", list(CUTS))
def test_layers_of_real_size(dtype, cut):
    """Two layers with the sizes of Qwen2.5-0.5B: what the kernels choose at real sizes
    (block shapes, tiles, pieces, fused paths) against the plain implementation."""
    cfg = H.config_of("R")
    seqs = {f"r{i}": H.random_ids(cfg, n, 700 + i) for i, n in enumerate([3, 75, 140, 330])}
    want = {rid: H.plain_logits("R", 1, ids) for rid, ids in seqs.items()}
    engine = H.make_engine("R", 1, dtype, page_size=64, num_pages=12, max_requests=4, max_batch_tokens=512)
    got = H.run_trace(engine, seqs, CUTS[cut](seqs))
    bad = H.first_wrong(got, want, TOL_REAL[dtype][0])
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
    err = torch.cat([(got[r].double() - want[r])[~torch.isnan(got[r]).any(1)].flatten() for r in seqs])
    assert float((err ** 2).mean().sqrt()) <= TOL_REAL[dtype][1]


@pytest.mark.parametrize("name", ["A", "B", "C", "R"])
@pytest.mark.parametrize("cut", ["whole", "portions", "mixed"])
def test_steps_of_many_rows_through_the_tiled_kernels(name, cut):
    """Matrices as small as these keep the few-row kernels up to 1,024 rows of a step; with
    that rule switched off every step of more than 64 rows takes the tiled kernels, as
    the steps of a large model do.  Same logits."""
    if name == "R":
        cfg = H.config_of("R")
        seqs = {f"r{i}": H.random_ids(cfg, n, 700 + i) for i, n in enumerate([3, 75, 140, 330])}
        engine = H.make_engine("R", 1, "bf16", page_size=64, num_pages=12, max_requests=4, max_batch_tokens=512)
        tol = TOL_REAL["bf16"][0]
    else:
        seqs = sequences_of(name)
        engine = H.make_engine(name, 1, "bf16", page_size=16, num_pages=40, max_requests=4)
        tol = H.TOL["bf16"]
    want = {rid: H.plain_logits(name, 1, ids) for rid, ids in seqs.items()}
    with engine.ops.debug.force(few_rows_max=64):
        got = H.run_trace(engine, seqs, CUTS[cut](seqs))
    bad = H.first_wrong(got, want, tol)
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("cut", ["decode", "portions", "mixed"])
def test_sums_left_in_pieces_reach_every_reader(name, cut):
    """With the threshold lowered so that the tiny models take that path too, the
    feed-forward's last product is left in pieces along its inner size, the next
    layer's q/k/v projection (or the output head) adds them as it reads the stream, and
    the attention output projection folds them in; steps of more rows fold them with the
    stand-alone kernel.  Same logits."""
    seqs = sequences_of(name)
    want = {rid: H.plain_logits(name, 1, ids) for rid, ids in seqs.items()}
    engine = H.make_engine(name, 1, "bf16", page_size=16, num_pages=40, max_requests=4)
    engine.ops.rules.min_steps_per_split = 1
    cfg = H.config_of(name)
    assert engine.ops.split_count(4, torch.bfloat16, cfg.hidden_size, cfg.intermediate_size) > 1
    got = H.run_trace(engine, seqs, CUTS[cut](seqs))
    bad = H.first_wrong(got, want, H.TOL["bf16"])
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("cut,from_rows", [("whole", 65), ("decode", 65), ("whole", 17), ("portions", 17),
                                           ("mixed", 17)])
def test_sums_of_many_rows_left_in_pieces(name, cut, from_rows):
    """The same for steps of many rows (tiled product cut along its inner size): the next
    layer's norm folds the pieces into the stream as it reads it, the final norm of
    gathered rows has them folded first.  Large matrices take this path from 17 rows on
    (the next reader is then a fused kernel of few rows or the norm): the tiny ones do
    too with the size limit taken away."""
    seqs = sequences_of(name)
    want = {rid: H.plain_logits(name, 1, ids) for rid, ids in seqs.items()}
    engine = H.make_engine(name, 1, "bf16", page_size=16, num_pages=40, max_requests=4)
    engine.ops.rules.forced_tiled_pieces = 2
    cfg = H.config_of(name)
    if from_rows == 17:
        engine.ops.rules.tiled_pieces_bytes = 0
        assert engine.ops.split_count(17, torch.bfloat16, cfg.hidden_size, cfg.intermediate_size) == 2
    assert engine.ops.split_count(130, torch.bfloat16, cfg.hidden_size, cfg.intermediate_size) > 1
    got = H.run_trace(engine, seqs, CUTS[cut](seqs))
    bad = H.first_wrong(got, want, H.TOL["bf16"])
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_cuts_agree_with_each_other_more_closely_than_with_plain(dtype):
    """The logits at a position do not depend on how the tokens were cut, beyond rounding."""
    seqs = sequences_of("B", seed=2)
    runs = {}
    for cut in CUTS:
        engine = H.make_engine("B", 1, dtype, page_size=16, num_pages=30, max_requests=4)
        runs[cut] = H.run_trace(engine, seqs, CUTS[cut](seqs))
    for cut in ("decode", "portions", "mixed"):
        assert H.max_error(runs[cut], {k: v.double() for k, v in runs["whole"].items()}) <= H.TOL[dtype]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_long_decoding(dtype, name):
    """600 tokens one by one after a short prompt: many pages, many steps of the
    keys per wave, a window that moves over page edges."""
    cfg = H.config_of(name)
    ids = H.random_ids(cfg, 640, 77)
    want = {"x": H.plain_logits(name, 1, ids)}
    engine = H.make_engine(name, 1, dtype, page_size=16, num_pages=48, max_seq_len=1024)
    steps = [([("x", 40, True)], [])] + [([("x", 1, True)], []) for _ in range(600)]
    got = H.run_trace(engine, {"x": ids}, steps)
    bad = H.first_wrong(got, want, H.TOL[dtype])
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"


@pytest.mark.parametrize("name,splits", [("A", 3), ("B", 7)])
def test_long_decoding_with_the_keys_split(name, splits):
    """Histories as short as a test's are left in one piece by the launch's own rule, so the
    split is fixed from outside: pieces that end inside a page, pieces past the end of a
    young history, the merge of their partial sums."""
    cfg = H.config_of(name)
    ids = H.random_ids(cfg, 400, 78)
    want = {"x": H.plain_logits(name, 1, ids)}
    engine = H.make_engine(name, 1, "bf16", page_size=16, num_pages=48, max_seq_len=1024)
    steps = [([("x", 3, True)], [])] + [([("x", 1, True)], []) for _ in range(397)]
    with engine.ops.debug.force(attention_splits=(cfg.head_dim, splits)):
        got = H.run_trace(engine, {"x": ids}, steps)
    bad = H.first_wrong(got, want, H.TOL["bf16"])
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_first_tokens_of_a_sequence(dtype):
    """Positions 0, 1, 2: one key, no rotation at position 0, a page that has just been handed out."""
    cfg = H.config_of("A")
    for n in (1, 2, 3):
        ids = H.random_ids(cfg, n, 5 + n)
        want = {"x": H.plain_logits("A", 1, ids)}
        engine = H.make_engine("A", 1, dtype)
        got = H.run_trace(engine, {"x": ids}, [([("x", 1, True)], []) for _ in range(n)])
        assert H.max_error(got, want) <= H.TOL[dtype]


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(name):
    cfg = H.config_of(name)
    tensors = H.make_tensors(cfg, 1)
    prompts = [H.random_ids(cfg, n, 30 + n) for n in (1, 7, 13, 29)]
    want = [plain_qwen2.greedy_generate(p, 16, tensors, cfg.to_dict()) for p in prompts]
    for graph in (False, True):
        engine = H.make_engine(name, 1, "f32", graph=graph, max_batch_tokens=16)
        got = engine.generate(prompts, max_new_tokens=16, eos_token_id=[])
        assert got == want
        m = engine.cache.metrics()
        assert m["rows_used"] == 0 and all(g["pages_used"] == 0 for g in m["groups"])
        if graph:
            assert engine.step_fn.graph_replays > 0
    # bfloat16 may part from the plain tokens only where the plain choice was closer than
    # its rounding (twice the bound on a logit); from there on its own history differs
    engine = H.make_engine(name, 1, "bf16", max_batch_tokens=16)
    got = engine.generate(prompts, max_new_tokens=16, eos_token_id=[])
    for prompt, g, w in zip(prompts, got, want):
        assert len(g) == 16
        logits = H.plain_logits(name, 1, prompt + w)
        for i, (a, b) in enumerate(zip(g, w)):
            if a != b:
                top = logits[len(prompt) + i - 1].topk(2).values
                assert float(top[0] - top[1]) <= 2 * H.TOL["bf16"], \
                    f"bfloat16 strays at a clear choice (margin {float(top[0] - top[1]):.3f}): {g} vs {w}"
                break


@pytest.mark.parametrize("name,graph", [("A", False), ("B", True)])
def test_many_requests_through_a_small_pool(name, graph):
    """Fourteen requests of random lengths, a token budget of 24 a step and pages for about
    three of them: requests wait for pages, prompts are cut into portions beside decodes,
    pages are handed on many times.  Every request's greedy tokens equal the plain
    implementation's (float32), and everything is given back at the end."""
    import random
    cfg = H.config_of(name)
    tensors = H.make_tensors(cfg, 1)
    rnd = random.Random(5)
    prompts = [H.random_ids(cfg, rnd.choice([1, 2, 5, 17, 33, 60, 90]), 500 + i) for i in range(14)]
    news = [rnd.choice([1, 3, 9, 20]) for _ in prompts]
    want = [plain_qwen2.greedy_generate(p, n, tensors, cfg.to_dict()) for p, n in zip(prompts, news)]
    engine = H.make_engine(name, 1, "f32", graph=graph, page_size=16, num_pages=21, max_requests=4,
                           max_batch_tokens=24)
    from llm_inference_lab_amd.sampling import SamplingConfig
    got = engine.generate(prompts, sampling=[SamplingConfig(max_new_tokens=n, eos_token_id=[]) for n in news])
    assert got == want
    engine.cache.check()
    m = engine.cache.metrics()
    assert m["rows_used"] == 0 and all(g["pages_used"] == 0 for g in m["groups"])


def test_default_page_pool_fits_the_free_memory(monkeypatch):
    """Nobody names a cache size: the pool holds every request at full length, or what the
    free memory takes, but one request of full length at least."""
    import llm_inference_lab_amd as lab
    cfg = H.config_of("B")
    tensors = H.make_tensors(cfg, 1)
    full = lab.Engine(config=cfg, tensors=tensors.items(), dtype="bf16", page_size=16, max_requests=4,
                      max_seq_len=512)
    assert full.cache.metrics()["groups"][0]["pages_total"] == 4 * 512 // 16
    per_page = sum(len(g.entries) * g.spec.bytes_per_token(torch.bfloat16) for g in full.model.cache_layout()[0]) * 16
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (int(50 * per_page / 0.9) + 1, 1 << 40))
    small = lab.Engine(config=cfg, tensors=tensors.items(), dtype="bf16", page_size=16, max_requests=4,
                       max_seq_len=512)
    assert small.cache.metrics()["groups"][0]["pages_total"] == 50
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (1, 1 << 40))
    least = lab.Engine(config=cfg, tensors=tensors.items(), dtype="bf16", page_size=16, max_requests=4,
                       max_seq_len=512)
    assert least.cache.metrics()["groups"][0]["pages_total"] == 512 // 16


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_decode_graph_replays_equal_eager(dtype):
    """Several replays with eager work and synchronisation between them, each checked."""
    cfg = H.config_of("B")
    seqs = {f"r{i}": H.random_ids(cfg, 90, 300 + i) for i in range(3)}
    want = {rid: H.plain_logits("B", 1, ids) for rid, ids in seqs.items()}
    engine = H.make_engine("B", 1, dtype, graph=True, page_size=16, num_pages=40)
    steps = [([(rid, 30, True) for rid in seqs], [])]
    steps += [([(rid, 1, True) for rid in seqs], []) for _ in range(60)]
    got = H.run_trace(engine, seqs, steps)
    assert engine.step_fn.graph_replays >= 50 and engine.step_fn.graph_captures >= 1
    bad = H.first_wrong(got, want, H.TOL[dtype])
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"


@pytest.mark.parametrize("graph", [False, True])
def test_many_decoding_requests_with_products_in_pieces(graph):
    """26 requests decode together at layers of real size, with the size limit taken away so
    that the rules for some rows of a large matrix hold: the down, the output and the
    q/k/v product go through the tiled kernel in pieces, the norms fold the pieces (too
    large for the fused kernels to read in every block), q/k/v is finished by the
    kernel that sums, rotates and writes the cache.  Eager and from a replayed graph."""
    cfg = H.config_of("R")
    seqs = {f"r{i:02d}": H.random_ids(cfg, 19 + 12, 900 + i) for i in range(26)}
    want = {rid: H.plain_logits("R", 1, ids) for rid, ids in seqs.items()}
    engine = H.make_engine("R", 1, "bf16", page_size=64, num_pages=30, max_requests=32, max_batch_tokens=512,
                           graph=graph)
    ops = engine.ops
    ops.rules.tiled_pieces_bytes, ops.rules.forced_tiled_pieces, ops.rules.pieces_per_block_bytes = 0, 2, 1 << 16
    assert ops.pieces_by_tiles(26, cfg.hidden_size, cfg.intermediate_size)
    assert ops.split_count(26, torch.bfloat16, cfg.hidden_size, cfg.intermediate_size) == 2
    steps = [([(rid, 19, True) for rid in seqs], [])]
    steps += [([(rid, 1, True) for rid in seqs], []) for _ in range(12)]
    got = H.run_trace(engine, seqs, steps)
    if graph:
        assert engine.step_fn.graph_replays >= 8
    bad = H.first_wrong(got, want, TOL_REAL["bf16"][0])
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_temperature_sampling_on_the_gpu(dtype):
    cfg = H.config_of("B")
    prompts = [H.random_ids(cfg, n, 70 + n) for n in (5, 40, 61)]
    engine = H.make_engine("B", 1, dtype, num_pages=30)
    a = engine.generate(prompts, max_new_tokens=24, temperature=0.8, seed=3, eos_token_id=[])
    b = engine.generate(prompts, max_new_tokens=24, temperature=0.8, seed=3, eos_token_id=[],
                        max_batch_tokens=8)
    c = engine.generate(prompts, max_new_tokens=24, temperature=0.8, seed=4, eos_token_id=[])
    again = engine.generate(prompts, max_new_tokens=24, temperature=0.8, seed=3, eos_token_id=[])
    assert a == again and a != c and all(len(x) == 24 for x in a)
    if dtype == "f32":
        # the same stream however the prompts are cut; in bfloat16 the logits of two
        # cuts differ by rounding, which may move a draw that sits on a boundary
        assert a == b
    else:
        assert [x[0] for x in a] == [x[0] for x in b]


def test_drawn_tokens_are_those_the_plain_implementation_predicts():
    """Config B in float32, three prompts, 24 tokens at temperature 0.8: token n of prompt
    i is the inverse-CDF draw from softmax(plain logits / 0.8) at uniform(seed + i, n)."""
    cfg = H.config_of("B")
    prompts = [H.random_ids(cfg, n, 70 + n) for n in (5, 40, 61)]
    engine = H.make_engine("B", 1, "f32", num_pages=30)
    got = engine.generate(prompts, max_new_tokens=24, temperature=0.8, seed=11, eos_token_id=[])
    for i, (prompt, tokens) in enumerate(zip(prompts, got)):
        assert len(tokens) == 24
        H.check_drawn_tokens("B", 1, prompt, tokens, 0.8, 11 + i)


def test_sampling_with_the_gpu_lagging_behind_the_host():
    """Greedy and sampled requests in one batch, of different lengths so that the batch
    changes while it runs, and a GPU that is a millisecond behind the host at every step
    (a sleeping kernel ahead of each): with one step of lookahead the host then fills the
    next step's temperatures and uniform numbers while this step's have not been copied
    yet.  Same tokens as without lookahead, and each the plain implementation's."""
    from llm_inference_lab_amd.sampling import SamplingConfig
    cfg = H.config_of("B")
    prompts = [H.random_ids(cfg, n, 170 + n) for n in (3, 9, 30, 17)]
    temps = [0.8, 0.0, 1.3, 0.0]
    news = [20, 7, 12, 16]
    sampling = [SamplingConfig(temperature=t, do_sample=t > 0, max_new_tokens=n, eos_token_id=[], seed=40 + i)
                for i, (t, n) in enumerate(zip(temps, news))]
    runs = {}
    for overlap in (True, False):
        engine = H.make_engine("B", 1, "f32", num_pages=30, max_batch_tokens=16)
        step = engine.step_fn.__call__

        def lagging(entries, step=step):
            torch.cuda._sleep(2_000_000)
            return step(entries)
        engine.step = lagging
        runs[overlap] = engine.generate(prompts, sampling=sampling, overlap=overlap)
    assert runs[True] == runs[False]
    for i, (prompt, tokens) in enumerate(zip(prompts, runs[True])):
        assert len(tokens) == news[i]
        H.check_drawn_tokens("B", 1, prompt, tokens, temps[i], 40 + i)


def write_model_dir(path, name, seed=1):
    from llm_inference_lab_amd.weights import save_safetensors
    cfg = H.config_of(name)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg.to_dict(), f)
    save_safetensors(os.path.join(path, "model.safetensors"), H.make_tensors(cfg, seed).items())
    return cfg


@pytest.mark.parametrize("dtype,key", [("float32", "f32"), ("bfloat16", "bf16")])
def test_trace_run_program(tmp_path, dtype, key):
    """bin/trace_run as a user runs it: steps on standard input, one `done` line per
    step, logits files for the steps that want some; mixed requests, pages reused."""
    import numpy as np
    cfg = write_model_dir(str(tmp_path / "model"), "B")
    seqs = {f"r{i}": H.random_ids(cfg, n, 500 + i) for i, n in enumerate([70, 33, 120, 64, 90])}
    want = {rid: H.plain_logits("B", 1, ids) for rid, ids in seqs.items()}
    steps = H.steps_mixed(seqs, seed=4, max_live=4)
    out_dir = tmp_path / "out"
    proc = subprocess.Popen(
        [sys.executable, os.path.join(H.ROOT, "bin", "trace_run"), "--model", str(tmp_path / "model"),
         "--dtype", dtype, "--out", str(out_dir), "--max-tokens", "384"],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    pos = {rid: 0 for rid in seqs}
    worst = 0.0
    try:
        for number, (entries, ends) in enumerate(steps):
            record = {"step": number, "entries": [], "end": ends}
            places = []
            for rid, count, _ in entries:
                toks = seqs[rid][pos[rid]:pos[rid] + count]
                wanted = [0, len(toks) - 1] if len(toks) > 1 else [0]
                if number % 5 == 4:
                    wanted = []
                record["entries"].append({"id": rid, "tokens": toks, "want": wanted})
                places += [(rid, pos[rid] + w) for w in wanted]
                pos[rid] += len(toks)
            proc.stdin.write(json.dumps(record) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {number}"
            path = out_dir / f"{number}.f32"
            if places:
                got = np.fromfile(path, dtype="<f4").reshape(len(places), cfg.vocab_size)
                for row, (rid, p) in enumerate(places):
                    worst = max(worst, float(np.abs(got[row] - want[rid][p].numpy()).max()))
            else:
                assert not path.exists()
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    assert worst <= H.TOL[key], worst
