"""Decode from replayed graphs in the schedules that serving meets: requests of very
different lengths in one replay, context buckets crossed while they decode, more graph
keys than are kept, and a long history (thousands of keys, many key splits) beside short
ones.  Every position's logits against the plain implementation, in 32-bit and in
bfloat16.

The reference checks the same at whole-model level: decode graphs against eager steps with
growing, ragged histories (rust/engine/src/runner/model/qwen2/engine.rs:2777-3096) and 64
teacher-forced steps behind 4,096 tokens, split against unsplit (engine.rs:4359-4442)."""
import pytest
import torch

import helpers as H

TOL_REAL = H.TOL_REAL

pytestmark = pytest.mark.gpu


def tolerance(name, dtype):
    return TOL_REAL[dtype][0] if name == "R" else H.TOL[dtype]


def ragged_decode(name, dtype, graph, splits=None, prompts=(5, 60, 130, 250), decoded=300):
    """Four requests whose prompts differ by 50x go in as one step and then decode together,
    one token each a step, so that one replayed graph serves histories of 6 and of 251
    tokens, and the longest crosses two powers of two on the way."""
    cfg = H.config_of(name)
    seqs = {f"r{i}": H.random_ids(cfg, n + decoded, 4100 + i) for i, n in enumerate(prompts)}
    want = {rid: H.plain_logits(name, 1, ids) for rid, ids in seqs.items()}
    page = 64 if name == "R" else 16
    pages = sum((len(ids) + page - 1) // page for ids in seqs.values())
    engine = H.make_engine(name, 1, dtype, graph=graph, page_size=page, num_pages=pages, max_requests=4,
                           max_batch_tokens=512, max_seq_len=1024)
    steps = [([(rid, n, True) for rid, n in zip(seqs, prompts)], [])]
    steps += [([(rid, 1, True) for rid in seqs], []) for _ in range(decoded)]
    if splits is None:
        got = H.run_trace(engine, seqs, steps)
    else:
        with engine.ops.debug.force(attention_splits=(cfg.head_dim, splits)):
            got = H.run_trace(engine, seqs, steps)
    assert not any(bool(torch.isnan(g).any()) for g in got.values()), "a position's logits did not come back"
    bad = H.first_wrong(got, want, tolerance(name, dtype))
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
    return engine


@pytest.mark.parametrize("name", ["A", "B", "R"])
@pytest.mark.parametrize("dtype,splits", [("f32", None), ("bf16", None), ("bf16", 3), ("bf16", 16)])
def test_ragged_requests_decode_from_graphs_across_context_buckets(name, dtype, splits):
    """The keys of the longest request size the grid and the splits of the capture; the
    shortest request's few keys then lie in the first split only and the others are empty
    for it.  Buckets 256, 512 and 1,024 are each captured once and replayed from then on."""
    engine = ragged_decode(name, dtype, True, splits)
    fn = engine.step_fn
    assert fn.graph_captures >= 3 and fn.graph_replays >= 250 and fn.graph_evictions == 0


@pytest.mark.parametrize("name,dtype", [("B", "bf16"), ("R", "bf16"), ("A", "f32")])
def test_graphs_chosen_by_the_engine_itself(name, dtype):
    """``graph="auto"``: the first decode step runs eagerly and is measured; models as small
    as these are then replayed."""
    engine = ragged_decode(name, dtype, "auto")
    fn = engine.step_fn
    assert fn.use_graph is True and fn.decode_calls > 0
    assert fn.graph_captures >= 3 and fn.graph_replays >= 250


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_more_graph_keys_than_are_kept(dtype):
    """Eighteen requests of different lengths decode together and end one after the other,
    so the number of requests in a step takes every value from 18 down, in two context
    buckets: more keys than graphs are kept.  Then the same again: the first keys have been
    dropped by then and are captured anew."""
    cfg = H.config_of("A")
    lengths = [34 + 6 * i for i in range(18)]               # 34 .. 136: the longest cross 128
    want, waves = {}, []
    for wave in range(2):
        seqs = {f"w{wave}r{i:02d}": H.random_ids(cfg, n, 5200 + 100 * wave + i) for i, n in enumerate(lengths)}
        want.update({rid: H.plain_logits("A", 1, ids) for rid, ids in seqs.items()})
        waves.append(seqs)
    engine = H.make_engine("A", 1, dtype, graph=True, page_size=16, num_pages=18 * 9, max_requests=18,
                           max_batch_tokens=512, max_seq_len=256)
    got = {}
    captures = []
    for seqs in waves:
        steps = [([(rid, 20, True) for rid in seqs], [])]
        for pos in range(20, max(lengths)):
            live = [rid for rid, ids in seqs.items() if pos < len(ids)]
            steps.append(([(rid, 1, True) for rid in live], [rid for rid in live if pos == len(seqs[rid]) - 1]))
        got.update(H.run_trace(engine, seqs, steps))
        captures.append(engine.step_fn.graph_captures)
    fn = engine.step_fn
    assert fn.graph_evictions > 0 and len(fn._graphs) <= fn.MAX_GRAPHS
    assert captures[0] > fn.MAX_GRAPHS and captures[1] > captures[0]        # dropped keys come back
    assert fn.graph_replays > 100
    assert not any(bool(torch.isnan(g).any()) for g in got.values()), "a position's logits did not come back"
    bad = H.first_wrong(got, want, H.TOL[dtype])
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
    m = engine.cache.metrics()
    assert m["rows_used"] == 0 and all(g["pages_used"] == 0 for g in m["groups"])


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("graph", [False, True])
def test_a_long_history_beside_short_ones(dtype, graph):
    """Layers of real size.  One request of 4,200 tokens comes in portions of 512 (the last
    portions are few rows behind a long history), then decodes 40 tokens one by one beside
    seven requests with histories of 4 to 80 tokens: the launch splits the keys sixteen
    ways by the longest history, and the short requests' keys end inside the first split."""
    cfg = H.config_of("R")
    long_len, tail = 4200, 40
    seqs = {"long": H.random_ids(cfg, long_len + tail, 6000)}
    short = [3, 9, 17, 26, 33, 40, 47]
    for i, n in enumerate(short):
        seqs[f"s{i}"] = H.random_ids(cfg, n + tail, 6001 + i)
    want = {rid: H.plain_logits("R", 1, ids) for rid, ids in seqs.items()}
    engine = H.make_engine("R", 1, dtype, graph=graph, page_size=64, num_pages=67 + 2 * len(short),
                           max_requests=8, max_batch_tokens=512, max_seq_len=4352)
    steps = []
    for at in range(0, long_len, 512):
        steps.append(([("long", min(512, long_len - at), True)], []))
    steps.append(([(f"s{i}", n, True) for i, n in enumerate(short)], []))
    for t in range(tail):
        steps.append(([(rid, 1, True) for rid in seqs], list(seqs) if t == tail - 1 else []))
    got = H.run_trace(engine, seqs, steps)
    bad = H.first_wrong(got, want, TOL_REAL[dtype][0])
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
    err = torch.cat([(got[r].double() - want[r]).flatten() for r in seqs])
    assert float((err ** 2).mean().sqrt()) <= TOL_REAL[dtype][1]
    if graph:
        assert engine.step_fn.graph_replays >= tail - 2


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_portions_behind_a_history_beside_decoding_requests(dtype):
    """Layers of real size.  One request of 1,200 tokens comes in portions of 128 while three
    others, with histories of 50, 300 and 700 tokens, decode one token a step beside it: from
    the fourth portion on the portion's rows sit behind 384 keys and more, so its keys are split
    over the waves of a block, and in bfloat16 the decoding requests' blocks then run in the
    same attention launch.  Against the plain implementation, and bit for bit the logits of
    an engine whose mixed steps take a launch for each kind of request."""
    cfg = H.config_of("R")
    long_len, portion = 1200, 128
    steps_of_long = -(-long_len // portion)
    peers = {"p0": 50, "p1": 300, "p2": 700}
    seqs = {"long": H.random_ids(cfg, long_len, 6100)}
    for i, (rid, n) in enumerate(peers.items()):
        seqs[rid] = H.random_ids(cfg, n + steps_of_long, 6101 + i)
    want = {rid: H.plain_logits("R", 1, ids) for rid, ids in seqs.items()}
    steps = [([(rid, n, True)], []) for rid, n in peers.items()]
    for at in range(0, long_len, portion):
        steps.append(([("long", min(portion, long_len - at), True)] + [(rid, 1, True) for rid in peers], []))

    def run(two_launches):
        engine = H.make_engine("R", 1, dtype, graph=False, page_size=64, num_pages=40, max_requests=4,
                               max_batch_tokens=768, max_seq_len=1280)
        if two_launches:
            with engine.ops.debug.force(attention_two_launches=cfg.head_dim):
                return H.run_trace(engine, seqs, steps)
        return H.run_trace(engine, seqs, steps)

    if dtype == "bf16":      # (the schedule is one that the rule serves with one launch)
        ops = H.make_engine("R", 1, dtype, page_size=64, num_pages=4, max_seq_len=128).ops
        lib = ops._attention_lib(cfg.head_dim)
        assert lib.llmlab_attention_mixed_launches(cfg.num_attention_heads, cfg.num_key_value_heads, 4, 3, portion,
                                                   9 * portion, 709, 0, ops.num_cus) == 1
    got = run(False)
    bad = H.first_wrong(got, want, TOL_REAL[dtype][0])
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
    other = run(True)
    for rid in seqs:
        assert torch.equal(got[rid], other[rid]), f"{rid}: one launch and two differ"


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("name", ["B", "R"])
def test_kept_launch_sequences_change_nothing(name, dtype):
    """A block's calls into the kernel libraries are written down at its first run for a
    step of some number of rows and made again from the list afterwards (attention anew each
    time, from the step's description).  Mixed steps whose row counts repeat with other
    requests, other lengths and other histories behind them: bit for bit the logits of an
    engine that runs every part's code every time, and within the bound of plain."""
    cfg = H.config_of(name)
    lengths = [150, 41, 97, 260, 33, 120]
    seqs = {f"r{i}": H.random_ids(cfg, n, 7100 + i) for i, n in enumerate(lengths)}
    want = {rid: H.plain_logits(name, 1, ids) for rid, ids in seqs.items()}
    steps = H.steps_mixed(seqs, seed=3, max_live=4, budget=48)
    steps += H.steps_prefill_then_decode({f"again{i}": ids for i, ids in enumerate(list(seqs.values())[:2])})
    seqs.update({f"again{i}": ids for i, ids in enumerate(list(seqs.values())[:2])})
    want.update({f"again{i}": want[f"r{i}"] for i in range(2)})
    page = 64 if name == "R" else 16
    runs = {}
    for keep in (True, False):
        engine = H.make_engine(name, 1, dtype, page_size=page, num_pages=60, max_requests=4, max_batch_tokens=512)
        engine.model.keep_launches = keep
        runs[keep] = H.run_trace(engine, seqs, steps)
        m = engine.metrics()["launch_sequences"]
        if keep:
            assert m["recorded"] > 0 and m["replayed"] > 2 * m["recorded"]
        else:
            assert m == {"recorded": 0, "replayed": 0}
    for rid in seqs:
        assert torch.equal(runs[True][rid].nan_to_num(7.0), runs[False][rid].nan_to_num(7.0))
    bad = H.first_wrong(runs[True], want, tolerance(name, dtype))
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
