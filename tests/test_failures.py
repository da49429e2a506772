"""What happens when something goes wrong in a step, on the CPU with the kernel
references and scripted failures: an entry that cannot run is left out with its error
and its peers still run (rust/engine/src/runner/model/qwen2/engine.rs:1943-2003); a step
that fails as a whole errs every member, drops their reservations and invalidates their
caches (engine.rs:2041-2045, rust/engine/src/runner/kv_pool/api.rs:257-262); a row of
logits without a finite value ends that request only (engine.rs:844-851).  After each
scenario the pool is back to its initial metrics."""
import pytest
import torch

import helpers as H
import llm_inference_lab_amd as lab
from emu_ops import EmuOps
from llm_inference_lab_amd.cache.pages import OutOfPages
from llm_inference_lab_amd.sampling import SamplingConfig


class ScriptedOps(EmuOps):
    """The kernel references with one scripted fault: the ``fail_at``-th call of ``fail_op``
    raises, or (``nan_at``) the head's output gets a row of NaN at that call."""

    def __init__(self, fail_op=None, fail_at=None, nan_at=None, nan_row=0):
        super().__init__("cpu")
        self.fail_op, self.fail_at, self.nan_at, self.nan_row = fail_op, fail_at, nan_at, nan_row
        self.head_calls = 0

    def _count(self, name):
        super()._count(name)
        if name == self.fail_op and self.calls[name] == self.fail_at:
            raise RuntimeError(f"scripted failure in {name}")

    def _poison(self, out):
        self.head_calls += 1
        if self.head_calls == self.nan_at and self.nan_row < out.shape[0]:
            out[self.nan_row] = float("nan")

    def linear_logits(self, x, w, out):
        super().linear_logits(x, w, out)
        self._poison(out)

    def fused_norm_logits(self, x, rows_index, norm_w, eps, w, out, pending=None):
        super().fused_norm_logits(x, rows_index, norm_w, eps, w, out, pending=pending)
        self._poison(out)


def engine_of(ops, name="A", **kw):
    kw.setdefault("page_size", 16)
    return H.make_engine(name, 1, "f32", ops=ops, device="cpu", **kw)


def pool_is_as_new(engine, initial):
    engine.cache.check()
    now = engine.cache.metrics()
    for g in now["groups"]:
        g.pop("pages_high_water")
    assert now == initial


def initial_metrics(engine):
    m = engine.cache.metrics()
    for g in m["groups"]:
        g.pop("pages_high_water")
    return m


def test_an_entry_that_cannot_run_is_left_out_and_its_peers_run():
    cfg = H.config_of("A")
    engine = engine_of(EmuOps(), num_pages=8, max_seq_len=64)
    initial = initial_metrics(engine)
    good_ids = H.random_ids(cfg, 9, 1)
    good, bad_token, too_long, twice = (engine.open(n) for n in ("good", "bad", "long", "twice"))
    result = engine.run_step([
        lab.StepEntry(bad_token, [1, cfg.vocab_size, 2], [2]),
        lab.StepEntry(good, good_ids, [8]),
        lab.StepEntry(too_long, [1] * 65, [0]),
        lab.StepEntry(twice, [5, 6], [1]),
        lab.StepEntry(twice, [7], [0]),
        lab.StepEntry(good, [], []),
    ])
    assert "vocabulary" in str(result.errors[0]) and result.errors[1] is None
    assert "exceed" in str(result.errors[2]) and result.errors[3] is None
    assert "twice" in str(result.errors[4]) and isinstance(result.errors[5], ValueError)
    assert result.shared_failure is None
    assert list(result.rows[1]) == [0] and list(result.rows[3]) == [1] and result.rows[0] is None
    want = H.plain_logits("A", 1, good_ids)[8]
    assert (result.logits[0].double() - want).abs().max() <= H.TOL["f32"]
    # the ones that ran moved on, the others hold nothing and can still be used
    assert good.computed_len == 9 and twice.computed_len == 2
    assert bad_token.computed_len == 0 and not bad_token.invalid and bad_token.pages[0] == []
    again = engine.run_step([lab.StepEntry(bad_token, [1, 2, 3], [2])])
    assert again.errors == [None]
    for r in (good, bad_token, too_long, twice):
        engine.close(r)
    pool_is_as_new(engine, initial)


def test_an_entry_that_finds_no_page_sits_out_alone():
    cfg = H.config_of("A")
    engine = engine_of(EmuOps(), num_pages=3, max_seq_len=64)
    initial = initial_metrics(engine)
    a, b = engine.open("a"), engine.open("b")
    result = engine.run_step([lab.StepEntry(a, H.random_ids(cfg, 30, 1), [29]),      # 2 pages
                              lab.StepEntry(b, H.random_ids(cfg, 20, 2), [19])])     # 2 more: only 1 left
    assert result.errors[0] is None and isinstance(result.errors[1], OutOfPages)
    assert a.computed_len == 30 and b.computed_len == 0 and b.pages[0] == [] and not b.invalid
    assert engine.cache.free_pages(0) == 1
    engine.close(a)
    assert engine.run_step([lab.StepEntry(b, H.random_ids(cfg, 20, 2), [19])]).errors == [None]
    engine.close(b)
    pool_is_as_new(engine, initial)


@pytest.mark.parametrize("fail_op,fail_at", [("paged_attention", 2), ("linear_swiglu", 1), ("embed", 2)])
def test_a_step_that_fails_as_a_whole_errs_every_member_and_invalidates_them(fail_op, fail_at):
    cfg = H.config_of("A")
    ops = ScriptedOps(fail_op, fail_at)
    engine = engine_of(ops, num_pages=8, max_seq_len=64)
    initial = initial_metrics(engine)
    a, b, outsider = engine.open("a"), engine.open("b"), engine.open("c")
    if fail_op == "embed":      # a first step that works, so that the failing one has history behind it
        assert engine.run_step([lab.StepEntry(a, H.random_ids(cfg, 20, 1), []),
                                lab.StepEntry(outsider, [1, 2, 3], [])]).errors == [None, None]
    before = a.computed_len
    result = engine.run_step([lab.StepEntry(a, H.random_ids(cfg, 17, 3), [16]),
                              lab.StepEntry(b, [1, 2, 999999], [0]),
                              lab.StepEntry(b, H.random_ids(cfg, 5, 4), [4])])
    assert "scripted failure" in str(result.shared_failure)
    assert result.errors[0] is result.shared_failure and result.errors[2] is result.shared_failure
    assert "vocabulary" in str(result.errors[1])          # its own error stays its own
    assert result.logits is None
    # nothing is pending, nothing moved, and what the step took is given back
    assert a.reserved_len == a.computed_len == before and b.reserved_len == b.computed_len == 0
    assert a.invalid and b.invalid and not outsider.invalid
    engine.cache.check()
    assert engine.step_fn.failed_steps == 1
    # an invalidated request is refused from then on; a request that was not in the step goes on
    later = engine.run_step([lab.StepEntry(a, [1], [0]), lab.StepEntry(outsider, [4], [0])])
    assert "failed" in str(later.errors[0]) and later.errors[1] is None
    with pytest.raises(ValueError, match="failed"):
        engine.step([lab.StepEntry(b, [1], [0])])
    for r in (a, b, outsider):
        engine.close(r)
    pool_is_as_new(engine, initial)


def test_the_strict_step_raises_before_anything_runs():
    cfg = H.config_of("A")
    engine = engine_of(EmuOps(), num_pages=8, max_seq_len=64)
    a, b = engine.open("a"), engine.open("b")
    with pytest.raises(ValueError, match="vocabulary"):
        engine.step([lab.StepEntry(a, [1, 2, 3], [2]), lab.StepEntry(b, [cfg.vocab_size], [0])])
    assert a.computed_len == 0 and a.reserved_len == 0 and a.pages[0] == [] and engine.step_fn.steps == 0
    roomy = engine_of(EmuOps(), num_pages=40, max_seq_len=512, max_batch_tokens=256)
    c = roomy.open("c")
    with pytest.raises(ValueError, match="max_batch_tokens"):
        roomy.run_step([lab.StepEntry(c, [1] * 300, [])])
    assert roomy.cache.free_pages(0) == 40 and c.reserved_len == 0


def test_the_strict_step_leaves_everything_as_it_was_when_a_page_is_missing():
    """``engine.step`` with an entry that finds no page raises before anything runs: the
    lengths, reservations and pages of every entry, also of those that came before it in
    the list and had got their pages, are as before, so the same peers can be fed the
    same tokens again at the same positions."""
    cfg = H.config_of("A")
    engine = engine_of(EmuOps(), num_pages=4, max_seq_len=64)
    initial = initial_metrics(engine)
    a, b, c = engine.open("a"), engine.open("b"), engine.open("c")
    first = H.random_ids(cfg, 10, 1)
    engine.step([lab.StepEntry(a, first, [])])                       # a holds 1 page of 4
    held = [list(r.pages[0]) for r in (a, b, c)]
    steps_before = engine.step_fn.steps
    more_a, ids_b, ids_c = H.random_ids(cfg, 20, 2), H.random_ids(cfg, 17, 3), H.random_ids(cfg, 20, 4)
    with pytest.raises(OutOfPages):
        engine.step([lab.StepEntry(a, more_a, [19]),                # 1 more page
                     lab.StepEntry(b, ids_b, [16]),                 # 2 pages: the pool is empty now
                     lab.StepEntry(c, ids_c, [19])])                # none left
    assert engine.step_fn.steps == steps_before
    assert (a.computed_len, a.reserved_len) == (10, 10) and not a.invalid
    for r in (b, c):
        assert (r.computed_len, r.reserved_len) == (0, 0) and not r.invalid
    assert [list(r.pages[0]) for r in (a, b, c)] == held and engine.cache.free_pages(0) == 3
    engine.cache.check()
    # the caller tries again without the one that did not fit: same logits as plain
    logits = engine.step([lab.StepEntry(a, more_a, [19]), lab.StepEntry(b, ids_b, [16])])
    assert (logits[0].double() - H.plain_logits("A", 1, first + more_a)[29]).abs().max() <= H.TOL["f32"]
    assert (logits[1].double() - H.plain_logits("A", 1, ids_b)[16]).abs().max() <= H.TOL["f32"]
    for r in (a, b, c):
        engine.close(r)
    pool_is_as_new(engine, initial)


@pytest.mark.parametrize("overlap", [False, True])
def test_scheduler_ends_the_requests_of_a_failed_step_and_goes_on(overlap):
    cfg = H.config_of("A")
    prompts = [H.random_ids(cfg, n, 60 + n) for n in (5, 12, 7, 9)]
    good = engine_of(EmuOps(), num_pages=12, max_requests=2)
    want = good.generate(prompts, max_new_tokens=4, eos_token_id=[], overlap=overlap)
    ops = ScriptedOps("paged_attention", 5)           # third step's first layer
    engine = engine_of(ops, num_pages=12, max_requests=2)
    initial = initial_metrics(engine)
    sched = engine.scheduler(overlap=overlap)
    ids = [sched.add_request(p, SamplingConfig(max_new_tokens=4, eos_token_id=[])) for p in prompts]
    done = sched.run()
    # the two that were running when the step failed end with its error; the two that
    # waited run afterwards, undisturbed
    for i in ids[:2]:
        assert done[i].finish_reason == "error" and "scripted failure" in str(done[i].error)
        assert done[i].generated == want[i][:len(done[i].generated)]
    for i in ids[2:]:
        assert done[i].error is None and done[i].generated == want[i]
    pool_is_as_new(engine, initial)
    m = engine.metrics()
    assert m["step"]["failed_steps"] == 1 and m["requests"]["failures"] == 2
    assert m["requests"]["requests"] == 4 and m["requests"]["in_flight"] == 0
    with pytest.raises(RuntimeError, match="scripted failure"):
        engine2 = engine_of(ScriptedOps("paged_attention", 1), num_pages=12)
        engine2.generate(prompts[:1], max_new_tokens=2)


@pytest.mark.parametrize("overlap", [False, True])
def test_a_row_without_a_finite_logit_ends_that_request_only(overlap):
    cfg = H.config_of("A")
    prompts = [H.random_ids(cfg, n, 80 + n) for n in (6, 3, 11)]
    good = engine_of(EmuOps(), num_pages=12)
    want = good.generate(prompts, max_new_tokens=6, eos_token_id=[], overlap=overlap)
    ops = ScriptedOps(nan_at=3, nan_row=1)             # third step (second decode), second request
    engine = engine_of(ops, num_pages=12)
    initial = initial_metrics(engine)
    sched = engine.scheduler(overlap=overlap)
    ids = [sched.add_request(p, SamplingConfig(max_new_tokens=6, eos_token_id=[])) for p in prompts]
    done = sched.run()
    assert isinstance(done[ids[1]].error, FloatingPointError) and done[ids[1]].finish_reason == "error"
    assert done[ids[1]].generated == want[1][:2]
    assert done[ids[0]].error is None and done[ids[0]].generated == want[0]
    assert done[ids[2]].error is None and done[ids[2]].generated == want[2]
    pool_is_as_new(engine, initial)
    # the plain call still raises for such a row
    with pytest.raises(FloatingPointError):
        sampler = lab.sampling.Sampler(EmuOps(), 4)
        sampler.sample(torch.full((2, 7), float("nan")), [0.0, 0.0], [0, 0], [0, 0])


def test_generation_config_names_the_end_of_sequence_ids(tmp_path):
    """config.json names one id, generation_config.json two: the model stops on both
    (engine.rs:403-407), a request's own ids go before both."""
    import json
    import os
    from llm_inference_lab_amd.config.errors import ConfigError
    from llm_inference_lab_amd.sampling.params import read_generation_config
    cfg = H.config_of("A")
    prompt = H.random_ids(cfg, 9, 3)
    draw = dict(temperature=20.0, seed=5)      # (greedy runs of this tiny model repeat one token)
    free_run = engine_of(EmuOps(), num_pages=8).generate([prompt], max_new_tokens=6, eos_token_id=[], **draw)[0]
    first, second = free_run[1], free_run[3]
    assert len(set(free_run[:4])) == 4
    raw = cfg.to_dict()
    raw["eos_token_id"] = second
    model = str(tmp_path / "model")
    lab.write_random_model(model, lab.Qwen2Config.from_dict(raw), 0)
    from llm_inference_lab_amd.weights import save_safetensors
    save_safetensors(os.path.join(model, "model.safetensors"), H.make_tensors(cfg, 1).items())

    def run(**kw):
        engine = lab.Engine(model, dtype="f32", ops=EmuOps(), device="cpu", page_size=16, num_pages=8,
                            max_requests=4, max_seq_len=64)
        return engine, engine.generate([prompt], max_new_tokens=6, **draw, **kw)[0]
    engine, out = run()
    assert engine.generation_config is None and engine.eos_token_ids == (second,)
    assert out == free_run[:4]
    with open(os.path.join(model, "generation_config.json"), "w") as f:
        json.dump({"eos_token_id": [first, second], "temperature": 0.7, "top_p": 0.8, "pad_token_id": 0,
                   "repetition_penalty": 1.05}, f)
    engine, out = run()
    assert engine.eos_token_ids == (first, second) and out == free_run[:2]
    assert engine.generation_config.temperature == 0.7 and engine.generation_config.top_p == 0.8
    assert run(eos_token_id=[])[1] == free_run            # the request's own (empty) list wins
    assert run(eos_token_id=second)[1] == free_run[:4]
    with open(os.path.join(model, "generation_config.json"), "w") as f:
        json.dump({"max_new_tokens": 4}, f)                # names no ids: config.json's stand
    assert run()[0].eos_token_ids == (second,)
    for bad in ({"eos_token_id": "7"}, {"eos_token_id": [1, -2]}, {"temperature": "hot"},
                {"do_sample": 1}, {"max_new_tokens": 2.5}):
        with open(os.path.join(model, "generation_config.json"), "w") as f:
            json.dump(bad, f)
        with pytest.raises(ConfigError, match=list(bad)[0]):
            read_generation_config(model)


def test_metrics_count_steps_tokens_and_requests():
    cfg = H.config_of("A")
    engine = engine_of(EmuOps(), num_pages=12)
    prompts = [H.random_ids(cfg, n, 20 + n) for n in (5, 30)]
    out = engine.generate(prompts, max_new_tokens=4, eos_token_id=[], max_batch_tokens=16, overlap=False)
    m = engine.metrics()
    step = m["step"]
    # 35 prompt tokens in portions of at most 16, then decode steps of two requests
    assert step["prefill"]["input_tokens"] + step["decode"]["input_tokens"] == 35 + 2 * 3
    assert step["prefill"]["steps"] + step["decode"]["steps"] == m["steps"]
    assert step["decode"]["steps"] >= 2 and step["failed_steps"] == 0
    assert step["batch_size"]["max"] == 2 and step["batch_size"]["count"] == m["steps"]
    assert step["decode"]["host_submit_seconds"]["count"] == step["decode"]["steps"]
    assert step["decode"]["step_wall_seconds"]["count"] >= 1
    req = m["requests"]
    assert req["requests"] == 2 and req["failures"] == 0 and req["in_flight"] == 0
    assert req["generated_tokens"] == sum(len(o) for o in out) == 8
    assert req["first_token_seconds"]["count"] == 2 and req["queue_wait_seconds"]["count"] == 2
    assert req["duration_seconds"]["success"]["count"] == 2
    assert req["output_tokens_per_second"]["count"] == 2
    assert m["graphs"]["captures"] == 0 and m["scratch"]["bytes"] > 0 and m["scratch"]["allocations"] > 0
    assert m["cache"]["rows_used"] == 0


def test_histogram_quantiles():
    from llm_inference_lab_amd.engine.instruments import Histogram
    h = Histogram()
    assert h.snapshot() == {"count": 0}
    for i in range(1, 101):
        h.record(i * 1e-3)
    s = h.snapshot()
    assert s["count"] == 100 and abs(s["sum"] - 5.05) < 1e-9 and s["min"] == 1e-3 and s["max"] == 0.1
    assert 0.04 <= s["p50"] <= 0.07 and 0.09 <= s["p95"] <= 0.1
