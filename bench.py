"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--context S]
                    [--shape 0.5b|7b|32b] [--layers L] [--dtype bf16|f32]
    python bench.py --mixed [--shape 7b] [--requests 64] [--chunk 512] [--outputs 64]

Default: the layer sizes of the Qwen2.5-0.5B shape with seeded random weights,
batch 8, context 4096, bfloat16.  A "step" is one decode step of the whole
batch through the scheduler's own path (step function + sampling, tokens fed
back).  One JSON line is printed: decoded tokens a second as ``value``, plus

* ``prefill``: one 2,048-token prompt in one step;
* ``roofline``: bytes the decode step has to read over its time against 8 TB/s;
* ``points``: decode at batch 1, 64 and 128; the same shape in float32 (``f32_*``); decode at
  batch 8 and 1 at the 7B shape (context 4096) and at the 32B shape (context 8192) with the
  fraction of 8 TB/s each reaches, and the ``--mixed`` run at the 7B shape (all tokens a
  second): each of these comes from a child process of its own;
* ``validation``: before anything is timed, the last-position logits of a 2,048-token
  prompt fed whole against the same prompt fed in portions of 256 (same token, largest
  difference below 1e-3 in float32 and 0.5 in bfloat16), and greedy tokens of two runs
  with fresh caches (identical), as the reference's bench does
  (rust/engine/benches/qwen2.rs:247-274, 317-369);
* ``samples``: every point is timed three times (``--samples``), each time with fresh requests
  and fresh cache pages, and the median counts (``value``, ``ms_per_step``, the prefill's
  ``ms``); the smallest and the largest are printed beside it, as the reference's bench
  reports mean / p50 / p95 over its iterations (rust/engine/benches/qwen2.rs:279-316);
* ``measured``: what this very GPU gives to the simplest kernels (``csrc/measure.hip``, run
  in a child process before anything else): a read stream and a copy over 4 GiB, and
  waves that only issue matrix instructions (bfloat16 16x16x32 and float32 32x32x2).
  ``roofline`` and ``prefill`` carry ``measured_peak`` and ``frac_measured`` beside the
  fractions of the published peaks (8 TB/s; 2.5 PFLOP/s bfloat16, 157.3 TFLOP/s float32);
* ``step_ms``: median and 95th percentile of single steps timed through GPU completion;
* ``eager`` or ``graph``: the same decode steps the other way (launched kernel by kernel,
  or replayed from a HIP graph; ``--graph auto``, the default, lets the engine choose).

``--profile``: for runs under ``rocprofv3``: collection is paused (rocTX) except around the
timed steps, so that the profile holds those and not the filling of the caches
(rust/engine/benches/qwen2.rs:110-114, 175-179, 297-301).

``--mixed``: many requests with prompts of different lengths go through the
scheduler with a small token budget, so that portions of prompts run beside the
decode tokens of the requests that are already in; one JSON line with all tokens
(prompt and generated) a second.
"""
import argparse
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FILL_TOKENS = 8192       # token budget of the steps that fill the caches before decoding is timed
PEAK_FLOPS = {"bf16": 2.5e15, "f32": 157.3e12}
PAGE = 64
COMMON = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", rms_norm_eps=1e-6, rope_theta=1e6,
              max_position_embeddings=32768, use_sliding_window=False)
SHAPES = {   # layer sizes of the published Qwen2.5 checkpoints; weights are random
    "0.5b": dict(COMMON, vocab_size=151936, hidden_size=896, intermediate_size=4864,
                 num_hidden_layers=24, num_attention_heads=14, num_key_value_heads=2, head_dim=64,
                 tie_word_embeddings=True),
    "7b": dict(COMMON, vocab_size=152064, hidden_size=3584, intermediate_size=18944,
               num_hidden_layers=28, num_attention_heads=28, num_key_value_heads=4, head_dim=128,
               tie_word_embeddings=False),
    "32b": dict(COMMON, vocab_size=152064, hidden_size=5120, intermediate_size=27648,
                num_hidden_layers=64, num_attention_heads=40, num_key_value_heads=8, head_dim=128,
                tie_word_embeddings=False),
    # further sizes of the same family, for measurements beside the three above
    "1.5b": dict(COMMON, vocab_size=151936, hidden_size=1536, intermediate_size=8960,
                 num_hidden_layers=28, num_attention_heads=12, num_key_value_heads=2, head_dim=128,
                 tie_word_embeddings=True),
    "3b": dict(COMMON, vocab_size=151936, hidden_size=2048, intermediate_size=11008,
               num_hidden_layers=36, num_attention_heads=16, num_key_value_heads=2, head_dim=128,
               tie_word_embeddings=True),
    "14b": dict(COMMON, vocab_size=152064, hidden_size=5120, intermediate_size=13824,
                num_hidden_layers=48, num_attention_heads=40, num_key_value_heads=8, head_dim=128,
                tie_word_embeddings=False),
    "72b": dict(COMMON, vocab_size=152064, hidden_size=8192, intermediate_size=29568,
                num_hidden_layers=80, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                tie_word_embeddings=False),
}
DEFAULT_CONTEXT = {"0.5b": 4096, "7b": 4096, "32b": 8192, "1.5b": 4096, "3b": 4096, "14b": 4096, "72b": 4096}


def prefill_flops(cfg, tokens):
    h, i, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    q, kv = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
    per_token_layer = 2 * (h * (q + 2 * kv) + q * h + 3 * h * i)
    attention_layer = 4 * (tokens * (tokens + 1) // 2) * q
    return cfg.num_hidden_layers * (tokens * per_token_layer + attention_layer) + 2 * h * v


def random_weights_on_the_gpu(expected, seed):
    """Random weights of a large shape drawn on the GPU (the 65 GB of the 32B shape take
    minutes on the host), by the product's own rule for every tensor."""
    import torch
    from llm_inference_lab_amd.weights import random_tensors
    return random_tensors(expected, seed, torch.bfloat16, device="cuda:0")


def fits_the_gpu(cfg, batch, context, dtype, gpu_bytes=288e9, share=0.8):
    """Whether the weights and the cache pages of ``batch`` requests of ``context`` tokens leave
    a fifth of the GPU's memory to scratch buffers and the allocator."""
    width = 2 if dtype == "bf16" else 4
    h, i, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    q, kv = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
    weights = cfg.num_hidden_layers * (h * (q + 2 * kv) + q * h + 3 * h * i) + (1 if cfg.tie_word_embeddings else 2) * h * v
    cache = batch * (context + PAGE) * cfg.num_hidden_layers * 2 * kv
    return (weights + cache) * width <= share * gpu_bytes


def make_engine(args, cfg, max_cache_tokens, max_requests, max_batch_tokens, max_seq_len):
    import llm_inference_lab_amd as lab
    from llm_inference_lab_amd.config import get_architecture
    from llm_inference_lab_amd.engine.model import CausalLM
    tensors = None
    if args.shape != "0.5b" and args.dtype == "bf16":
        expected = CausalLM(get_architecture(cfg.architecture).build_spec(cfg)).tensor_specs()
        tensors = random_weights_on_the_gpu(expected, 0)
    engine = lab.Engine(config=cfg, seed=0, tensors=tensors, dtype=args.dtype, device="cuda:0", page_size=PAGE,
                        max_cache_tokens=max_cache_tokens, max_requests=max_requests,
                        max_batch_tokens=max_batch_tokens, max_seq_len=max_seq_len,
                        graph=False if args.no_graph else args.graph)
    del tensors
    from llm_inference_lab_amd.engine import settle_collector
    settle_collector()      # (as a serving process does: full collections cost 35 to 70 ms otherwise)
    return engine


class ProfilerBracket:
    """``--profile``: the profiler collects inside ``with bracket:`` only.  rocTX's pause and
    resume calls, which ``rocprofv3`` obeys; without the library, or without the flag,
    nothing happens."""

    def __init__(self, enabled):
        self.lib = None
        if enabled:
            import ctypes
            for name in ("librocprofiler-sdk-roctx.so", "/opt/rocm/lib/librocprofiler-sdk-roctx.so"):
                try:
                    self.lib = ctypes.CDLL(name)
                    self.lib.roctxProfilerPause.argtypes = [ctypes.c_uint64]
                    self.lib.roctxProfilerResume.argtypes = [ctypes.c_uint64]
                    self.lib.roctxRangePushA.argtypes = [ctypes.c_char_p]
                    break
                except (OSError, AttributeError):
                    self.lib = None
            if self.lib is None:
                print("bench.py: --profile: no rocTX library found, the whole run is collected", file=sys.stderr)
            else:
                self.lib.roctxProfilerPause(0)

    def __enter__(self):
        if self.lib is not None:
            self.lib.roctxProfilerResume(0)
            self.lib.roctxRangePushA(b"timed steps")
        return self

    def __exit__(self, *exc):
        if self.lib is not None:
            self.lib.roctxRangePop()
            self.lib.roctxProfilerPause(0)
        return False


def spread(values, digits=4):
    """Median, smallest and largest of the samples."""
    ordered = sorted(values)
    n = len(ordered)
    median = ordered[n // 2] if n % 2 else 0.5 * (ordered[n // 2 - 1] + ordered[n // 2])
    return {"median": round(median, digits), "min": round(ordered[0], digits), "max": round(ordered[-1], digits),
            "n": n}


def measured_peaks():
    """What this GPU gives to the simplest kernels: GB/s of a read stream and of a copy over
    4 GiB, TFLOP/s of waves that only issue matrix instructions.  Medians of five launches."""
    import ctypes
    import torch
    from llm_inference_lab_amd.kernels import build
    lib = ctypes.CDLL(build.measure_library())
    vp, cs, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    lib.llmlab_measure_read.argtypes = [vp, cs, vp, ci, vp]
    lib.llmlab_measure_copy.argtypes = [vp, vp, cs, ci, vp]
    lib.llmlab_measure_mfma.argtypes = [ci, ci, ci, vp, ctypes.POINTER(ctypes.c_double), vp]
    lib.llmlab_measure_barrier.argtypes = [ci, ci, vp, vp, ctypes.c_long, vp]
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream().cuda_stream
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    size = 4 << 30
    src = torch.empty(size, dtype=torch.uint8, device="cuda:0")
    dst = torch.empty(size, dtype=torch.uint8, device="cuda:0")
    src.random_(0, 255)
    sink = torch.zeros(4096, dtype=torch.float32, device="cuda:0")

    def timed(launch, repeats=5):
        launch()
        torch.cuda.synchronize()
        times = []
        for _ in range(repeats):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            assert launch() == 0
            end.record()
            end.synchronize()
            times.append(start.elapsed_time(end) * 1e-3)
        return spread(times, 9)["median"]

    out = {"stream_bytes": size, "compute_units": cus}
    blocks = cus * 8
    t = timed(lambda: lib.llmlab_measure_read(src.data_ptr(), size, sink.data_ptr(), blocks, stream))
    out["hbm_read_gbs"] = round(size / t / 1e9, 1)
    t = timed(lambda: lib.llmlab_measure_copy(src.data_ptr(), dst.data_ptr(), size, blocks, stream))
    out["hbm_copy_gbs"] = round(2 * size / t / 1e9, 1)
    for name, f32, iterations in (("mfma_bf16_tflops", 0, 20000), ("mfma_f32_tflops", 1, 5000)):
        flops = ctypes.c_double(0.0)
        t = timed(lambda: lib.llmlab_measure_mfma(f32, cus * 8, iterations, sink.data_ptr(), ctypes.byref(flops),
                                                  stream))
        out[name] = round(flops.value / t / 1e12, 1)
    # a device-wide barrier inside one kernel: 200 rounds of all compute units meeting at a
    # counter, against the same launch with one round (the difference is the rounds alone)
    flags = torch.zeros(2, dtype=torch.int32, device="cuda:0")

    def barriers(rounds):
        flags.zero_()
        return lib.llmlab_measure_barrier(cus, rounds, flags.data_ptr(), flags.data_ptr() + 4, 1 << 22, stream)
    many, one = timed(lambda: barriers(201)), timed(lambda: barriers(1))
    if int(flags[1]) == 0:
        out["grid_barrier_us"] = round((many - one) / 200 * 1e6, 2)
    return out


class Runs:
    """The timed runs over one engine."""

    def __init__(self, engine, cfg, context, dtype, samples=3, bracket=None, measured=None):
        import torch
        self.torch = torch
        self.engine, self.cfg, self.context, self.dtype = engine, cfg, context, dtype
        self.gen = torch.Generator().manual_seed(1234)
        self.samples = max(1, int(samples))
        self.bracket = bracket or ProfilerBracket(False)
        self.measured = measured or {}
        self.settled = set()

    def random_ids(self, n):
        return self.torch.randint(0, self.cfg.vocab_size, (n,), generator=self.gen).tolist()

    def sync(self):
        self.torch.cuda.synchronize()

    def decode(self, batch, steps, warmup):
        """`batch` requests decode side by side and reach `context` tokens at the end.

        The scheduler decodes for requests whose prompts are in while it still
        fills the others, so every request gets outputs enough for the fill, the
        warm-up and the timed steps, and a prompt shorter by as much; none ends
        before the timed steps are over (checked below).  Returns the seconds of the
        timed steps and the tokens the live requests held on average meanwhile."""
        from llm_inference_lab_amd.sampling import SamplingConfig
        engine, context = self.engine, self.context
        fill_steps = batch * context // FILL_TOKENS + 2
        outputs = fill_steps + warmup + steps + 1
        prompt_len = context - outputs
        assert prompt_len > 0, "context too short for this many steps"
        sched = engine.scheduler(max_batch_tokens=FILL_TOKENS)
        for b in range(batch):      # no token ends a request: a fixed number of outputs, as the reference's bench
            sched.add_request(self.random_ids(prompt_len),
                              SamplingConfig(max_new_tokens=outputs, eos_token_id=[]))
        while any(not r.decoding for r in sched.active) or sched.waiting:
            sched.step()                      # prefill in portions; ends with every request decoding
        for _ in range(warmup):
            sched.step()
        if batch not in self.settled:       # (the launch sequences of this batch are kept by now)
            from llm_inference_lab_amd.engine import settle_collector
            settle_collector()
            self.settled.add(batch)
        assert len(sched.active) == batch
        live_tokens = sum(r.computed for r in sched.active)
        self.sync()
        with self.bracket:
            t0 = time.perf_counter()
            for _ in range(steps):
                sched.step()
            self.sync()
            seconds = time.perf_counter() - t0
        assert len(sched.active) == batch, "a request ended inside the timed steps"
        live_tokens = (live_tokens + sum(r.computed for r in sched.active)) / 2
        done = sched.run()
        assert engine.cache.live_requests == 0 and all(r.error is None for r in done.values())
        return seconds, live_tokens

    def decode_samples(self, batch, steps, warmup):
        """``decode`` as often as ``--samples`` says, every time with fresh requests and pages:
        (seconds of the median sample, live tokens, spread of ms a step)."""
        runs = [self.decode(batch, steps, warmup) for _ in range(self.samples)]
        ms = spread([sec / steps * 1e3 for sec, _ in runs])
        return ms["median"] * steps / 1e3, runs[0][1], ms

    def roofline(self, seconds, steps, live_tokens):
        step_bytes = self.engine.weight_bytes_per_step() + live_tokens * self.engine.cache.bytes_per_token()
        achieved = step_bytes / (seconds / steps) / 1e9
        out = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
               "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4)}
        if self.measured.get("hbm_read_gbs"):
            out["measured_peak"] = self.measured["hbm_read_gbs"]
            out["frac_measured"] = round(achieved / self.measured["hbm_read_gbs"], 4)
        return out

    def step_latencies(self, batch, steps=32):
        """Single decode steps, each timed through GPU completion: (p50, p95) in ms."""
        from llm_inference_lab_amd.sampling import SamplingConfig
        outputs = batch * self.context // FILL_TOKENS + 2 + 4 + steps + 1
        sched = self.engine.scheduler(max_batch_tokens=FILL_TOKENS)
        for b in range(batch):
            sched.add_request(self.random_ids(self.context - outputs),
                              SamplingConfig(max_new_tokens=outputs, eos_token_id=[]))
        while any(not r.decoding for r in sched.active) or sched.waiting:
            sched.step()
        for _ in range(4):
            sched.step()
        times = []
        for _ in range(steps):
            self.sync()
            t0 = time.perf_counter()
            sched.step()
            self.sync()
            times.append((time.perf_counter() - t0) * 1e3)
        sched.run()
        times.sort()
        return round(times[len(times) // 2], 4), round(times[min(len(times) - 1, int(len(times) * 0.95))], 4)

    def prefill(self, tokens=2048, repeats=None):
        """One prompt in one step, logits at its last place: one untimed run, then the median
        of ``repeats`` (at least ``--samples``, at least three) with a fresh request each."""
        from llm_inference_lab_amd.engine.step import StepEntry
        repeats = repeats or max(3, self.samples)
        times = []
        for i in range(repeats + 1):
            req = self.engine.open("prefill")
            ids = self.random_ids(tokens)
            self.sync()
            if i == 0:
                self.engine.step([StepEntry(req, ids, [tokens - 1])])
                self.sync()
            else:
                with self.bracket:
                    t0 = time.perf_counter()
                    self.engine.step([StepEntry(req, ids, [tokens - 1])])
                    self.sync()
                    times.append(time.perf_counter() - t0)
            self.engine.close(req)
        ms = spread([t * 1e3 for t in times], 3)
        median = ms["median"] * 1e-3
        flops = prefill_flops(self.cfg, tokens)
        out = {"value": round(tokens / median, 1), "tokens": tokens, "ms": ms["median"],
               "frac": round(flops / median / PEAK_FLOPS[self.dtype], 4), "ms_min": ms["min"], "ms_max": ms["max"],
               "samples": ms["n"]}
        key = "mfma_bf16_tflops" if self.dtype == "bf16" else "mfma_f32_tflops"
        if self.measured.get(key):
            out["measured_peak"] = self.measured[key]
            out["frac_measured"] = round(flops / median / (self.measured[key] * 1e12), 4)
        return out

    def validate(self, tokens=None, chunk=256):
        """Whole against portions at the last position of a long prompt, and two greedy runs
        with fresh caches; raises if they differ by more than rounding
        (rust/engine/benches/qwen2.rs:247-274, 317-369)."""
        from llm_inference_lab_amd.engine.step import StepEntry
        engine = self.engine
        tokens = tokens or min(2048, self.context // 2)
        ids = self.random_ids(tokens)
        initial = engine.cache.metrics()
        req = engine.open("whole")
        whole = engine.step([StepEntry(req, ids, [tokens - 1])])[0].clone()
        engine.close(req)
        req = engine.open("portions")
        for at in range(0, tokens, chunk):
            part = ids[at:at + chunk]
            out = engine.step([StepEntry(req, part, [len(part) - 1] if at + chunk >= tokens else [])])
        portions = out[0].clone()
        assert req.computed_len == tokens, "the portions did not add up to the prompt"
        engine.close(req)
        assert bool(self.torch.isfinite(whole).all() and self.torch.isfinite(portions).all()), "non-finite logits"
        err = float((whole - portions).abs().max())
        # the same choice from both, or one that the whole prompt's own logits prefer by no more
        # than the two runs differ (random weights leave the best logits close together)
        margin = float(whole.max() - whole[int(portions.argmax())])
        same_token = margin <= 2 * err
        limit = 1e-3 if self.dtype == "f32" else 0.5
        prompts = [self.random_ids(n) for n in (5, 130, 700)]
        first = engine.generate(prompts, max_new_tokens=12, eos_token_id=[])
        second = engine.generate(prompts, max_new_tokens=12, eos_token_id=[])      # pages and rows used again
        after = engine.cache.metrics()
        for m in (initial, after):
            for g in m["groups"]:
                g.pop("pages_high_water")
        result = {"tokens": tokens, "chunk": chunk, "max_abs_logit_error": round(err, 6), "limit": limit,
                  "same_token": same_token, "token_margin": round(margin, 6), "samples_identical": first == second,
                  "kv_released": initial == after}
        result["passed"] = err < limit and same_token and first == second and initial == after
        if not result["passed"]:
            raise SystemExit(f"bench.py: validation failed: {json.dumps(result)}")
        return result


def force_what_was_asked(engine, args):
    """``--force KEY=VALUE``: kernel choices fixed for the whole run."""
    if not getattr(args, "force", None):
        return
    forced = {}
    for item in args.force:
        key, _, value = item.partition("=")
        numbers = [float(v) if "." in v else int(v) for v in value.split(":")]
        forced[key] = numbers[0] if len(numbers) == 1 else tuple(numbers)
    engine.forced_for_this_run = engine.ops.debug.force(**forced)    # (kept: it restores when collected)
    engine.forced_for_this_run.__enter__()


def mixed_run(args, cfg, engine=None, bracket=None):
    """Requests with prompts of 128..2048 tokens, all admitted at once; the scheduler cuts
    the prompts into portions under a budget of ``--chunk`` tokens a step, beside one
    token for every request that is decoding.  Timed from the first step to the last."""
    import torch
    from llm_inference_lab_amd.sampling import SamplingConfig

    gen = torch.Generator().manual_seed(4321)
    lengths = torch.randint(128, 2049, (args.requests,), generator=gen).tolist()
    longest = max(lengths) + args.outputs
    if engine is None:
        engine = make_engine(args, cfg, sum(n + args.outputs + PAGE for n in lengths), args.requests,
                             args.chunk + args.requests, longest + PAGE)
        force_what_was_asked(engine, args)

    def one_run():
        sched = engine.scheduler(max_batch_tokens=args.chunk + args.requests)
        for n in lengths:
            ids = torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist()
            sched.add_request(ids, SamplingConfig(max_new_tokens=args.outputs, eos_token_id=[]))
        steps = 0
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while sched.active or sched.waiting:
            sched.step()
            steps += 1
        torch.cuda.synchronize()
        seconds = time.perf_counter() - t0
        assert engine.cache.live_requests == 0
        return seconds, steps

    one_run()                                   # warm-up: scratch buffers, graphs, kernel loading
    with bracket or ProfilerBracket(False):
        timed = sorted(one_run() for _ in range(max(1, getattr(args, "samples", 1))))
    seconds, steps = timed[len(timed) // 2]     # the median run; every run serves fresh requests
    prompt_tokens, new_tokens = sum(lengths), args.requests * args.outputs
    # every prompt token and every generated token but a request's last goes through the model once
    flops = sum(prefill_flops(cfg, n + args.outputs - 1) - 2 * cfg.hidden_size * cfg.vocab_size for n in lengths)
    flops += new_tokens * 2 * cfg.hidden_size * cfg.vocab_size
    return {
        "metric": "mixed_tokens_per_second", "value": round((prompt_tokens + new_tokens) / seconds, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": steps,
        "ms_per_step": round(seconds / steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {
            "model": f"Qwen2.5-{args.shape.upper()} shape, random weights", "global_batch": args.requests,
            "seq_len": longest, "parallelism": "single GPU", "layers": cfg.num_hidden_layers,
            "layers_of_full_model": SHAPES[args.shape]["num_hidden_layers"], "hidden_size": cfg.hidden_size,
            "num_attention_heads": cfg.num_attention_heads,
            "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "prompt_lengths": "uniform 128..2048", "prompt_tokens": prompt_tokens,
            "outputs_per_request": args.outputs, "token_budget": args.chunk + args.requests,
            "page_size": PAGE, "weights_seed": 0,
        },
        "seconds": round(seconds, 4), "seconds_min": round(timed[0][0], 4), "seconds_max": round(timed[-1][0], 4),
        "samples": len(timed), "generated_tokens_per_second": round(new_tokens / seconds, 1),
        "flops_frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4),
    }


def child(*flags, timeout=420):
    """`bench.py <flags>` in a child process: its JSON line, or None."""
    try:
        out = subprocess.run([sys.executable, os.path.abspath(__file__), *flags],
                             capture_output=True, text=True, timeout=timeout)
        lines = [ln for ln in out.stdout.splitlines() if ln.startswith("{")]
        if out.returncode != 0 or not lines:
            print(f"bench.py: child {' '.join(flags)} failed:\n{out.stderr[-2000:]}", file=sys.stderr)
            return None
        return json.loads(lines[-1])
    except Exception as err:
        print(f"bench.py: child {' '.join(flags)}: {err}", file=sys.stderr)
        return None


def side_points(args, measured):
    """The points of the default line that other shapes and the other dtype give, each from
    a child process of its own (run before this process touches the GPU)."""
    points, validation = {}, {}
    steps, warmup = str(max(8, args.steps // 2)), str(max(2, args.warmup // 2))
    common = ["--steps", steps, "--warmup", warmup, "--samples", str(args.samples)]
    line = child("--side", "7b", *common)
    if line is not None:
        points["decode_b8_7b"], points["hbm_frac_b8_7b"] = line["decode_b8"], line["hbm_frac_b8"]
        points["decode_b1_7b"], points["hbm_frac_b1_7b"] = line["decode_b1"], line["hbm_frac_b1"]
        points["mixed_7b_tokens_per_second"] = line["mixed_tokens_per_second"]
    line = child("--side", "32b", *common)
    if line is not None:
        points["decode_b8_32b"], points["hbm_frac_b8_32b"] = line["decode_b8"], line["hbm_frac_b8"]
        points["decode_b1_32b"], points["hbm_frac_b1_32b"] = line["decode_b1"], line["hbm_frac_b1"]
    line = child("--side", "f32", *common)
    if line is not None:
        for key in ("decode_b1", "decode_b8", "decode_b64", "prefill_tokens_per_second", "prefill_frac"):
            points[f"f32_{key}"] = line[key]
        validation["f32"] = line["validation"]
    return points, validation


def side_run(args):
    """One child's work: ``--side 7b`` (decode at batch 8, context 4096, then the mixed run
    on the same engine), ``--side 32b`` (decode at batch 8, context 8192), ``--side f32``
    (the 0.5B shape in float32: validation, decode at batch 1 / 8 / 64, the prefill)."""
    if args.side == "peaks":
        print(json.dumps(measured_peaks()))
        return
    import llm_inference_lab_amd as lab
    if args.side == "f32":
        args.shape, args.dtype = "0.5b", "f32"
        cfg = lab.Qwen2Config.from_dict(dict(SHAPES["0.5b"]))
        context = DEFAULT_CONTEXT["0.5b"]
        engine = make_engine(args, cfg, 64 * (context + PAGE), 64, FILL_TOKENS, context + PAGE)
        runs = Runs(engine, cfg, context, "f32", args.samples)
        out = {"validation": runs.validate()}
        for batch in (1, 8, 64):
            steps = max(4, args.steps // (1 if batch < 64 else 2))
            seconds, _, _ = runs.decode_samples(batch, steps, args.warmup)
            out[f"decode_b{batch}"] = round(batch * steps / seconds, 1)
        prefill = runs.prefill()
        out["prefill_tokens_per_second"], out["prefill_frac"] = prefill["value"], prefill["frac"]
        print(json.dumps(out))
        return
    args.shape, args.dtype = args.side, "bf16"
    cfg = lab.Qwen2Config.from_dict(dict(SHAPES[args.shape]))
    context = DEFAULT_CONTEXT[args.shape]
    import torch
    gen = torch.Generator().manual_seed(4321)
    lengths = torch.randint(128, 2049, (args.requests,), generator=gen).tolist()
    mixed_tokens = sum(n + args.outputs + PAGE for n in lengths) if args.shape == "7b" else 0
    engine = make_engine(args, cfg, max(8 * (context + PAGE), mixed_tokens), max(8, args.requests),
                         FILL_TOKENS, max(context, max(lengths) + args.outputs) + PAGE)
    runs = Runs(engine, cfg, context, "bf16", args.samples)
    seconds, live, _ = runs.decode_samples(8, args.steps, args.warmup)
    out = {"decode_b8": round(8 * args.steps / seconds, 1),
           "hbm_frac_b8": runs.roofline(seconds, args.steps, live)["frac"]}
    seconds, live, _ = runs.decode_samples(1, args.steps, args.warmup)      # (a batch of 64 takes too long to fill)
    out["decode_b1"] = round(args.steps / seconds, 1)
    out["hbm_frac_b1"] = runs.roofline(seconds, args.steps, live)["frac"]
    if args.shape == "7b":
        out["mixed_tokens_per_second"] = mixed_run(args, cfg, engine)["value"]
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=None, help="default: 4096 (8192 at the 32B shape)")
    ap.add_argument("--shape", default="0.5b", choices=sorted(SHAPES),
                    help="layer sizes: those of Qwen2.5-0.5B (default), 7B or 32B")
    ap.add_argument("--layers", type=int, default=None,
                    help="run fewer layers than the shape has (both numbers are reported)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f32"])
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--graph", default="auto", choices=["auto", "on"],
                    help="decode from a HIP graph: always, or where the engine expects it to pay")
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 / 64, the prefill and the children")
    ap.add_argument("--no-validate", action="store_true", help="skip the check of logits before the timing")
    ap.add_argument("--mixed", action="store_true",
                    help="mixed run: --requests prompts of 128..2048 tokens, portions of --chunk tokens "
                         "beside decode tokens, --outputs tokens each")
    ap.add_argument("--requests", type=int, default=64)
    ap.add_argument("--chunk", type=int, default=512)
    ap.add_argument("--outputs", type=int, default=64)
    ap.add_argument("--prefill-tokens", type=int, default=2048,
                    help="with --only-prefill: the length of the prompt (at most 8192, one step)")
    ap.add_argument("--only-prefill", action="store_true",
                    help="run nothing but the 2,048-token prefill (for profiling); prints its numbers")
    ap.add_argument("--samples", type=int, default=3,
                    help="how often every point is timed, each time with fresh requests; the median counts")
    ap.add_argument("--profile", action="store_true",
                    help="under rocprofv3: collect the timed steps only (rocTX pause / resume around them)")
    ap.add_argument("--no-measured", action="store_true", help="skip the stream and matrix-instruction loops")
    ap.add_argument("--force", action="append", default=[], metavar="KEY=VALUE",
                    help="fix a choice of the kernels for the whole run, to compare variants: a keyword of "
                         "engine.ops.debug.force, values separated by ':' (attention_splits=64:8, "
                         "attention_merge_kernel=64, gemm_tile=129)")
    ap.add_argument("--side", choices=["7b", "32b", "f32", "peaks"], help=argparse.SUPPRESS)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        sys.exit(2)
    bracket = ProfilerBracket(args.profile)       # (pauses collection now: loading and filling are not collected)
    if args.graph == "on":
        args.graph = True
    if args.side:
        side_run(args)
        return

    # The other shapes and the other dtype are points of the default line: each runs as a
    # child process of its own, before this process touches the GPU.
    default_line = not (args.mixed or args.no_points or args.only_prefill) and args.shape == "0.5b" \
        and args.dtype == "bf16"
    measured = {}
    if not (args.no_measured or args.mixed or args.profile):
        measured = child("--side", "peaks", timeout=120) or {}
    side, side_validation = side_points(args, measured) if default_line else ({}, {})

    import llm_inference_lab_amd as lab

    full_layers = SHAPES[args.shape]["num_hidden_layers"]
    layers = args.layers or full_layers
    cfg = lab.Qwen2Config.from_dict(dict(SHAPES[args.shape], num_hidden_layers=layers))
    if args.mixed:
        print(json.dumps(mixed_run(args, cfg, bracket=bracket)))
        return
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64, 128})
    context = args.context or DEFAULT_CONTEXT[args.shape]
    if not args.no_points and args.batch < 128 and not fits_the_gpu(cfg, 128, context, args.dtype):
        batches.remove(128)             # (the 32B and 72B shapes: weights and the cache of 128 requests exceed the GPU)
    max_batch = max(batches)
    engine = make_engine(args, cfg, max_batch * (context + PAGE), max_batch, FILL_TOKENS, context + PAGE)
    runs = Runs(engine, cfg, context, args.dtype, args.samples, bracket, measured)
    force_what_was_asked(engine, args)

    if args.only_prefill:
        if not 0 < args.prefill_tokens <= min(FILL_TOKENS, context):
            sys.exit(f"--prefill-tokens must be between 1 and {min(FILL_TOKENS, context)}")
        print(json.dumps({"prefill": runs.prefill(args.prefill_tokens)}))
        return

    validation = dict(side_validation)
    if not args.no_validate:
        validation[args.dtype] = runs.validate()

    seconds, live_tokens, ms_spread = runs.decode_samples(args.batch, args.steps, args.warmup)
    value = args.batch * args.steps / seconds
    result = {
        "metric": "decode_tokens_per_second", "value": round(value, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(seconds / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {
            "model": f"Qwen2.5-{args.shape.upper()} shape, random weights", "global_batch": args.batch,
            "seq_len": context, "parallelism": "single GPU", "layers": layers,
            "layers_of_full_model": full_layers, "hidden_size": cfg.hidden_size,
            "num_attention_heads": cfg.num_attention_heads,
            "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "tie_word_embeddings": cfg.tie_word_embeddings, "page_size": PAGE,
            "hip_graph_decode": bool(engine.step_fn.use_graph), "weights_seed": 0,
        },
        "roofline": runs.roofline(seconds, args.steps, live_tokens),
        "samples": {"ms_per_step": ms_spread},
    }
    if measured:
        result["measured"] = measured
    if validation:
        result["validation"] = validation
    if not args.no_points:
        # prefill: one prompt of 2,048 tokens in one step, logits at its last place
        result["prefill"] = runs.prefill()
        points = {}
        half_steps, half_warmup = max(8, args.steps // 2), max(2, args.warmup // 2)
        for b in (1, 64, 128):
            if b not in batches:
                continue
            if b == args.batch:
                points[f"decode_b{b}"] = round(value, 1)
                continue
            s, _, spread_b = runs.decode_samples(b, half_steps, half_warmup)
            points[f"decode_b{b}"] = round(b * half_steps / s, 1)
            result["samples"][f"decode_b{b}_ms_per_step"] = spread_b
        points.update(side)
        result["points"] = points
        p50, p95 = runs.step_latencies(args.batch)
        result["step_ms"] = {"p50": p50, "p95": p95}
        if not args.no_graph:             # the same steps the other way: kernel by kernel, or from a graph
            chosen, auto = bool(engine.step_fn.use_graph), engine.step_fn.auto_graph
            engine.step_fn.use_graph, engine.step_fn.auto_graph = not chosen, False
            s, _ = runs.decode(args.batch, half_steps, half_warmup)
            engine.step_fn.use_graph, engine.step_fn.auto_graph = chosen, auto
            result["eager" if chosen else "graph"] = {
                "value": round(args.batch * half_steps / s, 1),
                "ms_per_step": round(s / half_steps * 1e3, 4)}
        result["kernel_calls_per_decode_step"] = engine.step_fn.decode_calls
    print(json.dumps(result))


if __name__ == "__main__":
    main()
