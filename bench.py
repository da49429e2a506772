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
* ``points``: decode at batch 1 and 64; the same shape in float32 (``f32_*``); decode at
  batch 8 at the 7B shape (context 4096) and at the 32B shape (context 8192) with the
  fraction of 8 TB/s each reaches, and the ``--mixed`` run at the 7B shape (all tokens a
  second): each of these comes from a child process of its own;
* ``validation``: before anything is timed, the last-position logits of a 2,048-token
  prompt fed whole against the same prompt fed in portions of 256 (same token, largest
  difference below 1e-3 in float32 and 0.5 in bfloat16), and greedy tokens of two runs
  with fresh caches (identical), as the reference's bench does
  (rust/engine/benches/qwen2.rs:247-274, 317-369);
* ``step_ms``: median and 95th percentile of single steps timed through GPU completion;
* ``eager`` or ``graph``: the same decode steps the other way (launched kernel by kernel,
  or replayed from a HIP graph; ``--graph auto``, the default, lets the engine choose).

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
    minutes on the host): N(0, 0.02), norm weights 1 + N(0, 0.1), in bfloat16."""
    import torch
    from llm_inference_lab_amd.weights.loader import VECTOR
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(seed)
    for name, spec in expected.items():
        values = torch.randn(spec.shape, generator=gen, dtype=torch.bfloat16, device="cuda:0")
        if spec.kind == VECTOR and "norm" in name:
            yield name, (1.0 + 0.1 * values.float()).to(torch.bfloat16)
        else:
            yield name, values.mul_(0.02)


def make_engine(args, cfg, max_cache_tokens, max_requests, max_batch_tokens, max_seq_len):
    import llm_inference_lab_amd as lab
    from llm_inference_lab_amd.config import get_architecture
    from llm_inference_lab_amd.engine.model import CausalLM
    tensors = None
    if args.shape != "0.5b" and args.dtype == "bf16":
        expected = CausalLM(get_architecture(cfg.architecture).build_spec(cfg)).tensor_specs()
        tensors = random_weights_on_the_gpu(expected, 0)
    return lab.Engine(config=cfg, seed=0, tensors=tensors, dtype=args.dtype, device="cuda:0", page_size=PAGE,
                      max_cache_tokens=max_cache_tokens, max_requests=max_requests,
                      max_batch_tokens=max_batch_tokens, max_seq_len=max_seq_len,
                      graph=False if args.no_graph else args.graph)


class Runs:
    """The timed runs over one engine."""

    def __init__(self, engine, cfg, context, dtype):
        import torch
        self.torch = torch
        self.engine, self.cfg, self.context, self.dtype = engine, cfg, context, dtype
        self.gen = torch.Generator().manual_seed(1234)

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
        assert len(sched.active) == batch
        live_tokens = sum(r.computed for r in sched.active)
        self.sync()
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

    def roofline(self, seconds, steps, live_tokens):
        step_bytes = self.engine.weight_bytes_per_step() + live_tokens * self.engine.cache.bytes_per_token()
        achieved = step_bytes / (seconds / steps) / 1e9
        return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4)}

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

    def prefill(self, tokens=2048, repeats=4):
        from llm_inference_lab_amd.engine.step import StepEntry
        times = []
        for _ in range(repeats):
            req = self.engine.open("prefill")
            ids = self.random_ids(tokens)
            self.sync()
            t0 = time.perf_counter()
            self.engine.step([StepEntry(req, ids, [tokens - 1])])
            self.sync()
            times.append(time.perf_counter() - t0)
            self.engine.close(req)
        best = min(times[1:])
        return {"value": round(tokens / best, 1), "tokens": tokens, "ms": round(best * 1e3, 3),
                "frac": round(prefill_flops(self.cfg, tokens) / best / PEAK_FLOPS[self.dtype], 4)}

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
        same_token = int(whole.argmax()) == int(portions.argmax())
        limit = 1e-3 if self.dtype == "f32" else 0.5
        prompts = [self.random_ids(n) for n in (5, 130, 700)]
        first = engine.generate(prompts, max_new_tokens=12, eos_token_id=[])
        second = engine.generate(prompts, max_new_tokens=12, eos_token_id=[])      # pages and rows used again
        after = engine.cache.metrics()
        for m in (initial, after):
            for g in m["groups"]:
                g.pop("pages_high_water")
        result = {"tokens": tokens, "chunk": chunk, "max_abs_logit_error": round(err, 6), "limit": limit,
                  "same_token": same_token, "samples_identical": first == second,
                  "kv_released": initial == after}
        result["passed"] = err < limit and same_token and first == second and initial == after
        if not result["passed"]:
            raise SystemExit(f"bench.py: validation failed: {json.dumps(result)}")
        return result


def mixed_run(args, cfg, engine=None):
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
    seconds, steps = one_run()
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
        "seconds": round(seconds, 4), "generated_tokens_per_second": round(new_tokens / seconds, 1),
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


def side_points(args):
    """The points of the default line that other shapes and the other dtype give, each from
    a child process of its own (run before this process touches the GPU)."""
    points, validation = {}, {}
    steps, warmup = str(max(8, args.steps // 2)), str(max(2, args.warmup // 2))
    line = child("--side", "7b", "--steps", steps, "--warmup", warmup)
    if line is not None:
        points["decode_b8_7b"], points["hbm_frac_b8_7b"] = line["decode_b8"], line["hbm_frac_b8"]
        points["mixed_7b_tokens_per_second"] = line["mixed_tokens_per_second"]
    line = child("--side", "32b", "--steps", steps, "--warmup", warmup)
    if line is not None:
        points["decode_b8_32b"], points["hbm_frac_b8_32b"] = line["decode_b8"], line["hbm_frac_b8"]
    line = child("--side", "f32", "--steps", steps, "--warmup", warmup)
    if line is not None:
        for key in ("decode_b1", "decode_b8", "decode_b64", "prefill_tokens_per_second", "prefill_frac"):
            points[f"f32_{key}"] = line[key]
        validation["f32"] = line["validation"]
    return points, validation


def side_run(args):
    """One child's work: ``--side 7b`` (decode at batch 8, context 4096, then the mixed run
    on the same engine), ``--side 32b`` (decode at batch 8, context 8192), ``--side f32``
    (the 0.5B shape in float32: validation, decode at batch 1 / 8 / 64, the prefill)."""
    import llm_inference_lab_amd as lab
    if args.side == "f32":
        args.shape, args.dtype = "0.5b", "f32"
        cfg = lab.Qwen2Config.from_dict(dict(SHAPES["0.5b"]))
        context = DEFAULT_CONTEXT["0.5b"]
        engine = make_engine(args, cfg, 64 * (context + PAGE), 64, FILL_TOKENS, context + PAGE)
        runs = Runs(engine, cfg, context, "f32")
        out = {"validation": runs.validate()}
        for batch in (1, 8, 64):
            steps = max(4, args.steps // (1 if batch < 64 else 2))
            seconds, _ = runs.decode(batch, steps, args.warmup)
            out[f"decode_b{batch}"] = round(batch * steps / seconds, 1)
        prefill = runs.prefill(repeats=3)
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
    runs = Runs(engine, cfg, context, "bf16")
    seconds, live = runs.decode(8, args.steps, args.warmup)
    out = {"decode_b8": round(8 * args.steps / seconds, 1),
           "hbm_frac_b8": runs.roofline(seconds, args.steps, live)["frac"]}
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
    ap.add_argument("--side", choices=["7b", "32b", "f32"], help=argparse.SUPPRESS)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        sys.exit(2)
    if args.graph == "on":
        args.graph = True
    if args.side:
        side_run(args)
        return

    # The other shapes and the other dtype are points of the default line: each runs as a
    # child process of its own, before this process touches the GPU.
    default_line = not (args.mixed or args.no_points or args.only_prefill) and args.shape == "0.5b" \
        and args.dtype == "bf16"
    side, side_validation = side_points(args) if default_line else ({}, {})

    import llm_inference_lab_amd as lab

    full_layers = SHAPES[args.shape]["num_hidden_layers"]
    layers = args.layers or full_layers
    cfg = lab.Qwen2Config.from_dict(dict(SHAPES[args.shape], num_hidden_layers=layers))
    if args.mixed:
        print(json.dumps(mixed_run(args, cfg)))
        return
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
    max_batch = max(batches)
    context = args.context or DEFAULT_CONTEXT[args.shape]
    engine = make_engine(args, cfg, max_batch * (context + PAGE), max_batch, FILL_TOKENS, context + PAGE)
    runs = Runs(engine, cfg, context, args.dtype)

    if args.only_prefill:
        if not 0 < args.prefill_tokens <= min(FILL_TOKENS, context):
            sys.exit(f"--prefill-tokens must be between 1 and {min(FILL_TOKENS, context)}")
        print(json.dumps({"prefill": runs.prefill(args.prefill_tokens)}))
        return

    validation = dict(side_validation)
    if not args.no_validate:
        validation[args.dtype] = runs.validate()

    seconds, live_tokens = runs.decode(args.batch, args.steps, args.warmup)
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
    }
    if validation:
        result["validation"] = validation
    if not args.no_points:
        # prefill: one prompt of 2,048 tokens in one step, logits at its last place
        result["prefill"] = runs.prefill()
        points = {}
        half_steps, half_warmup = max(8, args.steps // 2), max(2, args.warmup // 2)
        for b in (1, 64):
            if b == args.batch:
                points[f"decode_b{b}"] = round(value, 1)
                continue
            s, _ = runs.decode(b, half_steps, half_warmup)
            points[f"decode_b{b}"] = round(b * half_steps / s, 1)
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
