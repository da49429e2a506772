"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--context S]
                    [--shape 0.5b|7b|32b] [--layers L]
    python bench.py --mixed [--shape 7b] [--requests 64] [--chunk 512] [--outputs 64]

Default: the layer sizes of the Qwen2.5-0.5B shape with seeded random weights,
batch 8, context 4096, bfloat16.  A "step" is one decode step of the whole
batch through the scheduler's own path (step function + sampling, tokens fed
back).  One JSON line is printed: decoded tokens a second as ``value``, plus
``prefill`` (one 2,048-token prompt), ``roofline`` (bytes the decode step has to
read over its time against 8 TB/s), ``points`` (decode at batch 1 and 64; the ``--mixed``
run at the 7B shape, all tokens a second), ``step_ms`` (median
and 95th percentile of single steps timed through GPU completion) and ``eager`` or ``graph``
(the same decode steps the other way: launched kernel by kernel, or replayed from a HIP
graph; ``--graph auto``, the default, lets the engine choose).

``--mixed``: many requests with prompts of different lengths go through the
scheduler with a small token budget, so that portions of prompts run beside the
decode tokens of the requests that are already in; one JSON line with all tokens
(prompt and generated) a second.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FILL_TOKENS = 8192       # token budget of the steps that fill the caches before decoding is timed
PEAK_FLOPS = {"bf16": 2.5e15, "f32": 157.3e12}
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
}


def prefill_flops(cfg, tokens):
    h, i, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    q, kv = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
    per_token_layer = 2 * (h * (q + 2 * kv) + q * h + 3 * h * i)
    attention_layer = 4 * (tokens * (tokens + 1) // 2) * q
    return cfg.num_hidden_layers * (tokens * per_token_layer + attention_layer) + 2 * h * v


def mixed_run(args, cfg, layers, full_layers):
    """Requests with prompts of 128..2048 tokens, all admitted at once; the scheduler cuts
    the prompts into portions under a budget of ``--chunk`` tokens a step, beside one
    token for every request that is decoding.  Timed from the first step to the last."""
    import torch
    import llm_inference_lab_amd as lab
    from llm_inference_lab_amd.sampling import SamplingConfig

    page = 64
    gen = torch.Generator().manual_seed(4321)
    lengths = torch.randint(128, 2049, (args.requests,), generator=gen).tolist()
    longest = max(lengths) + args.outputs
    engine = lab.Engine(config=cfg, seed=0, dtype=args.dtype, device="cuda:0", page_size=page,
                        max_cache_tokens=sum(n + args.outputs + page for n in lengths),
                        max_requests=args.requests, max_batch_tokens=args.chunk + args.requests,
                        max_seq_len=longest + page, graph=False if args.no_graph else args.graph)

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
    print(json.dumps({
        "metric": "mixed_tokens_per_second", "value": round((prompt_tokens + new_tokens) / seconds, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": steps,
        "ms_per_step": round(seconds / steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {
            "model": f"Qwen2.5-{args.shape.upper()} shape, random weights", "global_batch": args.requests,
            "seq_len": longest, "parallelism": "single GPU", "layers": layers,
            "layers_of_full_model": full_layers, "hidden_size": cfg.hidden_size,
            "num_attention_heads": cfg.num_attention_heads,
            "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "prompt_lengths": "uniform 128..2048", "prompt_tokens": prompt_tokens,
            "outputs_per_request": args.outputs, "token_budget": args.chunk + args.requests,
            "page_size": page, "weights_seed": 0,
        },
        "seconds": round(seconds, 4), "generated_tokens_per_second": round(new_tokens / seconds, 1),
        "flops_frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4),
    }))


def mixed_point(timeout=420):
    """`bench.py --mixed --shape 7b` in a child process: all tokens a second, or None."""
    import subprocess
    try:
        out = subprocess.run([sys.executable, os.path.abspath(__file__), "--mixed", "--shape", "7b"],
                             capture_output=True, text=True, timeout=timeout)
        lines = [ln for ln in out.stdout.splitlines() if ln.startswith("{")]
        return json.loads(lines[-1])["value"] if out.returncode == 0 and lines else None
    except Exception:
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--shape", default="0.5b", choices=sorted(SHAPES),
                    help="layer sizes: those of Qwen2.5-0.5B (default), 7B or 32B")
    ap.add_argument("--layers", type=int, default=None,
                    help="run fewer layers than the shape has (both numbers are reported)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f32"])
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--graph", default="auto", choices=["auto", "on"],
                    help="decode from a HIP graph: always, or where the engine expects it to pay")
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 / 64 and the prefill")
    ap.add_argument("--mixed", action="store_true",
                    help="mixed run: --requests prompts of 128..2048 tokens, portions of --chunk tokens "
                         "beside decode tokens, --outputs tokens each")
    ap.add_argument("--requests", type=int, default=64)
    ap.add_argument("--chunk", type=int, default=512)
    ap.add_argument("--outputs", type=int, default=64)
    ap.add_argument("--only-prefill", action="store_true",
                    help="run nothing but the 2,048-token prefill (for profiling); prints its numbers")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        sys.exit(2)

    # The mixed run at the 7B shape is a point of the default line: it runs as a child
    # process of its own, before this process touches the GPU.
    mixed_7b = None
    if not (args.mixed or args.no_points or args.only_prefill) and args.shape == "0.5b":
        mixed_7b = mixed_point()

    import torch
    import llm_inference_lab_amd as lab
    from llm_inference_lab_amd.engine.step import StepEntry
    from llm_inference_lab_amd.sampling import SamplingConfig

    full_layers = SHAPES[args.shape]["num_hidden_layers"]
    layers = args.layers or full_layers
    raw = dict(SHAPES[args.shape], num_hidden_layers=layers)
    cfg = lab.Qwen2Config.from_dict(raw)
    if args.mixed:
        mixed_run(args, cfg, layers, full_layers)
        return
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
    max_batch = max(batches)
    page = 64
    context = args.context
    engine = lab.Engine(config=cfg, seed=0, dtype=args.dtype, device="cuda:0", page_size=page,
                        max_cache_tokens=max_batch * (context + page), max_requests=max_batch,
                        max_batch_tokens=FILL_TOKENS, max_seq_len=context + page,
                        graph=False if args.no_graph else args.graph)
    gen = torch.Generator().manual_seed(1234)

    def random_ids(n):
        return torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist()

    def sync():
        torch.cuda.synchronize()

    def decode_run(batch, steps, warmup):
        """`batch` requests decode side by side and reach `context` tokens at the end.

        The scheduler decodes for requests whose prompts are in while it still
        fills the others, so every request gets outputs enough for the fill, the
        warm-up and the timed steps, and a prompt shorter by as much; none ends
        before the timed steps are over (checked below).
        """
        fill_tokens = FILL_TOKENS
        fill_steps = batch * context // fill_tokens + 2
        outputs = fill_steps + warmup + steps + 1
        prompt_len = context - outputs
        assert prompt_len > 0, "context too short for this many steps"
        sched = engine.scheduler(max_batch_tokens=fill_tokens)
        for b in range(batch):      # no token ends a request: a fixed number of outputs, as the reference's bench
            sched.add_request(random_ids(prompt_len),
                              SamplingConfig(max_new_tokens=outputs, eos_token_id=[]))
        while any(not r.decoding for r in sched.active) or sched.waiting:
            sched.step()                      # prefill in portions; ends with every request decoding
        for _ in range(warmup):
            sched.step()
        assert len(sched.active) == batch
        live_tokens = sum(r.computed for r in sched.active)
        sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            sched.step()
        sync()
        seconds = time.perf_counter() - t0
        assert len(sched.active) == batch, "a request ended inside the timed steps"
        live_tokens = (live_tokens + sum(r.computed for r in sched.active)) / 2
        sched.run()
        assert engine.cache.live_requests == 0
        return seconds, live_tokens

    def step_latencies(batch, steps=32):
        """Single decode steps, each timed through GPU completion: (p50, p95) in ms."""
        outputs = batch * context // FILL_TOKENS + 2 + 4 + steps + 1
        sched = engine.scheduler(max_batch_tokens=FILL_TOKENS)
        for b in range(batch):
            sched.add_request(random_ids(context - outputs), SamplingConfig(max_new_tokens=outputs, eos_token_id=[]))
        while any(not r.decoding for r in sched.active) or sched.waiting:
            sched.step()
        for _ in range(4):
            sched.step()
        times = []
        for _ in range(steps):
            sync()
            t0 = time.perf_counter()
            sched.step()
            sync()
            times.append((time.perf_counter() - t0) * 1e3)
        sched.run()
        times.sort()
        return round(times[len(times) // 2], 4), round(times[min(len(times) - 1, int(len(times) * 0.95))], 4)

    def prefill_run(tokens=2048, repeats=4):
        times = []
        for _ in range(repeats):
            req = engine.open("prefill")
            ids = random_ids(tokens)
            sync()
            t0 = time.perf_counter()
            engine.step([StepEntry(req, ids, [tokens - 1])])
            sync()
            times.append(time.perf_counter() - t0)
            engine.close(req)
        best = min(times[1:])
        return {"value": round(tokens / best, 1), "tokens": tokens, "ms": round(best * 1e3, 3),
                "frac": round(prefill_flops(cfg, tokens) / best / PEAK_FLOPS[args.dtype], 4)}

    if args.only_prefill:
        print(json.dumps({"prefill": prefill_run()}))
        return

    seconds, live_tokens = decode_run(args.batch, args.steps, args.warmup)
    ms_per_step = seconds / args.steps * 1e3
    value = args.batch * args.steps / seconds
    step_bytes = engine.weight_bytes_per_step() + live_tokens * engine.cache.bytes_per_token()
    achieved = step_bytes / (seconds / args.steps) / 1e9

    result = {
        "metric": "decode_tokens_per_second", "value": round(value, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {
            "model": f"Qwen2.5-{args.shape.upper()} shape, random weights", "global_batch": args.batch,
            "seq_len": context, "parallelism": "single GPU", "layers": layers,
            "layers_of_full_model": full_layers, "hidden_size": cfg.hidden_size,
            "num_attention_heads": cfg.num_attention_heads,
            "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "tie_word_embeddings": cfg.tie_word_embeddings, "page_size": page,
            "hip_graph_decode": bool(engine.step_fn.use_graph), "weights_seed": 0,
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        # prefill: one prompt of 2,048 tokens in one step, logits at its last place
        result["prefill"] = prefill_run()
        points = {}
        for b in (1, 64):
            if b == args.batch:
                points[f"decode_b{b}"] = round(value, 1)
                continue
            s, _ = decode_run(b, max(8, args.steps // 2), max(2, args.warmup // 2))
            points[f"decode_b{b}"] = round(b * max(8, args.steps // 2) / s, 1)
        if mixed_7b is not None:
            points["mixed_7b_tokens_per_second"] = mixed_7b
        result["points"] = points
        p50, p95 = step_latencies(args.batch)
        result["step_ms"] = {"p50": p50, "p95": p95}
        if not args.no_graph:             # the same steps the other way: kernel by kernel, or from a graph
            chosen = engine.step_fn.use_graph
            engine.step_fn.use_graph = not chosen
            s, _ = decode_run(args.batch, max(8, args.steps // 2), max(2, args.warmup // 2))
            engine.step_fn.use_graph = chosen
            result["eager" if chosen else "graph"] = {
                "value": round(args.batch * max(8, args.steps // 2) / s, 1),
                "ms_per_step": round(s / max(8, args.steps // 2) * 1e3, 4)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
