"""Command line: a model folder (or random weights) and a prompt to generated
tokens, with one JSON object on standard output.

Option names and meanings follow the reference's command line where it has
them (rust/engine/examples/qwen2.rs:38-73): ``--dtype``, ``--model-dir``,
``--prompt``, ``--max-new-tokens``, ``--max-batch-tokens``, ``--disable-overlap``, ``--reference-dir``,
``--repeat``, ``--cuda-graph``, ``--trace-steps``.  Not taken over:
``--prefix-cache`` (this engine has none).  Added:
token ids as input, random weights, temperature and seed, cache sizing.
The output object has the reference's fields (examples/qwen2.rs:262-268).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
import time
from typing import List, Optional


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="generate", description="Offline generation on one MI355X.")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f32"],
                    help="weight, activation and cache storage; reductions and accumulation stay FP32")
    ap.add_argument("--model-dir", help="local model folder (config.json, model.safetensors)")
    ap.add_argument("--prompt", default="Say hello.",
                    help="user message for the chat template (needs tokenizer.json in the model folder)")
    ap.add_argument("--prompt-ids", help="comma-separated token ids instead of --prompt; "
                                         "several prompts separated by ';'")
    ap.add_argument("--max-new-tokens", type=int, default=8, help="most generated tokens; positive")
    ap.add_argument("--max-batch-tokens", type=int, default=512,
                    help="most uncached input tokens per step, shared by decode and prefill")
    ap.add_argument("--disable-overlap", action="store_true",
                    help="wait for the host's token processing before the next step (serial baseline)")
    ap.add_argument("--reference-dir", help="folder with reference.json and logits.f32 to check against")
    ap.add_argument("--repeat", type=int, default=1, help="run the same prompt N times, checking equality")
    ap.add_argument("--cuda-graph", "--graph", dest="graph", action="store_true",
                    help="replay pure decode steps from a captured HIP graph; prefill stays eager")
    ap.add_argument("--trace-steps", action="store_true", help="per-step JSON metrics on standard error")
    ap.add_argument("--random-weights", metavar="CONFIG_JSON",
                    help="no model folder: write one from this config.json and --seed, then load it")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--temperature", type=float, default=None, help="sampling temperature (unset or 0: greedy)")
    ap.add_argument("--sampling-seed", type=int, default=0, help="seed of the sampling random stream")
    ap.add_argument("--page-size", type=int, default=64)
    ap.add_argument("--max-requests", type=int, default=64)
    ap.add_argument("--max-cache-tokens", type=int, default=None,
                    help="tokens the cache holds (default: what the prompts and their outputs need)")
    return ap


def _load_tokenizer(model_dir: str):
    path = os.path.join(model_dir, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    from tokenizers import Tokenizer
    return Tokenizer.from_file(path)


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    if args.max_new_tokens <= 0:
        print("--max-new-tokens must be positive", file=sys.stderr)
        return 2
    from . import Engine, write_random_model
    from .engine import settle_collector
    from .config.registry import architecture_of, read_config
    from .engine.step import StepEntry

    tmp = None
    model_dir = args.model_dir
    if args.random_weights:
        with open(args.random_weights, "r", encoding="utf-8") as f:
            raw = json.load(f)
        arch = architecture_of(raw, args.random_weights)
        tmp = tempfile.TemporaryDirectory(prefix="llmlab_random_")
        model_dir = write_random_model(tmp.name, arch.config_class.from_dict(raw, args.random_weights),
                                       args.seed)
    if model_dir is None:
        print("give --model-dir or --random-weights", file=sys.stderr)
        return 2

    tokenizer = None
    if args.prompt_ids:
        prompts = [[int(t) for t in part.split(",") if t.strip()] for part in args.prompt_ids.split(";")]
    else:
        tokenizer = _load_tokenizer(model_dir)
        if tokenizer is None:
            print(f"{model_dir} has no tokenizer.json: give --prompt-ids", file=sys.stderr)
            return 2
        # the architecture's registry entry says how a user's text is wrapped before it is
        # tokenised (rust/engine/examples/qwen2.rs:122-124 writes out the one of its model)
        template = read_config(model_dir)[0].chat_template
        text = template.replace("{prompt}", args.prompt) if template else args.prompt
        prompts = [tokenizer.encode(text, add_special_tokens=False).ids]

    reference = None
    if args.reference_dir:
        # reference.json: {"input_ids": [...], "generated_ids": [...]}; logits.f32: the
        # last-position logits of those input ids (the files the reference's checker reads,
        # rust/engine/examples/qwen2.rs:138-187)
        with open(os.path.join(args.reference_dir, "reference.json"), "r", encoding="utf-8") as f:
            reference = json.load(f)
    longest = max([len(p) + args.max_new_tokens for p in prompts]
                  + ([len(reference["input_ids"])] if reference else []))
    need = sum((len(p) + args.max_new_tokens + args.page_size) for p in prompts)
    if reference:
        need = max(need, len(reference["input_ids"]) + args.page_size)
    load_start = time.perf_counter()
    engine = Engine(model_dir, dtype=args.dtype, page_size=args.page_size,
                    max_cache_tokens=args.max_cache_tokens or need,
                    max_requests=max(args.max_requests, len(prompts)),
                    max_batch_tokens=args.max_batch_tokens,
                    max_seq_len=longest, graph=args.graph)
    load_seconds = time.perf_counter() - load_start
    settle_collector()

    def trace(event):
        print(json.dumps(event), file=sys.stderr, flush=True)

    validation = None
    if reference is not None:
        import numpy as np
        ids = [int(t) for t in reference["input_ids"]]
        want = np.fromfile(os.path.join(args.reference_dir, "logits.f32"), dtype="<f4")
        if want.size != engine.spec.vocab_size:
            print(f"reference logits hold {want.size} values, the vocabulary {engine.spec.vocab_size}",
                  file=sys.stderr)
            return 1
        req = engine.open("validation")
        got = None
        # (in portions of the token budget: the whole prompt need not fit one step)
        for at in range(0, len(ids), args.max_batch_tokens):
            part = ids[at:at + args.max_batch_tokens]
            got = engine.step([StepEntry(req, part, [len(part) - 1] if at + len(part) == len(ids) else [])])
        got = got[0].cpu().numpy()
        engine.close(req)
        err = float(abs(got - want).max())
        rms = float(np.sqrt(np.mean((got - want) ** 2)))
        # the reference's limits on the largest error (0.5 in bfloat16, 1e-3 in float32,
        # examples/qwen2.rs:170-173), and a bound on the root mean square beside them: one
        # logit may be off by a rounding of a large sum, all of them may not
        limit, rms_limit = (1e-3, 1e-3) if args.dtype == "f32" else (0.5, 0.05)
        expected = reference.get("generated_ids") or [int(want.argmax())]
        first_equal = int(got.argmax()) == int(expected[0])
        finite = bool(np.isfinite(got).all())
        validation = {"max_abs_logit_error": err, "rms_logit_error": rms, "limit": limit,
                      "rms_limit": rms_limit, "first_token": int(got.argmax()),
                      "first_token_equal": first_equal,
                      "passed": finite and err < limit and rms < rms_limit and first_equal}

    outputs = None
    elapsed = first = 0.0
    for _ in range(args.repeat):
        start = time.perf_counter()
        out = engine.generate(prompts, max_new_tokens=args.max_new_tokens,
                              temperature=args.temperature, seed=args.sampling_seed,
                              max_batch_tokens=args.max_batch_tokens,
                              trace=trace if args.trace_steps else None,
                              overlap=not args.disable_overlap)
        elapsed = time.perf_counter() - start
        firsts = [r.first_token_time - start for r in engine.last_scheduler.finished.values()
                  if r.first_token_time is not None]
        first = min(firsts) if firsts else 0.0
        if outputs is not None and out != outputs:
            print("repeated runs gave different tokens", file=sys.stderr)
            return 1
        outputs = out
    generated = sum(len(o) for o in outputs)
    metrics = engine.cache.metrics()
    released = metrics["rows_used"] == 0 and all(g["pages_used"] == 0 for g in metrics["groups"])
    result = {
        "model": model_dir if not args.random_weights else f"random:{args.random_weights}:seed{args.seed}",
        "compute_dtype": args.dtype,
        "input_ids": prompts[0] if len(prompts) == 1 else prompts,
        "request_id": 0,
        "output_ids": outputs[0] if len(outputs) == 1 else outputs,
        "text": tokenizer.decode(outputs[0]) if tokenizer is not None else None,
        "load_seconds": load_seconds,
        "elapsed_seconds": elapsed,
        "time_to_first_text_seconds": first,
        "generated_tokens": generated,
        "tokens_per_second": generated / elapsed if elapsed > 0 else None,
        "validation": validation,
        "kv_released": released,
    }
    print(json.dumps(result))
    if args.trace_steps:
        print(json.dumps({"event": "metrics", **engine.metrics()}), file=sys.stderr, flush=True)
    if tmp is not None:
        tmp.cleanup()
    return 0 if (validation is None or validation["passed"]) and released else 1


if __name__ == "__main__":
    sys.exit(main())
