"""Shared pieces of the tests: the tiny configurations, random tensors with
sharpened attention, and the four ways of cutting a set of requests into steps."""
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

import llm_inference_lab_amd as lab                                    # noqa: E402
from llm_inference_lab_amd.config import get_architecture                # noqa: E402
from llm_inference_lab_amd.engine.model import CausalLM                  # noqa: E402
from llm_inference_lab_amd.weights import random_tensors                 # noqa: E402
import plain_qwen2                                                       # noqa: E402

# Two tiny configurations that differ in every size and option, and a third whose
# heads do not add up to the hidden size.
TINY_A = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=256, hidden_size=64,
              intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
              num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-6, rope_theta=10000.0,
              max_position_embeddings=1024, tie_word_embeddings=True, use_sliding_window=False,
              eos_token_id=255)
TINY_B = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=515, hidden_size=96,
              intermediate_size=320, num_hidden_layers=3, num_attention_heads=3,
              num_key_value_heads=1, head_dim=32, rms_norm_eps=1e-5, rope_theta=1000000.0,
              max_position_embeddings=2048, tie_word_embeddings=False, use_sliding_window=True,
              sliding_window=24, max_window_layers=1, eos_token_id=[3, 4])
TINY_C = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=301, hidden_size=72,
              intermediate_size=200, num_hidden_layers=2, num_attention_heads=6,
              num_key_value_heads=3, head_dim=48, rms_norm_eps=1e-6, rope_theta=50000.0,
              max_position_embeddings=512, tie_word_embeddings=False, use_sliding_window=True,
              sliding_window=40, max_window_layers=0)
# The layer sizes of Qwen2.5-0.5B (two layers, a small odd vocabulary): the kernels'
# choices of block shape at real sizes, end to end.
REAL_LAYER = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=4099, hidden_size=896,
                  intermediate_size=4864, num_hidden_layers=2, num_attention_heads=14,
                  num_key_value_heads=2, head_dim=64, rms_norm_eps=1e-6, rope_theta=1000000.0,
                  max_position_embeddings=8192, tie_word_embeddings=True, use_sliding_window=False)
# The whole Qwen2.5-0.5B shape (24 layers, the real vocabulary), and one layer each with the
# widths of Qwen2.5-7B and Qwen2.5-32B (a small odd vocabulary): the sizes at which the
# kernels' rules for large matrices decide.
FULL_05B = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=151936, hidden_size=896,
                intermediate_size=4864, num_hidden_layers=24, num_attention_heads=14,
                num_key_value_heads=2, head_dim=64, rms_norm_eps=1e-6, rope_theta=1000000.0,
                max_position_embeddings=32768, tie_word_embeddings=True, use_sliding_window=False)
WIDE_7B = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=5003, hidden_size=3584,
               intermediate_size=18944, num_hidden_layers=1, num_attention_heads=28,
               num_key_value_heads=4, head_dim=128, rms_norm_eps=1e-6, rope_theta=1000000.0,
               max_position_embeddings=32768, tie_word_embeddings=False, use_sliding_window=False)
WIDE_32B = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=5003, hidden_size=5120,
                intermediate_size=27648, num_hidden_layers=1, num_attention_heads=40,
                num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-6, rope_theta=1000000.0,
                max_position_embeddings=32768, tie_word_embeddings=False, use_sliding_window=False)
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "R": REAL_LAYER, "F": FULL_05B, "W7": WIDE_7B,
           "W32": WIDE_32B}

# Decided before the first run and not widened since.  Logits of these models are
# of order 1.  float32: sums in another order than the float64 reference.
# bfloat16: activations rounded to 8 bits of mantissa between kernels.
TOL = {"f32": 1e-4, "bf16": 2e-2}
# Layers 896 wide (configuration R): float32 within 1e-3 of the float64 plain implementation
# (sums of 896 to 4864 terms).  For bfloat16 the floor is what rounding the activations to 8
# bits of mantissa at the engine's rounding points costs at this width: the emulation of the
# kernels on the CPU (tests/emu_ops.py, float32 arithmetic, the same roundings) is off the
# plain implementation by 0.09 to 0.10 at most and 0.016 to 0.017 in the root mean square
# over the logits of such sequences; the GPU may be off by half as much again.
TOL_REAL = {"f32": (1e-3, 1e-3), "bf16": (0.15, 0.025)}     # (max, root mean square)


def config_of(name):
    return lab.Qwen2Config.from_dict(dict(CONFIGS[name]))


def expected_tensors(cfg):
    return CausalLM(get_architecture(cfg.architecture).build_spec(cfg)).tensor_specs()


def make_tensors(cfg, seed, sharp=8.0):
    """Random bfloat16 tensors.  The q and k projections are scaled up so that the
    attention is peaked: with the plain N(0, 0.02) scores are nearly uniform and a
    wrong key, mask or page would change the logits by less than the tolerance."""
    tensors = dict(random_tensors(expected_tensors(cfg), seed, torch.bfloat16))
    if cfg.hidden_size > 128:       # (queries and keys grow with the root of the width as well)
        sharp *= (64.0 / cfg.hidden_size) ** 0.5
    for name in tensors:
        if name.endswith("q_proj.weight") or name.endswith("k_proj.weight"):
            tensors[name] = (tensors[name].float() * sharp).to(torch.bfloat16)
        if name.endswith("embed_tokens.weight"):
            # (a wide model's logits would grow with the root of its width: keep them of order 1)
            scale = 10.0 if cfg.hidden_size <= 128 else 10.0 * (64.0 / cfg.hidden_size) ** 0.5
            tensors[name] = (tensors[name].float() * scale).to(torch.bfloat16)
    return tensors


def random_ids(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist()


_PLAIN_CACHE = {}


_PLAIN_WEIGHTS = {}      # the float64 weights of the model asked for last (one model: they are large)


def plain_logits(name, seed, ids):
    key = (name, seed, tuple(ids))
    if key not in _PLAIN_CACHE:
        cfg = config_of(name)
        if (name, seed) not in _PLAIN_WEIGHTS:
            _PLAIN_WEIGHTS.clear()
            _PLAIN_WEIGHTS[(name, seed)] = {k: v.double() for k, v in make_tensors(cfg, seed).items()}
        _PLAIN_CACHE[key] = plain_qwen2.forward_logits(ids, _PLAIN_WEIGHTS[(name, seed)], cfg.to_dict())
    return _PLAIN_CACHE[key]


def make_engine(name, seed, dtype, ops=None, page_size=16, num_pages=32, max_requests=4,
                max_batch_tokens=256, max_seq_len=512, graph=False, device="cuda:0"):
    cfg = config_of(name)
    return lab.Engine(config=cfg, tensors=make_tensors(cfg, seed).items(), dtype=dtype, ops=ops,
                      device=device, page_size=page_size, num_pages=num_pages,
                      max_requests=max_requests, max_batch_tokens=max_batch_tokens,
                      max_seq_len=max_seq_len, graph=graph)


def run_trace(engine, sequences, steps):
    """``sequences``: id -> token list.  ``steps``: list of (entries, ends), an entry being
    (id, count, want_all).  Returns id -> float32 logits [tokens seen, vocab] (rows of
    positions whose logits were not asked for are NaN)."""
    live, done_len, out = {}, {}, {}
    vocab = engine.spec.vocab_size
    for rid, ids in sequences.items():
        out[rid] = torch.full((len(ids), vocab), float("nan"))
    for entries, ends in steps:
        batch, places = [], []
        for rid, count, want_all in entries:
            if rid not in live:
                live[rid] = engine.open(rid)
                done_len[rid] = 0
            start = done_len[rid]
            toks = sequences[rid][start:start + count]
            want = list(range(len(toks))) if want_all else []
            batch.append(lab.StepEntry(live[rid], toks, want))
            places += [(rid, start + w) for w in want]
            done_len[rid] = start + len(toks)
        logits = engine.step(batch)
        if logits is not None:
            logits = logits.float().cpu()
            for row, (rid, pos) in enumerate(places):
                out[rid][pos] = logits[row]
        for rid in ends:
            engine.close(live.pop(rid))
    for rid in list(live):
        engine.close(live.pop(rid))
    return out


def steps_whole(sequences):
    return [([(rid, len(ids), True)], [rid]) for rid, ids in sequences.items()]


def steps_prefill_then_decode(sequences, tail=32):
    steps = []
    for rid, ids in sequences.items():
        head = max(1, len(ids) - tail)
        steps.append(([(rid, head, True)], []))
        for i in range(head, len(ids)):
            steps.append(([(rid, 1, True)], [rid] if i == len(ids) - 1 else []))
        if head == len(ids):
            steps[-1] = (steps[-1][0], [rid])
    return steps


def steps_portions(sequences, sizes=(13, 2, 7, 5, 2, 16, 3, 2, 31, 2, 64, 9)):
    steps = []
    for rid, ids in sequences.items():
        pos, i = 0, 0
        while pos < len(ids):
            n = min(sizes[i % len(sizes)], len(ids) - pos)
            pos += n
            i += 1
            steps.append(([(rid, n, True)], [rid] if pos == len(ids) else []))
    return steps


def steps_mixed(sequences, seed=0, max_live=4, budget=48):
    """Up to ``max_live`` live requests; prompts enter in portions of changing size
    while others decode one token at a time; a finished request makes room for the
    next, so its pages are handed to someone else."""
    g = torch.Generator().manual_seed(seed)
    waiting = list(sequences)
    live, pos, steps = [], {}, []
    decode_from = {rid: max(1, len(ids) - 12) for rid, ids in sequences.items()}
    while waiting or live:
        while waiting and len(live) < max_live:
            rid = waiting.pop(0)
            live.append(rid)
            pos[rid] = 0
        entries, ends = [], []
        left = budget
        for rid in list(live):
            n_left = len(sequences[rid]) - pos[rid]
            if pos[rid] >= decode_from[rid]:
                n = 1
            else:
                n = int(torch.randint(2, 20, (1,), generator=g))
                n = min(n, decode_from[rid] - pos[rid], max(left, 0))
                if n < 2 and decode_from[rid] - pos[rid] >= 2:
                    continue                       # sits this step out
                n = max(n, 1)
            n = min(n, n_left)
            if int(torch.randint(0, 5, (1,), generator=g)) == 0 and len(live) > 1 and entries:
                continue                           # left out of this step, goes on later
            entries.append((rid, n, True))
            left -= n
            pos[rid] += n
            if pos[rid] == len(sequences[rid]):
                ends.append(rid)
                live.remove(rid)
        if entries:
            steps.append((entries, ends))
    return steps


def max_error(got, want):
    """Largest absolute difference over the rows that were asked for."""
    worst = 0.0
    for rid in got:
        rows = ~torch.isnan(got[rid]).any(dim=1)
        assert rows.any(), f"no logits came back for request {rid}"
        worst = max(worst, (got[rid][rows].double() - want[rid][rows]).abs().max().item())
    return worst


def first_wrong(got, want, tol):
    """(request, position, error) of the first position beyond the tolerance, for the
    failure message: what is special about its place says where the fault is."""
    for rid in got:
        for pos in range(got[rid].shape[0]):
            if torch.isnan(got[rid][pos]).any():
                continue
            err = (got[rid][pos].double() - want[rid][pos]).abs().max().item()
            if err > tol:
                return rid, pos, err
    return None


def check_drawn_tokens(name, seed, prompt, generated, temperature, stream_seed, slack=1e-5):
    """Every generated token is the one the plain implementation predicts from the tokens
    before it: the argmax at temperature 0, else the inverse-CDF draw from
    ``softmax(plain logits / temperature)`` at ``uniform(stream_seed, n)`` for the n-th
    token.  A draw closer than ``slack`` to a boundary of the cumulative sums may fall to
    either side (float32 sums on the GPU, float64 here)."""
    from llm_inference_lab_amd.sampling.sampler import uniform
    ids = list(prompt)
    for n, token in enumerate(generated):
        logits = plain_logits(name, seed, ids)[-1]
        if temperature <= 0.0:
            best = plain_qwen2.argmax_smallest_index(logits)
            assert token == best or float(logits[best] - logits[token]) < 1e-4, \
                f"token {n}: {token} is not the argmax {best}"
        else:
            probs = plain_qwen2.temperature_probs(logits, temperature)
            u = uniform(stream_seed, n)
            cdf = torch.cumsum(probs, 0)
            below = float(cdf[token - 1]) if token > 0 else 0.0
            assert below - slack < u <= float(cdf[token]) + slack and float(probs[token]) > 0.0, \
                (f"token {n}: {token} covers ({below}, {float(cdf[token])}], the draw is {u}; "
                 f"plain predicts {plain_qwen2.inverse_cdf_token(probs, u)}")
        ids.append(token)
