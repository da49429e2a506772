"""Configurations drawn at random (every size and option that config.json gives: head
size in steps of 16, heads and groups, widths that are multiples of 8 and nothing else,
odd vocabularies, layers, eps, rope base, windows on some layers, tied or untied head),
each replayed in portions and in mixed batches through a small page pool, in 32-bit and
in bfloat16, against the plain implementation."""
import random

import pytest

import helpers as H

pytestmark = pytest.mark.gpu


def drawn_config(seed):
    r = random.Random(1000 + seed)
    d = 16 * (1 + seed % 8)                       # 16 .. 128: every head size three times
    nkv = r.choice([1, 2, 3])
    group = r.choice([1, 2, 3, 5])
    window = r.choice([None, r.randrange(9, 70)])
    layers = r.choice([1, 2, 3])
    cfg = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=r.randrange(90, 700),
               hidden_size=8 * r.randrange(5, 30), intermediate_size=8 * r.randrange(6, 50),
               num_hidden_layers=layers, num_attention_heads=nkv * group, num_key_value_heads=nkv, head_dim=d,
               rms_norm_eps=r.choice([1e-6, 1e-5, 3e-5]), rope_theta=r.choice([1e4, 5e4, 1e6]),
               max_position_embeddings=1024, tie_word_embeddings=r.random() < 0.5,
               use_sliding_window=window is not None)
    if window is not None:
        cfg.update(sliding_window=window, max_window_layers=r.randrange(0, layers + 1))
    return cfg


_FLOORS = {}


def rounding_floor(seed, name, seqs, want):
    """What rounding to bfloat16 costs this configuration, measured without any code of the
    product: the plain implementation with every stored activation rounded to bfloat16
    where the reference rounds to its storage type (norm outputs, q, k, v, attention and
    SwiGLU outputs; float64 sums), against the plain implementation without."""
    if seed not in _FLOORS:
        import torch
        import plain_qwen2
        cfg = H.config_of(name)
        weights = {k: v.double() for k, v in H.make_tensors(cfg, 2).items()}
        round_bf16 = lambda t: t.to(torch.bfloat16).to(t.dtype)
        _FLOORS[seed] = max(
            float((plain_qwen2.forward_logits(ids, weights, cfg.to_dict(), cast=round_bf16) - want[rid]).abs().max())
            for rid, ids in seqs.items())
    return _FLOORS[seed]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("cut", ["decode", "portions", "mixed"])
@pytest.mark.parametrize("seed", range(24))
def test_drawn_configuration(seed, cut, dtype):
    name = f"Z{seed}"
    H.CONFIGS[name] = drawn_config(seed)
    cfg = H.config_of(name)
    r = random.Random(seed)
    lengths = [r.randrange(1, 20), r.randrange(20, 80), r.randrange(80, 170), r.randrange(2, 120), r.randrange(30, 90)]
    seqs = {f"r{i}": H.random_ids(cfg, n, 900 + 10 * seed + i) for i, n in enumerate(lengths)}
    want = {rid: H.plain_logits(name, 2, ids) for rid, ids in seqs.items()}
    page_size = r.choice([16, 32, 64])
    longest = sorted((len(v) for v in seqs.values()), reverse=True)[:4]
    num_pages = sum((n + page_size - 1) // page_size for n in longest)
    engine = H.make_engine(name, 2, dtype, page_size=page_size, num_pages=num_pages, max_requests=4)
    steps = {"decode": H.steps_prefill_then_decode, "portions": H.steps_portions, "mixed": H.steps_mixed}[cut](seqs)
    got = H.run_trace(engine, seqs, steps)
    # The suite's bounds hold for logits of order 1 to 16 (configurations A to C).  A drawn
    # configuration with a tied head has logits up to 25, and deeper or wider ones round more
    # often.  float32: the bound grows with the largest logit beyond 8.  bfloat16: what the
    # roundings cost for this very configuration is measured with the plain implementation
    # itself (``rounding_floor``: no code of the product, so a mistake of the engine cannot
    # widen its own bound); the GPU may be off by half as much again (its probabilities are
    # rounded too, its sums are float32 in other orders), never by less than the suite's
    # bound allows.
    if dtype == "f32":
        bound = H.TOL[dtype] * max(1.0, max(float(w.abs().max()) for w in want.values()) / 8.0)
    else:
        bound = max(H.TOL[dtype], 1.5 * rounding_floor(seed, name, seqs, want))
    bad = H.first_wrong(got, want, bound)
    assert bad is None, f"{H.CONFIGS[name]}: first wrong logits at (request, position, error) = {bad}"
    engine.cache.check()
    m = engine.cache.metrics()
    assert m["rows_used"] == 0 and all(g["pages_used"] == 0 for g in m["groups"])
