"""What fixes the plain implementation beside the reference's text: special cases
that reduce to a library routine, invariants, and the closed-form vectors of the
reference's own tests.  Each case is chosen so that a plausible mistake (a wrong
sign or pairing in the rotation, a norm in the wrong place, an off-by-one in a
mask or window, the wrong kv head) fails it."""
import math

import pytest
import torch

import helpers as H
import plain_qwen2 as P

F = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F)


# ------------------------------------------------------------------ RMSNorm
def test_rms_norm_unit_weight_gives_unit_rms_and_ignores_scale():
    x = rnd(5, 96, seed=1) * 3
    y = P.rms_norm(x, torch.ones(96, dtype=F), 1e-12)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=F), atol=1e-9)
    assert torch.allclose(P.rms_norm(7.0 * x, torch.ones(96, dtype=F), 1e-12), y, atol=1e-9)
    w = rnd(96, seed=2)
    assert torch.allclose(P.rms_norm(x, w, 1e-5), x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w)
    # eps sits inside the root, beside the mean (not beside the sum, not outside)
    tiny = torch.full((1, 4), 1e-3, dtype=F)
    assert torch.allclose(P.rms_norm(tiny, torch.ones(4, dtype=F), 1e-6), tiny / math.sqrt(1e-6 + 1e-6))


# ------------------------------------------------------------------- linear
def test_linear_reference_vectors():
    """x = ((i*17 % 31) - 15)/32, W = ((i*7 + 11) % 29)/64 - 14/64, b = (i + 7)/128
    (rust/engine/src/runner/model/qwen2/engine.rs:3574-3612), against explicit sums."""
    m, k, n = 3, 96, 65
    x = ((torch.arange(m * k) * 17 % 31) - 15).to(F).view(m, k) / 32
    w = ((torch.arange(n * k) * 7 + 11) % 29).to(F).view(n, k) / 64 - 14 / 64
    b = (torch.arange(n).to(F) + 7) / 128
    got = P.linear(x, w, b)
    for i, j in [(0, 0), (2, 64), (1, 33)]:
        assert abs(got[i, j] - (sum(x[i, c] * w[j, c] for c in range(k)) + b[j])) < 1e-12


# --------------------------------------------------------------------- RoPE
def test_rope_position_zero_is_identity_and_pairs_keep_their_length():
    x = rnd(4, 3, 32, seed=3)
    assert torch.equal(P.rope(x, torch.zeros(4, dtype=torch.long), 1e4), x)
    y = P.rope(x, torch.tensor([1, 17, 300, 4000]), 1e6)
    lo, hi, ylo, yhi = x[..., :16], x[..., 16:], y[..., :16], y[..., 16:]
    assert torch.allclose(lo ** 2 + hi ** 2, ylo ** 2 + yhi ** 2, atol=1e-9)


def test_rope_is_a_complex_rotation_of_split_halves():
    d, theta = 16, 1e4
    x = rnd(5, 2, d, seed=4)
    pos = torch.tensor([0, 1, 2, 50, 1000])
    inv = theta ** (-torch.arange(0, d, 2, dtype=F) / d)
    z = torch.complex(x[..., :d // 2], x[..., d // 2:]) * torch.exp(1j * pos.to(F)[:, None, None] * inv)
    y = P.rope(x, pos, theta)
    assert torch.allclose(y[..., :d // 2], z.real, atol=1e-9) and torch.allclose(y[..., d // 2:], z.imag, atol=1e-9)
    # pairing is (i, i + d/2), not (2i, 2i+1): with only element 0 set, position 1
    # moves weight into element d/2 and nowhere else
    e = torch.zeros(1, 1, d, dtype=F)
    e[0, 0, 0] = 1.0
    r = P.rope(e, torch.tensor([1]), theta)[0, 0]
    assert abs(r[0] - math.cos(1.0)) < 1e-12 and abs(r[d // 2] - math.sin(1.0)) < 1e-12
    assert r[1:d // 2].abs().max() == 0 and r[d // 2 + 1:].abs().max() == 0
    # frequencies fall with the index: the last pair turns by theta^(-(d-2)/d) per position
    e = torch.zeros(1, 1, d, dtype=F)
    e[0, 0, d // 2 - 1] = 1.0
    r = P.rope(e, torch.tensor([1]), theta)[0, 0]
    assert abs(r[d // 2 - 1] - math.cos(theta ** (-(d - 2) / d))) < 1e-12


def test_rope_scores_depend_on_distance_only():
    q, k = rnd(1, 1, 32, seed=5), rnd(1, 1, 32, seed=6)
    def score(p, p2):
        return (P.rope(q, torch.tensor([p]), 1e6) * P.rope(k, torch.tensor([p2]), 1e6)).sum()
    assert abs(score(10, 3) - score(110, 103)) < 1e-9
    assert abs(score(10, 3) - score(3, 10)) > 1e-6              # but on its sign


# ---------------------------------------------------------------- attention
def test_attention_reduces_to_library_softmax_without_mask_effects():
    """The last query sees everything: softmax(q K^T / sqrt(d)) V with the library's softmax."""
    t, d = 9, 16
    q, k, v = rnd(t, 1, d, seed=7), rnd(t, 1, d, seed=8), rnd(t, 1, d, seed=9)
    pos = torch.arange(t)
    out = P.causal_attention(q, k, v, pos)
    want = torch.softmax(q[-1, 0] @ k[:, 0].T / math.sqrt(d), dim=0) @ v[:, 0]
    assert torch.allclose(out[-1, 0], want, atol=1e-12)
    assert torch.allclose(out[0, 0], v[0, 0], atol=1e-12)          # a single visible key: its value
    # equal scores: the mean of the visible values
    out = P.causal_attention(torch.zeros(t, 1, d, dtype=F), k, v, pos)
    assert torch.allclose(out[4, 0], v[:5, 0].mean(0), atol=1e-12)


def test_attention_loop_and_dense_forms_agree_on_reference_vectors():
    """q = ((i*13 % 89) - 44)*0.01, k = ((i*7 + r*11) % 97)*0.003 - 0.144, v = ((i*17 + r*29)
    % 103)*0.01 - 0.51 (rust/engine/src/runner/model/qwen2/engine.rs:3248-3279)."""
    t, nq, nkv, d = 33, 4, 2, 16
    i = torch.arange(d)
    q = torch.stack([torch.stack([(((i + 3 * h + r) * 13 % 89) - 44).to(F) * 0.01 for h in range(nq)]) for r in range(t)])
    k = torch.stack([torch.stack([((i * 7 + (r + 5 * h) * 11) % 97).to(F) * 0.003 - 0.144 for h in range(nkv)]) for r in range(t)])
    v = torch.stack([torch.stack([((i * 17 + (r + 2 * h) * 29) % 103).to(F) * 0.01 - 0.51 for h in range(nkv)]) for r in range(t)])
    pos = torch.arange(t)
    for window in (None, 1, 7, 33, 100):
        a = P.causal_attention(q, k, v, pos, window)
        b = P.causal_attention_dense(q, k, v, pos, window)
        assert torch.allclose(a, b, atol=1e-12)


def test_attention_head_to_kv_head_mapping():
    t, nq, nkv, d = 6, 6, 3, 8
    q, k, v = rnd(t, nq, d, seed=10), rnd(t, nkv, d, seed=11), rnd(t, nkv, d, seed=12)
    out = P.causal_attention(q, k, v, torch.arange(t))
    for h in range(nq):
        alone = P.causal_attention(q[:, h:h + 1], k[:, h // 2:h // 2 + 1], v[:, h // 2:h // 2 + 1], torch.arange(t))
        assert torch.allclose(out[:, h], alone[:, 0], atol=1e-12)      # heads 2g, 2g+1 share kv head g


def test_window_edges():
    t, d = 12, 8
    q, k, v = rnd(t, 2, d, seed=13), rnd(t, 1, d, seed=14), rnd(t, 1, d, seed=15)
    pos = torch.arange(t)
    full = P.causal_attention(q, k, v, pos)
    assert torch.allclose(P.causal_attention(q, k, v, pos, window=t), full, atol=1e-12)
    assert torch.allclose(P.causal_attention(q, k, v, pos, window=1), v.expand(t, 2, d), atol=1e-12)
    # window w: exactly the keys p-w+1 .. p.  Moving key p-w far away changes nothing; key p-w+1 does.
    w, p = 4, 9
    base = P.causal_attention(q, k, v, pos, window=w)[p]
    k2 = k.clone(); k2[p - w] += 100.0
    assert torch.allclose(P.causal_attention(q, k2, v, pos, window=w)[p], base, atol=1e-12)
    k3 = k.clone(); k3[p - w + 1] += 100.0
    assert not torch.allclose(P.causal_attention(q, k3, v, pos, window=w)[p], base, atol=1e-6)
    # the future is never seen
    k4 = k.clone(); k4[p + 1] += 100.0
    assert torch.allclose(P.causal_attention(q, k4, v, pos, window=w)[p], base, atol=1e-12)


# ------------------------------------------------------------- feed-forward
def test_silu_and_swiglu():
    assert P.silu(torch.tensor(0.0, dtype=F)) == 0
    assert abs(P.silu(torch.tensor(30.0, dtype=F)) - 30.0) < 1e-9
    assert abs(P.silu(torch.tensor(-30.0, dtype=F))) < 1e-9
    x, g, u, dn = rnd(3, 8, seed=16), rnd(12, 8, seed=17), rnd(12, 8, seed=18), rnd(8, 12, seed=19)
    gate = x @ g.T
    assert torch.allclose(P.swiglu_mlp(x, g, u, dn), (torch.nn.functional.silu(gate) * (x @ u.T)) @ dn.T, atol=1e-12)
    # gate and up are not interchangeable
    assert not torch.allclose(P.swiglu_mlp(x, g, u, dn), P.swiglu_mlp(x, u, g, dn), atol=1e-6)


# -------------------------------------------------------------- whole model
def weights64(name, seed=1):
    cfg = H.config_of(name)
    return cfg, {k: v.to(F) for k, v in H.make_tensors(cfg, seed).items()}


def test_layer_with_zero_output_weights_is_identity():
    cfg, w = weights64("A")
    for key in list(w):
        if key.endswith("o_proj.weight") or key.endswith("down_proj.weight"):
            w[key] = torch.zeros_like(w[key])
    x = rnd(5, 64, seed=20)
    assert torch.equal(P.decoder_layer(x, torch.arange(5), w, cfg.to_dict(), 0), x)


def test_tied_and_untied_heads():
    cfg, w = weights64("A")
    ids = H.random_ids(cfg, 6, 0)
    tied = P.forward_logits(ids, w, cfg.to_dict())
    raw = dict(cfg.to_dict(), tie_word_embeddings=False)
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"]
    assert torch.allclose(P.forward_logits(ids, w2, raw), tied)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"] * 2
    assert torch.allclose(P.forward_logits(ids, w2, raw), 2 * tied)


def test_logits_depend_on_distances_not_on_absolute_positions():
    """Shifting every position by a constant changes nothing: positions enter only
    through rotated q.k products (checked on one layer's output)."""
    cfg, w = weights64("B")
    x = rnd(7, 96, seed=21)
    a = P.decoder_layer(x, torch.arange(7), w, cfg.to_dict(), 1)
    b = P.decoder_layer(x, torch.arange(7) + 1000, w, cfg.to_dict(), 1)
    assert torch.allclose(a, b, atol=1e-8)


def test_causality_and_window_of_the_whole_model():
    cfg, w = weights64("B")
    ids = H.random_ids(cfg, 40, 2)
    base = P.forward_logits(ids, w, cfg.to_dict())
    changed = list(ids)
    changed[30] = (changed[30] + 1) % cfg.vocab_size
    other = P.forward_logits(changed, w, cfg.to_dict())
    assert torch.allclose(base[:30], other[:30], atol=1e-12)       # the past does not see the future
    assert not torch.allclose(base[30], other[30], atol=1e-6)
    # layer 0 is full attention, so the first token still reaches the last position
    changed = list(ids)
    changed[0] = (changed[0] + 1) % cfg.vocab_size
    assert not torch.allclose(P.forward_logits(changed, w, cfg.to_dict())[-1], base[-1], atol=1e-9)
    # with every layer windowed (config C: window 40, all layers) a token 40 back is out of reach
    cfgc, wc = weights64("C")
    ids = H.random_ids(cfgc, 90, 3)
    base = P.forward_logits(ids, wc, cfgc.to_dict())
    changed = list(ids)
    changed[5] = (changed[5] + 1) % cfgc.vocab_size
    other = P.forward_logits(changed, wc, cfgc.to_dict())
    reach = 5 + cfgc.num_hidden_layers * (40 - 1)                    # each layer carries it 39 further
    assert torch.allclose(base[reach + 1:], other[reach + 1:], atol=1e-12)
    assert not torch.allclose(base[5 + 39], other[5 + 39], atol=1e-9)


def test_argmax_vectors():
    """rust/engine/src/runner/model/qwen2/engine.rs:2289-2349."""
    v = torch.zeros(300)
    v[299] = 1.0
    assert P.argmax_smallest_index(v) == 299
    v = torch.zeros(5000)
    v[4097] = v[7] = 3.0
    assert P.argmax_smallest_index(v) == 7
    assert P.argmax_smallest_index(torch.full((10,), float("-inf"))) == 0


def test_temperature_probabilities():
    logits = torch.tensor([1.0, 0.0, -1.0, 2.0])
    assert torch.allclose(P.temperature_probs(logits, 0.5), torch.softmax(logits.double() / 0.5, 0))
    assert P.temperature_probs(logits, 1e-3).argmax() == 3
