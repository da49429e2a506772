"""Plain implementation of the Qwen2 decoder: whole sequences, no cache, one
function for each part, written from the reference's formulas.  It shares no
code with the engine.  ``E`` = rust/engine/src/runner/model/qwen2/engine.rs,
``K`` = rust/engine/src/runner/model/qwen2/kernels.rs of the reference.

Everything is computed in one floating-point type (float64 by default, so that
the engine's float32 path is compared with something more exact than itself).
In that setting the reference's ``cast_T`` roundings are the identity.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def embedding(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """x[r, :] = table[id_r, :]  (K:46-57, E:970-999)."""
    return table[ids.long()]


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """ms = sum_c x_c^2 / H; inv = 1/sqrt(ms + eps); y = (x * inv) * w  (K:546-582)."""
    ms = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    inv = 1.0 / torch.sqrt(ms + eps)
    return (x * inv) * weight


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = x . W^T (+ bias); W is [out, in] as in the checkpoint  (K:156-178, K:393-418)."""
    out = x @ weight.transpose(0, 1)
    if bias is not None:
        out = out + bias
    return out


def rope_inv_freq(head_dim: int, theta: float, dtype=torch.float64) -> torch.Tensor:
    """inv_freq_i = theta^(-2i/d), i in [0, d/2)  (E:304-306)."""
    i = torch.arange(0, head_dim // 2, dtype=dtype)
    return torch.tensor(theta, dtype=dtype) ** (-(2.0 * i) / head_dim)


def rope(x: torch.Tensor, positions: torch.Tensor, theta: float) -> torch.Tensor:
    """Split-half rotation of x [tokens, heads, d]: lo = x[..., :d/2], hi =
    x[..., d/2:], angle = pos * inv_freq; out = [lo*cos - hi*sin, hi*cos + lo*sin]
    (K:587-631)."""
    d = x.shape[-1]
    half = d // 2
    inv_freq = rope_inv_freq(d, theta, x.dtype)
    angles = positions.to(x.dtype)[:, None] * inv_freq[None, :]          # [tokens, d/2]
    c = torch.cos(angles)[:, None, :]
    s = torch.sin(angles)[:, None, :]
    lo, hi = x[..., :half], x[..., half:]
    return torch.cat([lo * c - hi * s, hi * c + lo * s], dim=-1)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, positions: torch.Tensor,
                     window: Optional[int] = None, scale: Optional[float] = None) -> torch.Tensor:
    """q [T, nq, d], k and v [T, nkv, d] of ONE whole sequence.  Head h reads kv
    head h // (nq / nkv) (E:3383).  For the query at position p the keys j with
    hs <= j <= p are visible (K:760-766), hs = max(0, p - window + 1) with a
    window and 0 without; scores s_j = (q . k_j) * scale, scale = 1/sqrt(d)
    (K:744, K:980); out = sum_j softmax(s)_j v_j (K:702-853)."""
    t, nq, d = q.shape
    nkv = k.shape[1]
    group = nq // nkv
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    out = torch.zeros_like(q)
    for h in range(nq):
        kvh = h // group
        for i in range(t):
            p = int(positions[i])
            hs = 0 if window is None else max(0, p - window + 1)
            visible = [j for j in range(t) if hs <= int(positions[j]) <= p]
            scores = torch.stack([(q[i, h] * k[j, kvh]).sum() * scale for j in visible])
            m = scores.max()
            e = torch.exp(scores - m)
            probs = e / e.sum()
            acc = torch.zeros(d, dtype=q.dtype)
            for w, j in zip(probs, visible):
                acc = acc + w * v[j, kvh]
            out[i, h] = acc
    return out


def causal_attention_dense(q, k, v, positions, window=None, scale=None):
    """The same attention with whole-matrix operations (a faster equal of
    ``causal_attention``; the tests check that the two agree)."""
    t, nq, d = q.shape
    nkv = k.shape[1]
    group = nq // nkv
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    kk = k.repeat_interleave(group, dim=1)          # head h -> kv head h // group
    vv = v.repeat_interleave(group, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, kk) * scale
    pi = positions[:, None]
    pj = positions[None, :]
    visible = pj <= pi
    if window is not None:
        visible = visible & (pj >= pi - window + 1)
    scores = scores.masked_fill(~visible[None], float("-inf"))
    m = scores.max(dim=-1, keepdim=True).values
    e = torch.exp(scores - m)
    probs = e / e.sum(dim=-1, keepdim=True)
    return torch.einsum("hij,jhd->ihd", probs, vv)


def silu(z: torch.Tensor) -> torch.Tensor:
    """silu(z) = z / (1 + exp(-z))  (K:1469-1486)."""
    return z / (1.0 + torch.exp(-z))


def swiglu_mlp(x, gate_w, up_w, down_w, cast=None):
    """down( silu(x Wg^T) * (x Wu^T) )  (E:1234-1294).  ``cast``: see ``decoder_layer``."""
    act = silu(linear(x, gate_w)) * linear(x, up_w)
    return linear(act if cast is None else cast(act), down_w)


def layer_window(config: dict, layer: int) -> Optional[int]:
    """Layer l is windowed iff use_sliding_window and l >= max_window_layers
    (not in the reference, which rejects use_sliding_window, E:262)."""
    if config.get("use_sliding_window") and config.get("sliding_window") is not None \
            and layer >= config.get("max_window_layers", config["num_hidden_layers"]):
        return int(config["sliding_window"])
    return None


def decoder_layer(x, positions, w: Dict[str, torch.Tensor], config: dict, layer: int,
                  attention=causal_attention_dense, cast=None):
    """norm -> q/k/v (+bias) -> rope(q, k) -> attention -> o-proj -> add;
    norm -> SwiGLU -> add  (E:1065-1122, E:1133-1296).

    ``cast`` (None: nothing) is applied where the reference stores an activation in its
    storage type ``T`` (its ``cast_T``: the output of a norm K:575-581, q and k after the
    rotation and v K:620-630, the attention output K:846-852, the SwiGLU output K:1484);
    the residual stream and the sums stay as they are.  With ``cast`` rounding to bfloat16
    this is what a bfloat16 engine computes, up to the order of its sums: the tests measure
    the price of those roundings with it."""
    if cast is None:
        cast = lambda t: t
    p = f"model.layers.{layer}."
    nq, nkv = config["num_attention_heads"], config["num_key_value_heads"]
    d = config.get("head_dim") or config["hidden_size"] // nq
    eps, theta = config["rms_norm_eps"], config["rope_theta"]
    t = x.shape[0]
    n = cast(rms_norm(x, w[p + "input_layernorm.weight"], eps))
    q = linear(n, w[p + "self_attn.q_proj.weight"], w[p + "self_attn.q_proj.bias"]).view(t, nq, d)
    k = linear(n, w[p + "self_attn.k_proj.weight"], w[p + "self_attn.k_proj.bias"]).view(t, nkv, d)
    v = cast(linear(n, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"]).view(t, nkv, d))
    q = cast(rope(q, positions, theta))
    k = cast(rope(k, positions, theta))
    a = cast(attention(q, k, v, positions, layer_window(config, layer)).reshape(t, nq * d))
    res = x + linear(a, w[p + "self_attn.o_proj.weight"])
    n2 = cast(rms_norm(res, w[p + "post_attention_layernorm.weight"], eps))
    return res + swiglu_mlp(n2, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                            w[p + "mlp.down_proj.weight"], cast)


def forward_logits(ids: List[int], weights: Dict[str, torch.Tensor], config: dict,
                   dtype=torch.float64, attention=causal_attention_dense, cast=None) -> torch.Tensor:
    """Logits [tokens, vocab] of one whole sequence; the head is the embedding
    table iff tie_word_embeddings (E:299-303); final norm then head (E:1298-1319).
    ``cast``: see ``decoder_layer``."""
    w = {k: v.to(dtype) for k, v in weights.items()}
    ids_t = torch.tensor(list(ids), dtype=torch.long)
    positions = torch.arange(len(ids), dtype=torch.long)
    x = embedding(w["model.embed_tokens.weight"], ids_t)
    for layer in range(config["num_hidden_layers"]):
        x = decoder_layer(x, positions, w, config, layer, attention, cast)
    x = rms_norm(x, w["model.norm.weight"], config["rms_norm_eps"])
    if cast is not None:
        x = cast(x)
    head = w["model.embed_tokens.weight"] if config["tie_word_embeddings"] else w["lm_head.weight"]
    return linear(x, head)


def argmax_smallest_index(logits: torch.Tensor) -> int:
    """Largest value; ties go to the smallest index (K:1489-1552)."""
    best, best_i = None, -1
    for i, v in enumerate(logits.tolist()):
        if best is None or v > best:
            best, best_i = v, i
    return best_i


def greedy_generate(prompt: List[int], steps: int, weights, config, dtype=torch.float64) -> List[int]:
    """Whole-sequence recomputation for every new token."""
    ids = list(prompt)
    out = []
    for _ in range(steps):
        logits = forward_logits(ids, weights, config, dtype)
        nxt = argmax_smallest_index(logits[-1])
        out.append(nxt)
        ids.append(nxt)
    return out


def temperature_probs(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """p = softmax(logits / temperature)."""
    z = logits.to(torch.float64) / temperature
    e = torch.exp(z - z.max())
    return e / e.sum()


def inverse_cdf_token(probs: torch.Tensor, u: float) -> int:
    """The smallest token whose cumulative probability reaches ``u`` (a uniform number
    in [0, 1)); tokens of probability 0 are never chosen."""
    target = u * float(probs.sum())
    run, last = 0.0, -1
    for i, p in enumerate(probs.tolist()):
        if p > 0.0:
            last = i
            run += p
            if run >= target:
                return i
    return last
