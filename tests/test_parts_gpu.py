"""Each part alone against the plain function of the same name, and a toy mixer
with state of its own (defined here, not in the framework) registered, built
and stepped without a change to the framework's files."""
import dataclasses
import math

import pytest
import torch

import helpers as H
import plain_qwen2 as P
from llm_inference_lab_amd.config import (BlockSpec, ModelSpec, PartSpec, ScheduleEntry,
                                          register_architecture, unregister_architecture)
from llm_inference_lab_amd.parts import (CacheSpec, Mixer, PageTensor, Part, RMSNorm, RotaryEmbedding, SwiGLU,
                                         TokenEmbedding, LinearHead, register_part, build_part)
from llm_inference_lab_amd.parts.registry import unregister_part
from llm_inference_lab_amd.weights import TensorSpec, MATRIX

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from llm_inference_lab_amd.kernels.hip_ops import HipOps
    return HipOps(DEV)


class Scratch:
    """The part of a step context that parts without a cache need."""

    def __init__(self):
        self.bufs = {}

    def scratch(self, name, shape, dtype):
        key = (name, tuple(shape), dtype)
        if key not in self.bufs:
            self.bufs[key] = torch.empty(shape, dtype=dtype, device=DEV)
        return self.bufs[key]


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


TOLS = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(ops, dtype):
    norm = RMSNorm(size=96, eps=1e-5, tensors={"weight": "w"})
    w = (1 + 0.1 * rnd((96,), 1)).to(torch.bfloat16)
    norm.bind({"w": w.to(DEV)}, ops, dtype)
    x = rnd((11, 96), 2, 2.0)
    out = torch.empty(11, 96, dtype=dtype, device=DEV)
    norm.forward(x.to(DEV), out)
    want = P.rms_norm(x.double(), w.double(), 1e-5)
    assert (out.double().cpu() - want).abs().max() < TOLS[dtype] * 4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotary_part_general_path(ops, dtype):
    rope = RotaryEmbedding(dim=32, theta=1e6)
    rope.bind({}, ops, dtype)
    q, k = rnd((9, 3, 32), 3).to(dtype), rnd((9, 1, 32), 4).to(dtype)
    pos = torch.tensor([0, 1, 2, 3, 100, 1000, 4095, 7, 8], dtype=torch.int32)
    qd, kd = q.to(DEV), k.to(DEV)
    rope.apply(qd, kd, pos.to(DEV))
    assert (qd.double().cpu() - P.rope(q.double(), pos.long(), 1e6)).abs().max() < TOLS[dtype] * 4
    assert (kd.double().cpu() - P.rope(k.double(), pos.long(), 1e6)).abs().max() < TOLS[dtype] * 4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_part(ops, dtype):
    ffn = SwiGLU(hidden_size=72, intermediate_size=200,
                 tensors=dict(gate_weight="g", up_weight="u", down_weight="d"))
    g, u, d = (rnd(s, i, 0.2).to(torch.bfloat16) for i, s in enumerate([(200, 72), (200, 72), (72, 200)]))
    ffn.bind({"g": g.to(dtype).to(DEV), "u": u.to(dtype).to(DEV), "d": d.to(dtype).to(DEV)}, ops, dtype)
    x = rnd((13, 72), 5).to(torch.bfloat16)
    resid = rnd((13, 72), 6)
    got = resid.clone().to(DEV)
    ffn.forward(x.to(dtype).to(DEV), got, Scratch())
    want = resid.double() + P.swiglu_mlp(x.double(), g.double(), u.double(), d.double())
    assert (got.double().cpu() - want).abs().max() < TOLS[dtype] * 4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_and_head_parts(ops, dtype):
    table = rnd((301, 72), 7).to(torch.bfloat16)
    emb = TokenEmbedding(vocab_size=301, hidden_size=72, tensors={"weight": "t"})
    head = LinearHead(vocab_size=301, hidden_size=72, tensors={"weight": "t"})
    loaded = {"t": table.to(dtype).to(DEV)}
    emb.bind(loaded, ops, dtype)
    head.bind(loaded, ops, dtype)
    assert head.weight.data_ptr() == emb.table.data_ptr()            # tied: one tensor
    ids = torch.tensor([0, 300, 17, 17], dtype=torch.int32)
    x = torch.empty(4, 72, device=DEV)
    emb.forward(ids.to(DEV), x)
    assert torch.equal(x.cpu(), table.float()[ids.long()])
    h = rnd((4, 72), 8).to(torch.bfloat16)
    logits = torch.empty(4, 301, device=DEV)
    head.forward(h.to(dtype).to(DEV), logits)
    assert (logits.double().cpu() - P.linear(h.double(), table.double())).abs().max() < 1e-3


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("name,layer", [("A", 0), ("B", 0), ("B", 2), ("C", 1)])
def test_block_alone(dtype, name, layer):
    """One decoder layer (norm, attention with its cache, norm, feed-forward) on a
    random residual stream, in two portions, against the plain layer."""
    cfg = H.config_of(name)
    engine = H.make_engine(name, 1, dtype, page_size=16, num_pages=8)
    tensors = {k: v.double() for k, v in H.make_tensors(cfg, 1).items()}
    x = rnd((50, cfg.hidden_size), 9, 2.0)
    want = P.decoder_layer(x.double(), torch.arange(50), tensors, cfg.to_dict(), layer)
    req = engine.open("x")
    view = engine.model.entries[layer]
    block = engine.model.blocks[view.block]
    outs = []
    for lo, hi in ((0, 33), (33, 50)):
        engine.cache.reserve(req, hi - lo)
        engine.step_fn.ctx.fill([H.lab.StepEntry(req, [0] * (hi - lo), [])], engine.cache)
        resid = x[lo:hi].clone().to(DEV)
        block.forward(resid, engine.step_fn.ctx, view)
        engine.cache.commit(req)
        outs.append(resid.cpu())
    got = torch.cat(outs)
    tol = 2e-4 if dtype == "f32" else 5e-2
    assert (got.double() - want).abs().max() < tol * max(1.0, want.abs().max().item() / 4)
    engine.close(req)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("name,layer,cuts", [("A", 1, (0, 40, 41, 42, 50)), ("B", 2, (0, 2, 35, 50)),
                                             ("C", 0, (0, 50))])
def test_attention_part_alone(dtype, name, layer, cuts):
    """The attention mixer alone, handed activations that are normed already (so its
    fused-norm kernel is not the one that runs): projections with bias, rotation,
    cache, attention (with the layer's window, if it has one), output projection
    and the sum into the residual rows, over portions and single tokens."""
    cfg = H.config_of(name)
    conf = cfg.to_dict()
    engine = H.make_engine(name, 2, dtype, page_size=16, num_pages=8)
    w = {k: v.double() for k, v in H.make_tensors(cfg, 2).items()}
    nq, nkv = cfg.num_attention_heads, cfg.num_key_value_heads
    d = conf.get("head_dim") or cfg.hidden_size // nq
    t = cuts[-1]
    h = rnd((t, cfg.hidden_size), 12).to(torch.bfloat16)          # what a norm would have left
    resid = rnd((t, cfg.hidden_size), 13, 2.0)
    p = f"model.layers.{layer}.self_attn."
    hd, pos = h.double(), torch.arange(t)
    q = P.rope(P.linear(hd, w[p + "q_proj.weight"], w[p + "q_proj.bias"]).view(t, nq, d), pos, conf["rope_theta"])
    k = P.rope(P.linear(hd, w[p + "k_proj.weight"], w[p + "k_proj.bias"]).view(t, nkv, d), pos, conf["rope_theta"])
    v = P.linear(hd, w[p + "v_proj.weight"], w[p + "v_proj.bias"]).view(t, nkv, d)
    a = P.causal_attention_dense(q, k, v, pos, P.layer_window(conf, layer)).reshape(t, nq * d)
    want = resid.double() + P.linear(a, w[p + "o_proj.weight"])

    req = engine.open("x")
    view = engine.model.entries[layer]
    mixer = engine.model.blocks[view.block].mixer
    outs = []
    for lo, hi in zip(cuts, cuts[1:]):
        engine.cache.reserve(req, hi - lo)
        engine.step_fn.ctx.fill([H.lab.StepEntry(req, [0] * (hi - lo), [])], engine.cache)
        rows = resid[lo:hi].clone().to(DEV)
        mixer.forward(h[lo:hi].to(mixer.dtype).to(DEV), rows, engine.step_fn.ctx, view)
        engine.cache.commit(req)
        outs.append(rows.cpu())
    got = torch.cat(outs)
    tol = 2e-4 if dtype == "f32" else 5e-2
    assert (got.double() - want).abs().max() < tol * max(1.0, want.abs().max().item() / 4)
    engine.close(req)


# ---------------------------------------------------------------- toy mixer
class RunningMean(Mixer):
    """A mixer with state of fixed size and no cache: the output at a token is a
    projection of the mean of all inputs of its request so far.  The state (sum
    and count) lives in the cache manager's per-request slots."""

    graph_safe = False        # it finds its state rows through host lists: not for a replayed graph

    def __init__(self, hidden_size, tensors):
        super().__init__(tensors)
        self.hidden_size = hidden_size
        self.weight = None

    def tensor_specs(self):
        return {self.tensor_names["weight"]: TensorSpec((self.hidden_size, self.hidden_size), MATRIX)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        self.weight = ops.prepare_weight(tensors[self.tensor_names["weight"]])

    def state_spec(self):
        return {"sum": ((self.hidden_size,), torch.float32), "count": ((1,), torch.float32)}

    def forward(self, h, residual, ctx, entry):
        total, count = entry.state["sum"], entry.state["count"]
        mean = torch.empty(h.shape, dtype=torch.float32, device=h.device)
        for b in range(ctx.n_reqs):
            r0, r1, slot = ctx.host_q_start[b], ctx.host_q_start[b + 1], ctx.host_req_rows[b]
            run = total[slot] + torch.cumsum(h[r0:r1].float(), dim=0)
            n = count[slot] + torch.arange(1, r1 - r0 + 1, device=h.device, dtype=torch.float32)[:, None]
            mean[r0:r1] = run / n
            total[slot] = run[-1]
            count[slot] = n[-1]
        self.ops.linear_residual(mean.to(self.dtype), self.weight, residual)


@dataclasses.dataclass(frozen=True)
class ToyConfig:
    vocab_size: int
    hidden_size: int
    eps: float
    architecture: str = "ToyForCausalLM"

    @classmethod
    def from_dict(cls, raw, where="config.json"):
        return cls(raw["vocab_size"], raw["hidden_size"], raw["eps"])

    def to_dict(self):
        return {"architectures": [self.architecture], "vocab_size": self.vocab_size,
                "hidden_size": self.hidden_size, "eps": self.eps}


def toy_spec(cfg):
    h = cfg.hidden_size
    norm = lambda n: PartSpec("rmsnorm", dict(size=h, eps=cfg.eps), dict(weight=n))
    ffn = lambda p: PartSpec("swiglu", dict(hidden_size=h, intermediate_size=2 * h),
                             dict(gate_weight=p + "gate", up_weight=p + "up", down_weight=p + "down"))
    toy = BlockSpec("prenorm", dict(
        mixer=PartSpec("toy_running_mean", dict(hidden_size=h), dict(weight="l0.mix")),
        feed_forward=ffn("l0."), norm1=norm("l0.n1"), norm2=norm("l0.n2")), params=dict(hidden_size=h))
    attn = BlockSpec("prenorm", dict(mixer=PartSpec(
        "gqa_attention", dict(hidden_size=h, num_heads=2, num_kv_heads=1, head_dim=h // 2, qkv_bias=False,
                              position=None, window=None),
        dict(q_weight="l1.q", k_weight="l1.k", v_weight="l1.v", o_weight="l1.o")),
        feed_forward=ffn("l1."), norm1=norm("l1.n1"), norm2=norm("l1.n2")), params=dict(hidden_size=h))
    sizes = dict(vocab_size=cfg.vocab_size, hidden_size=h)
    return ModelSpec("ToyForCausalLM", cfg.vocab_size, h, 4096,
                     PartSpec("token_embedding", sizes, dict(weight="embed")), (toy, attn),
                     # the toy block runs twice: two runs, two states
                     (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0)),
                     norm("final"), PartSpec("linear_head", sizes, dict(weight="embed")))


def toy_plain(ids, w, cfg):
    """Whole-sequence reference of the toy model, float64."""
    h = cfg.hidden_size
    x = w["embed"][torch.tensor(ids)]
    t = len(ids)
    def toy_block(x):
        n = P.rms_norm(x, w["l0.n1"], cfg.eps)
        mean = torch.cumsum(n, 0) / torch.arange(1, t + 1, dtype=x.dtype)[:, None]
        x = x + P.linear(mean, w["l0.mix"])
        return x + P.swiglu_mlp(P.rms_norm(x, w["l0.n2"], cfg.eps), w["l0.gate"], w["l0.up"], w["l0.down"])
    x = toy_block(x)
    n = P.rms_norm(x, w["l1.n1"], cfg.eps)
    q = P.linear(n, w["l1.q"]).view(t, 2, h // 2)
    k = P.linear(n, w["l1.k"]).view(t, 1, h // 2)
    v = P.linear(n, w["l1.v"]).view(t, 1, h // 2)
    a = P.causal_attention_dense(q, k, v, torch.arange(t)).reshape(t, h)      # no position encoding
    x = x + P.linear(a, w["l1.o"])
    x = x + P.swiglu_mlp(P.rms_norm(x, w["l1.n2"], cfg.eps), w["l1.gate"], w["l1.up"], w["l1.down"])
    x = toy_block(x)
    return P.linear(P.rms_norm(x, w["final"], cfg.eps), w["embed"])


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_toy_mixer_with_state_is_registered_built_and_stepped(dtype):
    register_part("mixer", "toy_running_mean", RunningMean, replace=True)
    register_architecture("ToyForCausalLM", ToyConfig, toy_spec, replace=True)
    try:
        cfg = ToyConfig(vocab_size=97, hidden_size=64, eps=1e-5)
        from llm_inference_lab_amd.engine.model import CausalLM
        from llm_inference_lab_amd.weights import random_tensors
        tensors = dict(random_tensors(CausalLM(toy_spec(cfg)).tensor_specs(), 3, torch.bfloat16))
        for n in ("embed", "l1.q", "l1.k"):
            tensors[n] = (tensors[n].float() * 8).to(torch.bfloat16)
        engine = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype=dtype, page_size=16, num_pages=16,
                              max_requests=3, max_batch_tokens=128, max_seq_len=256)
        groups, states = engine.model.cache_layout()
        assert len(groups) == 1 and groups[0].entries == [1] and sorted(states) == [0, 2]
        g = torch.Generator().manual_seed(0)
        seqs = {f"r{i}": torch.randint(0, 97, (n,), generator=g).tolist() for i, n in enumerate([45, 80, 23, 60])}
        w64 = {k: v.double() for k, v in tensors.items()}
        want = {rid: toy_plain(ids, w64, cfg) for rid, ids in seqs.items()}
        for steps in (H.steps_whole(seqs), H.steps_portions(seqs), H.steps_mixed(seqs, seed=2, max_live=3)):
            got = H.run_trace(engine, seqs, steps)
            bad = H.first_wrong(got, want, H.TOL[dtype])
            assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
        # Graphs asked for: the mixer says that it cannot be captured (it indexes its state
        # with host lists, which a replay would freeze), so the model's decode steps run
        # eagerly and are right; the same model without that mixer's word would be captured.
        assert not engine.model.graph_safe
        graphed = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype=dtype, page_size=16, num_pages=16,
                               max_requests=3, max_batch_tokens=128, max_seq_len=256, graph=True)
        three = {rid: seqs[rid] for rid in ("r0", "r1", "r3")}
        steps = [([(rid, 12, True) for rid in three], [])]
        steps += [([(rid, 1, True) for rid in three], []) for _ in range(30)]
        got = H.run_trace(graphed, three, steps)
        assert graphed.step_fn.use_graph is True
        assert graphed.step_fn.graph_captures == 0 and graphed.step_fn.graph_replays == 0
        for rid in three:
            assert (got[rid][:42].double() - want[rid][:42]).abs().max() <= H.TOL[dtype]
    finally:
        unregister_part("mixer", "toy_running_mean")
        unregister_architecture("ToyForCausalLM")


# ------------------------------------- toy feed-forward with routing, toy position encoding
from llm_inference_lab_amd.parts import FeedForward, PositionEncoding    # noqa: E402


class TopOneExperts(FeedForward):
    """A feed-forward with routing: router logits in float32, the best of E experts
    per token, each expert one square matrix; the expert's output is scaled by the
    router's softmax weight.  Rows are gathered per expert, multiplied by the
    framework's product kernel, and scattered back into the residual."""

    def __init__(self, hidden_size, num_experts, tensors):
        super().__init__(tensors)
        self.hidden_size, self.num_experts = hidden_size, num_experts

    def tensor_specs(self):
        t, h = self.tensor_names, self.hidden_size
        specs = {t["router"]: TensorSpec((self.num_experts, h), MATRIX)}
        for e in range(self.num_experts):
            specs[f'{t["experts"]}.{e}'] = TensorSpec((h, h), MATRIX)
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        t = self.tensor_names
        self.router = tensors[t["router"]].float()
        self.experts = [ops.prepare_weight(tensors[f'{t["experts"]}.{e}']) for e in range(self.num_experts)]

    def forward(self, h, residual, ctx):
        logits = h.float() @ self.router.t()                      # float32 router
        weight, choice = torch.softmax(logits, dim=-1).max(dim=-1)
        for e in range(self.num_experts):
            rows = torch.nonzero(choice == e).flatten()
            if rows.numel() == 0:
                continue
            out = torch.zeros(rows.numel(), self.hidden_size, dtype=torch.float32, device=h.device)
            self.ops.linear_residual(h[rows].contiguous(), self.experts[e], out)
            residual.index_add_(0, rows, out * weight[rows, None])


class HalfRotary(PositionEncoding):
    """Another position encoding: only the first half of every head is rotated
    (pairs (i, i + d/4) of that half), the second half carries no position."""

    def __init__(self, dim, theta, tensors=None):
        super().__init__(tensors)
        self.dim, self.theta = dim, theta

    def tensor_specs(self):
        return {}

    def rotary_table(self):
        return None                      # not the split-half rotation the fused kernel applies

    def apply(self, q, k, positions):
        r = self.dim // 2
        inv = 1.0 / (self.theta ** (torch.arange(0, r, 2, dtype=torch.float64, device=q.device) / r))
        ang = positions.double()[:, None] * inv[None, :]
        cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
        for x in (q, k):
            lo, hi = x[..., :r // 2].double(), x[..., r // 2:r].double()
            x[..., :r // 2] = (lo * cos - hi * sin).to(x.dtype)
            x[..., r // 2:r] = (hi * cos + lo * sin).to(x.dtype)


@dataclasses.dataclass(frozen=True)
class Toy2Config:
    vocab_size: int
    hidden_size: int
    num_experts: int
    theta: float
    eps: float
    architecture: str = "Toy2ForCausalLM"

    @classmethod
    def from_dict(cls, raw, where="config.json"):
        return cls(raw["vocab_size"], raw["hidden_size"], raw["num_experts"], raw["theta"], raw["eps"])

    def to_dict(self):
        return {"architectures": [self.architecture], **dataclasses.asdict(self)}


def toy2_spec(cfg):
    h = cfg.hidden_size
    norm = lambda n: PartSpec("rmsnorm", dict(size=h, eps=cfg.eps), dict(weight=n))
    block = BlockSpec(
        "prenorm", dict(
            mixer=PartSpec("gqa_attention",
                           dict(hidden_size=h, num_heads=2, num_kv_heads=2, head_dim=h // 2, qkv_bias=False,
                                position=PartSpec("toy_half_rotary", dict(dim=h // 2, theta=cfg.theta)), window=None),
                           dict(q_weight="q", k_weight="k", v_weight="v", o_weight="o")),
            feed_forward=PartSpec("toy_top_one_experts", dict(hidden_size=h, num_experts=cfg.num_experts),
                                  dict(router="router", experts="expert")),
            norm1=norm("n1"), norm2=norm("n2")), params=dict(hidden_size=h))
    sizes = dict(vocab_size=cfg.vocab_size, hidden_size=h)
    return ModelSpec("Toy2ForCausalLM", cfg.vocab_size, h, 4096,
                     PartSpec("token_embedding", sizes, dict(weight="embed")), (block,),
                     (ScheduleEntry(0),), norm("final"), PartSpec("linear_head", sizes, dict(weight="head")))


def toy2_plain(ids, w, cfg):
    h, t = cfg.hidden_size, len(ids)
    d, r = h // 2, h // 4
    x = w["embed"][torch.tensor(ids)]
    n = P.rms_norm(x, w["n1"], cfg.eps)
    q, k, v = (P.linear(n, w[s]).view(t, 2, d) for s in "qkv")
    inv = 1.0 / (cfg.theta ** (torch.arange(0, r, 2, dtype=torch.float64) / r))
    ang = torch.arange(t, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    def rot(y):
        y = y.clone()
        lo, hi = y[..., :r // 2].clone(), y[..., r // 2:r].clone()
        y[..., :r // 2], y[..., r // 2:r] = lo * cos - hi * sin, hi * cos + lo * sin
        return y
    a = P.causal_attention_dense(rot(q), rot(k), v, torch.arange(t)).reshape(t, h)
    x = x + P.linear(a, w["o"])
    n = P.rms_norm(x, w["n2"], cfg.eps)
    probs = torch.softmax(P.linear(n, w["router"]), dim=-1)
    weight, choice = probs.max(dim=-1)
    y = torch.stack([P.linear(n[i:i + 1], w[f"expert.{int(choice[i])}"])[0] * weight[i] for i in range(t)])
    x = x + y
    return P.linear(P.rms_norm(x, w["final"], cfg.eps), w["head"])


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_toy_routed_feed_forward_and_other_position_encoding(dtype):
    """A feed-forward with routing and a position encoding of another kind, both
    defined here, are registered, built into an architecture and stepped in every
    cut without a change to the framework's files."""
    register_part("feed_forward", "toy_top_one_experts", TopOneExperts, replace=True)
    register_part("position", "toy_half_rotary", HalfRotary, replace=True)
    register_architecture("Toy2ForCausalLM", Toy2Config, toy2_spec, replace=True)
    try:
        cfg = Toy2Config(vocab_size=61, hidden_size=64, num_experts=3, theta=100.0, eps=1e-6)
        from llm_inference_lab_amd.engine.model import CausalLM
        from llm_inference_lab_amd.weights import random_tensors
        tensors = dict(random_tensors(CausalLM(toy2_spec(cfg)).tensor_specs(), 5, torch.bfloat16))
        for n in ("embed", "q", "k"):
            tensors[n] = (tensors[n].float() * 8).to(torch.bfloat16)
        # a decisive router: the best expert wins by a margin that bfloat16 rounding cannot turn
        tensors["router"] = (tensors["router"].float() * 40).to(torch.bfloat16)
        engine = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype=dtype, page_size=16, num_pages=16,
                              max_requests=3, max_batch_tokens=128, max_seq_len=256)
        g = torch.Generator().manual_seed(1)
        seqs = {f"r{i}": torch.randint(0, 61, (n,), generator=g).tolist() for i, n in enumerate([40, 70, 19])}
        w64 = {k: v.double() for k, v in tensors.items()}
        want = {rid: toy2_plain(ids, w64, cfg) for rid, ids in seqs.items()}
        for steps in (H.steps_whole(seqs), H.steps_portions(seqs), H.steps_mixed(seqs, seed=3, max_live=3)):
            got = H.run_trace(engine, seqs, steps)
            bad = H.first_wrong(got, want, H.TOL[dtype])
            assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
    finally:
        unregister_part("feed_forward", "toy_top_one_experts")
        unregister_part("position", "toy_half_rotary")
        unregister_architecture("Toy2ForCausalLM")


# ------------------- toy embedding that reads positions, toy mixer with a cache of its own shape
class PositionalEmbedding(Part):
    """``x = table[id] + places[position]``: a learned table of absolute positions beside
    the token table.  It needs the step's positions, which the embedding part is handed
    with the step's description."""

    def __init__(self, vocab_size, hidden_size, max_positions, tensors):
        super().__init__(tensors)
        self.vocab_size, self.hidden_size, self.max_positions = vocab_size, hidden_size, max_positions

    def tensor_specs(self):
        t = self.tensor_names
        return {t["weight"]: TensorSpec((self.vocab_size, self.hidden_size), MATRIX),
                t["places"]: TensorSpec((self.max_positions, self.hidden_size), MATRIX)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        self.table = ops.prepare_weight(tensors[self.tensor_names["weight"]], shared=True)
        self.places = tensors[self.tensor_names["places"]].float()

    def forward(self, ids, out, ctx=None):
        self.ops.embed(self.table, ids, out)
        out += self.places[ctx.positions.long()]


class LatentMixer(Mixer):
    """A mixer that keeps ONE vector of width r per token (not keys and values): c = h Wc^T
    goes to the cache, and the output at a token is ``(softmax(q . c_j / sqrt(r)) c) Wo^T``
    over the tokens j up to it, with q = h Wq^T.  Its cache is a page tensor ``[P, r]`` under
    the name "latent"; it finds pages through the group's block table like attention does."""

    graph_safe = False

    def __init__(self, hidden_size, latent_size, tensors):
        super().__init__(tensors)
        self.hidden_size, self.latent_size = hidden_size, latent_size

    def tensor_specs(self):
        t, h, r = self.tensor_names, self.hidden_size, self.latent_size
        return {t["down"]: TensorSpec((r, h), MATRIX), t["query"]: TensorSpec((r, h), MATRIX),
                t["up"]: TensorSpec((h, r), MATRIX)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        t = self.tensor_names
        self.w_down, self.w_query, self.w_up = (ops.prepare_weight(tensors[t[n]].contiguous())
                                                for n in ("down", "query", "up"))

    def cache_spec(self):
        return CacheSpec((("latent", PageTensor((self.latent_size,), 0)),), window=None)

    def forward(self, h, residual, ctx, entry):
        rows, r = h.shape[0], self.latent_size
        group = ctx.group(entry.group)
        page = group.page_size
        c = ctx.scratch("latent.c", (rows, r), self.dtype)
        q = ctx.scratch("latent.q", (rows, r), self.dtype)
        self.ops.linear(h, self.w_down, c)
        self.ops.linear(h, self.w_query, q)
        store = entry.cache["latent"]                                  # [pages, P, r]
        pos = ctx.positions.long()
        pages = group.block_table[ctx.row_req.long(), pos // page].long()
        store[pages, pos % page] = c
        mixed = torch.empty((rows, r), dtype=torch.float32, device=h.device)
        for b in range(ctx.n_reqs):
            r0, r1 = ctx.host_q_start[b], ctx.host_q_start[b + 1]
            end = ctx.host_start_pos[b] + (r1 - r0)
            used = group.block_table[b, :(end + page - 1) // page].long()
            seen = store[used].reshape(-1, r)[:end].float()            # the request's latents, in order
            scores = q[r0:r1].float() @ seen.t() / math.sqrt(r)
            late = torch.arange(end, device=h.device)[None, :] > pos[r0:r1, None]
            mixed[r0:r1] = torch.softmax(scores.masked_fill(late, float("-inf")), dim=-1) @ seen
        self.ops.linear_residual(mixed.to(self.dtype), self.w_up, residual)


@dataclasses.dataclass(frozen=True)
class Toy3Config:
    vocab_size: int
    hidden_size: int
    latent_size: int
    max_positions: int
    eps: float
    architecture: str = "Toy3ForCausalLM"

    @classmethod
    def from_dict(cls, raw, where="config.json"):
        return cls(*(raw[k] for k in ("vocab_size", "hidden_size", "latent_size", "max_positions", "eps")))

    def to_dict(self):
        return {"architectures": [self.architecture], **dataclasses.asdict(self)}


def toy3_spec(cfg):
    h = cfg.hidden_size
    norm = lambda n: PartSpec("rmsnorm", dict(size=h, eps=cfg.eps), dict(weight=n))
    def block(p):
        return BlockSpec(
            "prenorm", dict(
                mixer=PartSpec("toy_latent_mixer", dict(hidden_size=h, latent_size=cfg.latent_size),
                               dict(down=p + "down", query=p + "query", up=p + "up")),
                feed_forward=PartSpec("swiglu", dict(hidden_size=h, intermediate_size=2 * h),
                                      dict(gate_weight=p + "gate", up_weight=p + "ffn_up", down_weight=p + "ffn_down")),
                norm1=norm(p + "n1"), norm2=norm(p + "n2")), params=dict(hidden_size=h))
    sizes = dict(vocab_size=cfg.vocab_size, hidden_size=h)
    return ModelSpec("Toy3ForCausalLM", cfg.vocab_size, h, cfg.max_positions,
                     PartSpec("toy_positional_embedding", dict(max_positions=cfg.max_positions, **sizes),
                              dict(weight="embed", places="places")),
                     (block("a."), block("b.")), (ScheduleEntry(0), ScheduleEntry(1)),
                     norm("final"), PartSpec("linear_head", sizes, dict(weight="head")))


def toy3_plain(ids, w, cfg):
    t, r = len(ids), cfg.latent_size
    x = w["embed"][torch.tensor(ids)] + w["places"][:t]
    late = torch.arange(t)[None, :] > torch.arange(t)[:, None]
    for p in ("a.", "b."):
        n = P.rms_norm(x, w[p + "n1"], cfg.eps)
        c, q = P.linear(n, w[p + "down"]), P.linear(n, w[p + "query"])
        probs = torch.softmax((q @ c.t() / math.sqrt(r)).masked_fill(late, float("-inf")), dim=-1)
        x = x + P.linear(probs @ c, w[p + "up"])
        x = x + P.swiglu_mlp(P.rms_norm(x, w[p + "n2"], cfg.eps), w[p + "gate"], w[p + "ffn_up"], w[p + "ffn_down"])
    return P.linear(P.rms_norm(x, w["final"], cfg.eps), w["head"])


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_toy_embedding_with_positions_and_mixer_with_a_cache_of_its_own_shape(dtype):
    """An embedding that adds a learned vector per absolute position, and a mixer whose
    per-token cache is one latent vector (a page tensor [P, r] by the name it chose, in a
    group and with a block table of its own): registered, built and stepped in every cut,
    with pages used again, without a change to the framework's files."""
    register_part("embedding", "toy_positional_embedding", PositionalEmbedding, replace=True)
    register_part("mixer", "toy_latent_mixer", LatentMixer, replace=True)
    register_architecture("Toy3ForCausalLM", Toy3Config, toy3_spec, replace=True)
    try:
        cfg = Toy3Config(vocab_size=83, hidden_size=64, latent_size=24, max_positions=256, eps=1e-5)
        from llm_inference_lab_amd.engine.model import CausalLM
        from llm_inference_lab_amd.weights import random_tensors
        tensors = dict(random_tensors(CausalLM(toy3_spec(cfg)).tensor_specs(), 7, torch.bfloat16))
        for n in tensors:
            if n in ("embed", "places") or n.endswith(("down", "query")) and "ffn" not in n:
                tensors[n] = (tensors[n].float() * 8).to(torch.bfloat16)
        engine = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype=dtype, page_size=16, num_pages=14,
                              max_requests=3, max_batch_tokens=128, max_seq_len=256)
        groups, _ = engine.model.cache_layout()
        assert len(groups) == 1 and groups[0].entries == [0, 1]
        assert tuple(engine.cache.storage[0]["latent"].shape) == (2, 14, 16, 24)
        assert engine.model.entries[1].cache["latent"].shape[0] == 14 and engine.model.entries[1].k_cache is None
        g = torch.Generator().manual_seed(4)
        seqs = {f"r{i}": torch.randint(0, 83, (n,), generator=g).tolist() for i, n in enumerate([45, 80, 23, 60])}
        w64 = {k: v.double() for k, v in tensors.items()}
        want = {rid: toy3_plain(ids, w64, cfg) for rid, ids in seqs.items()}
        for steps in (H.steps_whole(seqs), H.steps_prefill_then_decode(seqs), H.steps_portions(seqs),
                      H.steps_mixed(seqs, seed=2, max_live=3)):
            got = H.run_trace(engine, seqs, steps)
            bad = H.first_wrong(got, want, H.TOL[dtype])
            assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
        engine.cache.check()
        m = engine.cache.metrics()
        assert m["rows_used"] == 0 and m["groups"][0]["pages_used"] == 0 and m["groups"][0]["pages_high_water"] >= 10
    finally:
        unregister_part("embedding", "toy_positional_embedding")
        unregister_part("mixer", "toy_latent_mixer")
        unregister_architecture("Toy3ForCausalLM")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_toy_block_of_another_arrangement_in_random_weights_mode(dtype, tmp_path):
    """A block kind with one norm and two parallel sublayers and a norm kind whose tensors
    are not called norm (tests/toy_parallel.py): registered, written by the random-weights
    mode, loaded and stepped without a change to the framework's files."""
    import toy_parallel
    toy_parallel.run(dtype, str(tmp_path / "toy4"))
