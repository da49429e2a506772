"""Each HIP kernel alone against its plain PyTorch reference (tests/emu_ops.py),
at sizes other than the engine's: widths and vocabularies that are no power of
two, partial tiles, every head size in steps of 16, odd group counts."""
import math

import pytest
import torch

from emu_ops import EmuOps
from llm_inference_lab_amd.cache import layout as cache_layout

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from llm_inference_lab_amd.kernels.hip_ops import HipOps
    return HipOps(DEV)


@pytest.fixture(scope="module")
def emu():
    return EmuOps("cpu")


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def close(got, want, dtype, what, scale=1.0):
    got, want = got.float().cpu(), want.float().cpu()
    # float32: rounding of sums in another order; bfloat16: one rounding of the result
    tol = 2e-5 if dtype == torch.float32 else 1.0 / 128
    bound = tol * max(1.0, scale)
    err = (got - want).abs().max().item()
    assert err <= bound, f"{what}: max abs error {err} > {bound}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,hidden,vocab", [(1, 64, 256), (37, 896, 1000), (5, 100, 33), (9, 104, 77)])
def test_embed(ops, emu, dtype, rows, hidden, vocab):
    table = rnd((vocab, hidden), dtype, 1)
    ids = torch.randint(0, vocab, (rows,), generator=torch.Generator().manual_seed(2)).int()
    ids[0] = vocab - 1
    want = torch.empty(rows, hidden)
    emu.embed(table, ids, want)
    got = torch.empty(rows, hidden, device=DEV)
    ops.embed(table.to(DEV), ids.to(DEV), got)
    assert torch.equal(got.cpu(), want)
    if dtype == torch.bfloat16 and hidden % 8 == 0:       # the same rows out of the packed order
        got.zero_()
        ops.embed(ops.prepare_weight(table.to(DEV)), ids.to(DEV), got)
        assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,hidden,eps", [(1, 64, 1e-6), (19, 896, 1e-5), (7, 3584, 1e-6), (3, 100, 1e-3),
                                           (4, 1130, 1e-6), (3, 5120, 1e-6), (2, 8192, 1e-5)])
def test_rmsnorm(ops, emu, dtype, wdtype, rows, hidden, eps):
    x = rnd((rows, hidden), torch.float32, 3, 3.0)
    w = (1 + 0.1 * torch.randn(hidden, generator=torch.Generator().manual_seed(4))).to(wdtype)
    want = torch.empty(rows, hidden, dtype=dtype)
    emu.rmsnorm(x, w, eps, want)
    got = torch.empty(rows, hidden, dtype=dtype, device=DEV)
    ops.rmsnorm(x.to(DEV), w.to(DEV), eps, got)
    close(got, want, dtype, "rmsnorm", 4.0)
    # gathered rows
    if rows > 2:
        idx = torch.tensor([rows - 1, 0, rows - 2], dtype=torch.int32)
        want = torch.empty(3, hidden, dtype=dtype)
        emu.rmsnorm(x, w, eps, want, idx)
        got = torch.empty(3, hidden, dtype=dtype, device=DEV)
        ops.rmsnorm(x.to(DEV), w.to(DEV), eps, got, idx.to(DEV))
        close(got, want, dtype, "rmsnorm gather", 4.0)
    # sums left in pieces: folded into the stream and normed in one pass
    from llm_inference_lab_amd.parts.base import PendingSums
    pieces = rnd((4, rows, hidden), torch.float32, 9, 2.0)
    whole = x + pieces[:3].sum(0)
    want = torch.empty(rows, hidden, dtype=dtype)
    emu.rmsnorm(whole, w, eps, want)
    xs, got = x.to(DEV), torch.empty(rows, hidden, dtype=dtype, device=DEV)
    ops.rmsnorm(xs, w.to(DEV), eps, got, pending=PendingSums(pieces.to(DEV), 3))
    close(got, want, dtype, "rmsnorm with pieces", 4.0)
    assert torch.allclose(xs.cpu(), whole, rtol=1e-6, atol=1e-6)


LINEAR_SHAPES = [
    (1, 96, 64), (5, 90, 96), (16, 1152, 896), (17, 65, 104), (33, 200, 64), (64, 896, 4864),
    (65, 130, 72), (128, 896, 896), (200, 1152, 896), (300, 257, 136), (513, 384, 264),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", LINEAR_SHAPES)
def test_linear_bias(ops, emu, dtype, m, n, k):
    x, w = rnd((m, k), dtype, 5), rnd((n, k), dtype, 6, 0.1)
    for bias in (None, rnd((n,), torch.float32, 7), rnd((n,), torch.bfloat16, 8)):
        if dtype == torch.float32 and bias is not None and bias.dtype == torch.bfloat16:
            continue
        want = torch.empty(m, n, dtype=dtype)
        emu.linear(x, w, want, bias)
        got = torch.empty(m, n, dtype=dtype, device=DEV)
        ops.linear(x.to(DEV), ops.prepare_weight(w.to(DEV)), got, None if bias is None else bias.to(DEV))
        close(got, want, dtype, f"linear {m}x{n}x{k}", want.float().abs().max().item())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", LINEAR_SHAPES)
def test_linear_residual_and_logits(ops, emu, dtype, m, n, k):
    x, w = rnd((m, k), dtype, 9), rnd((n, k), dtype, 10, 0.1)
    resid = rnd((m, n), torch.float32, 11)
    want = resid.clone()
    emu.linear_residual(x, w, want)
    got = resid.clone().to(DEV)
    ops.linear_residual(x.to(DEV), ops.prepare_weight(w.to(DEV)), got)
    close(got, want, torch.float32, f"linear_residual {m}x{n}x{k}", want.abs().max().item())
    want = torch.empty(m, n)
    emu.linear_logits(x, w, want)
    got = torch.empty(m, n, device=DEV)
    ops.linear_logits(x.to(DEV), ops.prepare_weight(w.to(DEV)), got)
    close(got, want, torch.float32, f"linear_logits {m}x{n}x{k}", want.abs().max().item())


@pytest.mark.parametrize("fma", [False, True])
@pytest.mark.parametrize("m,n,k", [(65, 130, 72), (200, 1152, 896), (300, 257, 137), (513, 384, 264), (129, 64, 1161),
                                   (2048, 2304, 200), (1100, 4864, 96), (70, 33, 19)])
def test_float32_products_of_many_rows(ops, emu, fma, m, n, k):
    """The float32 products of more than 64 rows, on the matrix cores (both tiles: the large
    one where its blocks fill the chip) and by the plain FMA kernel that stays beside them:
    store with bias, add into the stream, SwiGLU pairs; inner sizes that are no multiple of
    4 or of the step, edges inside a tile.  Both are true 32-bit products: the same bound."""
    from llm_inference_lab_amd.parts.feed_forward import interleave_gate_up
    x, w, bias = rnd((m, k), torch.float32, 5), rnd((n, k), torch.float32, 6, 0.1), rnd((n,), torch.float32, 7)
    resid = rnd((m, n), torch.float32, 11)
    with ops.debug.force(f32_fma=fma):
        want = torch.empty(m, n)
        emu.linear(x, w, want, bias)
        got = torch.empty(m, n, device=DEV)
        ops.linear(x.to(DEV), w.to(DEV), got, bias.to(DEV))
        close(got, want, torch.float32, f"linear {m}x{n}x{k}", want.abs().max().item())
        want = resid.clone()
        emu.linear_residual(x, w, want)
        got = resid.clone().to(DEV)
        ops.linear_residual(x.to(DEV), w.to(DEV), got)
        close(got, want, torch.float32, f"linear_residual {m}x{n}x{k}", want.abs().max().item())
        inter = max(1, n // 3)
        gate, up = rnd((inter, k), torch.float32, 13, 0.2), rnd((inter, k), torch.float32, 14, 0.2)
        wgu = interleave_gate_up(gate, up)
        want = torch.empty(m, inter)
        emu.linear_swiglu(x, wgu, want)
        got = torch.empty(m, inter, device=DEV)
        ops.linear_swiglu(x.to(DEV), wgu.to(DEV), got)
        close(got, want, torch.float32, f"linear_swiglu {m}x{inter}x{k}", want.abs().max().item())


@pytest.mark.parametrize("tile", [64, 130, 129, 131, 132, 133])
@pytest.mark.parametrize("m,n,k", [(65, 130, 72), (200, 1152, 896), (300, 257, 136), (513, 384, 264), (129, 64, 1160),
                                   (70, 300, 24), (130, 90, 40), (257, 520, 8)])
def test_every_tile_shape_of_the_tiled_products(ops, emu, tile, m, n, k):
    """Every epilogue with each of the six tile shapes forced, on sizes with ragged edges
    in all three dimensions (the chooser would pick only one of them per size)."""
    from llm_inference_lab_amd.parts.feed_forward import interleave_gate_up
    bf = torch.bfloat16
    with ops.debug.force(gemm_tile=tile, few_rows_max=64):        # (small matrices: the few-row kernels would take them)
        x, w, bias = rnd((m, k), bf, 5), rnd((n, k), bf, 6, 0.1), rnd((n,), torch.float32, 7)
        pw = ops.prepare_weight(w.to(DEV))
        want = torch.empty(m, n, dtype=bf)
        emu.linear(x, w, want, bias)
        got = torch.empty(m, n, dtype=bf, device=DEV)
        ops.linear(x.to(DEV), pw, got, bias.to(DEV))
        close(got, want, bf, "store", want.float().abs().max().item())
        resid = rnd((m, n), torch.float32, 11)
        want = resid.clone()
        emu.linear_residual(x, w, want)
        got = resid.clone().to(DEV)
        ops.linear_residual(x.to(DEV), pw, got)
        close(got, want, torch.float32, "residual", want.abs().max().item())
        want = torch.empty(m, n)
        emu.linear_logits(x, w, want)
        got = torch.empty(m, n, device=DEV)
        ops.linear_logits(x.to(DEV), pw, got)
        close(got, want, torch.float32, "logits", want.abs().max().item())
        inter = n // 2 + 3
        gu = interleave_gate_up(rnd((inter, k), bf, 12, 0.1), rnd((inter, k), bf, 13, 0.1))
        want = torch.empty(m, inter, dtype=bf)
        emu.linear_swiglu(x, gu, want)
        got = torch.empty(m, inter, dtype=bf, device=DEV)
        ops.linear_swiglu(x.to(DEV), ops.prepare_weight(gu.to(DEV)), got)
        close(got, want, bf, "swiglu", want.float().abs().max().item())
        parts = torch.zeros(3, m, n, device=DEV)
        ops.linear_partials(x.to(DEV), pw, parts, 3)
        whole = x.float() @ w.float().t()
        close(parts.sum(0), whole, torch.float32, "pieces", whole.abs().max().item())


def test_linear_reference_vectors(ops):
    """The closed-form vectors of the reference's own linear tests
    (rust/engine/src/runner/model/qwen2/engine.rs:3574-3612): x = ((i*17 % 31) - 15)/32,
    W = ((i*7 + part*11) % 29)/64 - 14/64, b = (i + part*7)/128, with partial tiles."""
    for m, k, n in [(1, 96, 90), (5, 96, 90), (3, 96, 65)]:
        i = torch.arange(m * k)
        x = (((i * 17) % 31) - 15).float().view(m, k) / 32
        j = torch.arange(n * k)
        w = (((j * 7 + 11) % 29).float() / 64 - 14 / 64).view(n, k)
        b = (torch.arange(n).float() + 7) / 128
        want = x.double() @ w.double().t() + b.double()
        got = torch.empty(m, n, device=DEV)
        ops.linear(x.to(DEV), ops.prepare_weight(w.to(DEV)), got, b.to(DEV))
        assert (got.cpu().double() - want).abs().max().item() < 1e-4
        # all these values are exact in bfloat16, so that path must agree after one rounding
        gotb = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
        ops.linear(x.bfloat16().to(DEV), ops.prepare_weight(w.bfloat16().to(DEV)), gotb, b.to(DEV))
        assert torch.equal(gotb.cpu(), want.float().bfloat16())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,inter,k", [(1, 128, 64), (7, 320, 96), (16, 4864, 896), (40, 100, 72),
                                       (64, 320, 96), (70, 136, 64), (260, 4864, 896), (150, 50, 40)])
def test_linear_swiglu(ops, emu, dtype, m, inter, k):
    from llm_inference_lab_amd.parts.feed_forward import interleave_gate_up
    x = rnd((m, k), dtype, 12)
    gate, up = rnd((inter, k), dtype, 13, 0.2), rnd((inter, k), dtype, 14, 0.2)
    w = interleave_gate_up(gate, up)
    want = torch.empty(m, inter, dtype=dtype)
    emu.linear_swiglu(x, w, want)
    # the interleaving itself, against the separate matrices
    g = x.float() @ gate.float().t()
    direct = g / (1 + torch.exp(-g)) * (x.float() @ up.float().t())
    assert (want.float() - direct).abs().max() < 1e-2 * max(1.0, direct.abs().max().item())
    got = torch.empty(m, inter, dtype=dtype, device=DEV)
    ops.linear_swiglu(x.to(DEV), ops.prepare_weight(w.to(DEV)), got)
    close(got, want, dtype, f"linear_swiglu {m}x{inter}x{k}", want.float().abs().max().item())


@pytest.mark.parametrize("m", [1, 3, 8, 16, 17, 32, 40, 64])
@pytest.mark.parametrize("n,k", [(896, 896), (90, 96), (1000, 4864), (151936, 896), (65, 104), (3584, 18944)])
def test_few_row_products(ops, emu, m, n, k):
    """bfloat16 products of at most 64 rows take the block kernel with the K split
    inside the block; every epilogue against the plain reference."""
    if n * k > 40e6 and m not in (1, 8, 64):
        pytest.skip("large case: three row counts are enough")
    dtype = torch.bfloat16
    x, w = rnd((m, k), dtype, 40), rnd((n, k), dtype, 41, 0.05)
    bias = rnd((n,), torch.float32, 42)
    want = torch.empty(m, n, dtype=dtype)
    emu.linear(x, w, want, bias)
    got = torch.empty(m, n, dtype=dtype, device=DEV)
    ops.linear(x.to(DEV), ops.prepare_weight(w.to(DEV)), got, bias.to(DEV))
    close(got, want, dtype, "few-row linear", want.float().abs().max().item())
    resid = rnd((m, n), torch.float32, 43)
    want = resid.clone()
    emu.linear_residual(x, w, want)
    got = resid.clone().to(DEV)
    ops.linear_residual(x.to(DEV), ops.prepare_weight(w.to(DEV)), got)
    close(got, want, torch.float32, "few-row residual", want.abs().max().item() * 4)


@pytest.mark.parametrize("m", [65, 100, 333, 1024])
@pytest.mark.parametrize("n,k,inter,vocab", [(896, 896, 320, 515), (90, 96, 128, 256), (65, 104, 72, 301)])
def test_few_row_kernels_beyond_64_rows(ops, emu, m, n, k, inter, vocab):
    """Small matrices keep the few-row kernels beyond 64 rows, in tiles of 16 rows that
    separate blocks take (up to 1,024 rows; the rule that stops earlier for larger
    matrices is taken away here): every epilogue, with and without the fused norm, rows
    gathered for the logits among them."""
    from llm_inference_lab_amd.parts.feed_forward import interleave_gate_up
    bf = torch.bfloat16
    with ops.debug.force(few_rows_read_bytes=1e15, few_rows_max=1024):
        assert ops.few_rows_take(m, n, k) and ops.can_fuse(m, bf, k, max(n, 2 * inter, vocab))
        x, w, bias = rnd((m, k), bf, 40), rnd((n, k), bf, 41, 0.05), rnd((n,), torch.float32, 42)
        gu = interleave_gate_up(rnd((inter, k), bf, 52, 0.1), rnd((inter, k), bf, 53, 0.1))
        head = rnd((vocab, k), bf, 54, 0.1)
        pw, pgu, phead = (ops.prepare_weight(t.to(DEV)) for t in (w, gu, head))
        calls = ops.calls_made
        want = torch.empty(m, n, dtype=bf)
        emu.linear(x, w, want, bias)
        got = torch.empty(m, n, dtype=bf, device=DEV)
        ops.linear(x.to(DEV), pw, got, bias.to(DEV))
        close(got, want, bf, "linear", want.float().abs().max().item())
        resid = rnd((m, n), torch.float32, 43)
        want = resid.clone()
        emu.linear_residual(x, w, want)
        got = resid.clone().to(DEV)
        ops.linear_residual(x.to(DEV), pw, got)
        close(got, want, torch.float32, "residual", want.abs().max().item() * 4)
        xs = rnd((m + 5, k), torch.float32, 50, 3.0)
        nw = (1 + 0.1 * rnd((k,), torch.float32, 51)).to(bf)
        want = torch.empty(m, inter, dtype=bf)
        emu.fused_norm_swiglu(xs[:m], nw, 1e-5, gu, want)
        got = torch.empty(m, inter, dtype=bf, device=DEV)
        ops.fused_norm_swiglu(xs[:m].contiguous().to(DEV), nw.to(DEV), 1e-5, pgu, got)
        close(got, want, bf, "fused norm + swiglu", want.float().abs().max().item())
        idx = torch.randperm(m + 5, generator=torch.Generator().manual_seed(55))[:m].int()
        want = torch.empty(m, vocab)
        emu.fused_norm_logits(xs, idx, nw, 1e-5, head, want)
        got = torch.empty(m, vocab, device=DEV)
        ops.fused_norm_logits(xs.to(DEV), idx.to(DEV), nw.to(DEV), 1e-5, phead, got)
        close(got, want, torch.float32, "fused norm + logits", want.abs().max().item() * 40)
        assert ops.calls_made - calls == 4          # one kernel each
    with pytest.raises(ValueError):
        ops.fused_norm_swiglu(torch.zeros(1025, k, device=DEV), nw.to(DEV), 1e-5, pgu,
                              torch.empty(1025, inter, dtype=bf, device=DEV))


@pytest.mark.parametrize("mb", [1, 2, 4])
@pytest.mark.parametrize("stage", [0, 1])
@pytest.mark.parametrize("nsb,kw", [(1, 1), (1, 4), (1, 16), (2, 2), (2, 8), (4, 1), (4, 4), (8, 2), (16, 1)])
def test_few_row_products_in_every_block_shape(ops, emu, nsb, kw, stage, mb):
    """The block shape (strips per block, K slices per strip, staged rows or not, rows
    per tile) is chosen by a cost estimate, so most shapes never run at a given size:
    each is forced here.  A shape that does not fit says so and computes nothing."""
    from llm_inference_lab_amd.kernels.hip_ops import KernelError
    from llm_inference_lab_amd.parts.feed_forward import interleave_gate_up
    dtype = torch.bfloat16
    ran = 0
    for m, n, k in ((5, 130, 264), (40, 896, 1160), (64, 320, 96)):
        x, w = rnd((m, k), dtype, 44), rnd((n, k), dtype, 45, 0.1)
        bias, resid = rnd((n,), torch.float32, 46), rnd((m, n), torch.float32, 47)
        gate_up = interleave_gate_up(w, rnd((n, k), dtype, 48, 0.1))
        want = torch.empty(m, n, dtype=dtype)
        emu.linear(x, w, want, bias)
        want_resid = resid.clone()
        emu.linear_residual(x, w, want_resid)
        want_act = torch.empty(m, n, dtype=dtype)
        emu.linear_swiglu(x, gate_up, want_act)
        xd, wd, gd = x.to(DEV), ops.prepare_weight(w.to(DEV)), ops.prepare_weight(gate_up.to(DEV))
        def forced(fn):
            """Runs fn under the forced shape; False if the kernel refused the shape."""
            try:
                with ops.debug.force(skinny_shape=(nsb, kw, stage, mb)):
                    fn()
                return True
            except KernelError as err:
                assert "does not fit" in str(err) or "no block shape" in str(err), err
                return False

        got = torch.full((m, n), float("nan"), dtype=dtype, device=DEV)
        if forced(lambda: ops.linear(xd, wd, got, bias.to(DEV))):
            ran += 1
            close(got, want, dtype, f"forced {nsb}x{kw} linear", want.float().abs().max().item())
        got_resid = resid.clone().to(DEV)
        if forced(lambda: ops.linear_residual(xd, wd, got_resid)):
            ran += 1
            close(got_resid, want_resid, torch.float32, f"forced {nsb}x{kw} residual", want_resid.abs().max().item() * 4)
        got_act = torch.full((m, n), float("nan"), dtype=dtype, device=DEV)
        if forced(lambda: ops.linear_swiglu(xd, gd, got_act)):
            ran += 1
            close(got_act, want_act, dtype, f"forced {nsb}x{kw} swiglu", want_act.float().abs().max().item())
    assert ran > 0 or nsb * kw > 8, "no size ran this shape"


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 8, 17, 33, 64])
@pytest.mark.parametrize("hidden,inter,vocab", [(64, 128, 256), (96, 320, 515), (896, 4864, 3001), (72, 200, 301)])
def test_fused_norm_products(ops, emu, wdtype, m, hidden, inter, vocab):
    from llm_inference_lab_amd.parts.feed_forward import interleave_gate_up
    bf = torch.bfloat16
    x = rnd((m + 5, hidden), torch.float32, 50, 3.0)
    nw = (1 + 0.1 * rnd((hidden,), torch.float32, 51)).to(wdtype)
    eps = 1e-5
    # SwiGLU
    w = interleave_gate_up(rnd((inter, hidden), bf, 52, 0.1), rnd((inter, hidden), bf, 53, 0.1))
    want = torch.empty(m, inter, dtype=bf)
    emu.fused_norm_swiglu(x[:m], nw, eps, w, want)
    got = torch.empty(m, inter, dtype=bf, device=DEV)
    ops.fused_norm_swiglu(x[:m].contiguous().to(DEV), nw.to(DEV), eps, ops.prepare_weight(w.to(DEV)), got)
    close(got, want, bf, "fused norm + swiglu", want.float().abs().max().item())
    # logits of gathered rows
    head = rnd((vocab, hidden), bf, 54, 0.1)
    idx = torch.randperm(m + 5, generator=torch.Generator().manual_seed(55))[:m].int()
    want = torch.empty(m, vocab)
    emu.fused_norm_logits(x, idx, nw, eps, head, want)
    got = torch.empty(m, vocab, device=DEV)
    ops.fused_norm_logits(x.to(DEV), idx.to(DEV), nw.to(DEV), eps, ops.prepare_weight(head.to(DEV)), got)
    close(got, want, torch.float32, "fused norm + logits", want.abs().max().item() * 40)


@pytest.mark.parametrize("nq,nkv,d,page,hidden", [(4, 2, 16, 16, 64), (3, 1, 32, 32, 96), (14, 2, 64, 64, 896),
                                                 (6, 3, 48, 16, 72), (8, 8, 128, 64, 256), (2, 1, 256, 16, 64)])
@pytest.mark.parametrize("rotate,rows_per", [(True, [5, 1, 9]), (False, [5, 1, 9]), (True, [17, 30, 16]),
                                             (True, [70, 1, 130]), (True, [300, 90, 2])])
def test_fused_norm_qkv_rope_write(ops, emu, nq, nkv, d, page, hidden, rotate, rows_per):
    bf = torch.bfloat16
    starts, reqs = [3, 40, 0], 3
    needs = [(s0 + c + page - 1) // page for s0, c in zip(starts, rows_per)]
    num_pages = 16 + sum(needs)
    rows = sum(rows_per)
    x = rnd((rows, hidden), torch.float32, 60, 2.0)
    nw = (1 + 0.1 * rnd((hidden,), torch.float32, 61)).to(bf)
    n = (nq + 2 * nkv) * d
    w, b = rnd((n, hidden), bf, 62, 0.2), rnd((n,), bf, 63)
    positions = torch.cat([torch.arange(s, s + c) for s, c in zip(starts, rows_per)]).int()
    row_req = torch.cat([torch.full((c,), i) for i, c in enumerate(rows_per)]).int()
    table = torch.full((reqs, max(8, max(needs))), -1, dtype=torch.int32)
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(64)).int()
    at = 0
    for i in range(reqs):
        need = (starts[i] + rows_per[i] + page - 1) // page
        table[i, :need] = perm[at:at + need]
        at += need
    inv_freq = (1.0 / (1e4 ** (torch.arange(0, d, 2, dtype=torch.float64) / d))).float() if rotate else None
    kc, vc = make_cache(num_pages, nkv, page, d, bf, 65)
    want_q, want_k, want_v = torch.empty(rows, nq * d, dtype=bf), kc.clone(), vc.clone()
    emu.fused_norm_qkv(x, nw, 1e-6, w, b, nq, nkv, d, inv_freq, positions, row_req, table, page,
                       want_k, want_v, want_q)
    got_q, got_k, got_v = torch.empty(rows, nq * d, dtype=bf, device=DEV), kc.to(DEV), vc.to(DEV)
    ops.fused_norm_qkv(x.to(DEV), nw.to(DEV), 1e-6, ops.prepare_weight(w.to(DEV)), b.to(DEV), nq, nkv, d,
                       None if inv_freq is None else inv_freq.to(DEV), positions.to(DEV), row_req.to(DEV),
                       table.to(DEV), page, got_k, got_v, got_q)
    scale = want_q.float().abs().max().item()
    close(got_q, want_q, bf, "fused q", scale)
    close(got_k, want_k, bf, "fused key cache", scale)
    close(got_v, want_v, bf, "fused value cache", scale)
    untouched = (want_k == kc)
    assert torch.equal(got_k.cpu()[untouched], kc[untouched])


@pytest.mark.parametrize("nq,nkv,d,page,hidden", [(4, 2, 16, 16, 64), (14, 2, 64, 64, 896), (6, 3, 48, 16, 72),
                                                 (8, 8, 128, 64, 256), (2, 1, 256, 16, 64)])
@pytest.mark.parametrize("rows_per,few_rows_max", [([5, 1, 9], 64), ([20, 1, 1, 3], 64), ([17, 30, 16], 64),
                                                   ([70, 1, 130], 64), ([300, 2, 2, 90], 64),
                                                   ([70, 1, 130], 1024), ([300, 2, 2, 90], 1024), ([1000, 24], 1024)])
def test_qkv_rope_cache_of_normed_rows(ops, emu, nq, nkv, d, page, hidden, rows_per, few_rows_max):
    """Up to 64 rows the few-row kernel; more rows the tiled kernel with rotation and cache
    write in its epilogue, or (matrices as small as these, unless the rule is switched off)
    the few-row kernel again in tiles of 16 rows."""
    # (heads of 128: the large tile, which this few rows would not get)
    with ops.debug.force(gemm_tile=128 if d == 128 and sum(rows_per) > 64 else 0, few_rows_max=few_rows_max):
        check_qkv_rope_cache(ops, emu, nq, nkv, d, page, hidden, rows_per)


@pytest.mark.parametrize("nq,nkv,d,page,hidden", [(4, 2, 16, 16, 64), (14, 2, 64, 64, 896), (7, 1, 32, 16, 72),
                                                 (8, 8, 128, 64, 256), (2, 1, 256, 16, 64)])
@pytest.mark.parametrize("rows_per", [[70, 1, 130], [300, 2, 2, 90]])
@pytest.mark.parametrize("tile", [131, 132, 133])
def test_qkv_rope_cache_with_the_widest_tiles(ops, emu, nq, nkv, d, page, hidden, rows_per, tile):
    """The tiles of 256 columns and eight waves, which only large products get by
    themselves: heads of every size that divides them, a head of 256 among them."""
    with ops.debug.force(gemm_tile=tile, few_rows_max=64):
        assert ops.can_fuse_qkv_rope(sum(rows_per), torch.bfloat16, d, (nq + 2 * nkv) * d, hidden)
        check_qkv_rope_cache(ops, emu, nq, nkv, d, page, hidden, rows_per)


@pytest.mark.parametrize("nq,nkv,d,page,hidden", [(4, 2, 16, 16, 64), (14, 2, 64, 64, 896), (6, 3, 48, 16, 72),
                                                 (8, 8, 128, 64, 256), (2, 1, 256, 16, 64)])
@pytest.mark.parametrize("rows_per", [[20, 1, 1, 3], [17, 30, 16], [5, 8, 11]])
@pytest.mark.parametrize("pieces", [2, 5])
def test_qkv_rope_cache_through_pieces(ops, emu, nq, nkv, d, page, hidden, rows_per, pieces):
    """17 to 64 rows of a large matrix: the product is cut along its inner size and a second
    kernel sums the pieces, adds the bias, rotates and writes the cache.  The small
    matrices of the test take that way with the size limit taken away."""
    with ops.debug.force(tiled_pieces_bytes=0, forced_tiled_pieces=pieces):
        assert ops.pieces_by_tiles(sum(rows_per), (nq + 2 * nkv) * d, hidden)
        assert sum(rows_per) >= ops.rules.qkv_pieces_min_rows
        check_qkv_rope_cache(ops, emu, nq, nkv, d, page, hidden, rows_per)
    assert ops.rules.forced_tiled_pieces == 0 and ops.rules.tiled_pieces_bytes == 16e6


def check_qkv_rope_cache(ops, emu, nq, nkv, d, page, hidden, rows_per, starts=(3, 40, 0, 7)):
    bf = torch.bfloat16
    rows, reqs = sum(rows_per), len(rows_per)
    num_pages = 16 + sum((max(starts) + c + page - 1) // page for c in rows_per)
    if not ops.can_fuse_qkv_rope(rows, bf, d, (nq + 2 * nkv) * d, hidden):
        with pytest.raises(ValueError):
            ops.qkv_rope_cache(torch.zeros(rows, hidden, dtype=bf, device=DEV),
                               ops.prepare_weight(torch.zeros((nq + 2 * nkv) * d, hidden, dtype=bf, device=DEV)),
                               None, nq, nkv, d, None, torch.zeros(rows, dtype=torch.int32, device=DEV), None,
                               None, page, None, None, torch.empty(rows, nq * d, dtype=bf, device=DEV))
        return
    starts = list(starts)[:reqs]
    h = rnd((rows, hidden), bf, 70)
    n = (nq + 2 * nkv) * d
    w, b = rnd((n, hidden), bf, 72, 0.2), rnd((n,), bf, 73)
    positions = torch.cat([torch.arange(s, s + c) for s, c in zip(starts, rows_per)]).int()
    row_req = torch.cat([torch.full((c,), i) for i, c in enumerate(rows_per)]).int()
    table = torch.full((reqs, max((s0 + c + page - 1) // page for s0, c in zip(starts, rows_per))), -1,
                       dtype=torch.int32)
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(74)).int()
    at = 0
    for i in range(reqs):
        need = (starts[i] + rows_per[i] + page - 1) // page
        table[i, :need] = perm[at:at + need]
        at += need
    assert at <= num_pages
    inv_freq = (1.0 / (1e4 ** (torch.arange(0, d, 2, dtype=torch.float64) / d))).float()
    kc, vc = make_cache(num_pages, nkv, page, d, bf, 75)
    want_q, want_k, want_v = torch.empty(rows, nq * d, dtype=bf), kc.clone(), vc.clone()
    emu.qkv_rope_cache(h, w, b, nq, nkv, d, inv_freq, positions, row_req, table, page, want_k, want_v, want_q)
    got_q, got_k, got_v = torch.empty(rows, nq * d, dtype=bf, device=DEV), kc.to(DEV), vc.to(DEV)
    ops.qkv_rope_cache(h.to(DEV), ops.prepare_weight(w.to(DEV)), b.to(DEV), nq, nkv, d, inv_freq.to(DEV),
                       positions.to(DEV), row_req.to(DEV), table.to(DEV), page, got_k, got_v, got_q)
    scale = want_q.float().abs().max().item()
    close(got_q, want_q, bf, "q", scale)
    close(got_k, want_k, bf, "key cache", scale)
    close(got_v, want_v, bf, "value cache", scale)
    untouched = (want_k == kc)
    assert torch.equal(got_k.cpu()[untouched], kc[untouched])
    untouched = (want_v == vc)
    assert torch.equal(got_v.cpu()[untouched], vc[untouched])


@pytest.mark.parametrize("nq,nkv,d,page,hidden", [(4, 2, 16, 16, 64), (14, 2, 64, 64, 896), (8, 8, 128, 64, 256),
                                                 (2, 1, 256, 16, 64)])
@pytest.mark.parametrize("rows_per,starts", [([72, 4, 124], (0, 64, 8)), ([70, 6, 125], (2, 61, 9)),
                                             ([8, 4, 4, 180], (12, 0, 28, 100))])
@pytest.mark.parametrize("tile", [0, 129, 132, 133])
def test_values_of_four_positions_written_together(ops, emu, nq, nkv, d, page, hidden, rows_per, starts, tile):
    """The values of four consecutive positions of a request that start at a multiple of four go
    to their page as one piece of 32 bytes per four numbers of a head, others number by number:
    requests whose rows and positions line up so (a prompt from its start, a portion that starts
    at a multiple of four), requests that do not, and short requests between them."""
    with ops.debug.force(gemm_tile=tile, few_rows_max=64):
        check_qkv_rope_cache(ops, emu, nq, nkv, d, page, hidden, rows_per, starts)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 40])
def test_attention_of_a_mixed_step(ops, emu, window, dtype):
    """Portions of prompts beside decoding requests with long histories, one of which has a
    key that stands out far back."""
    spec = [(700, 1), (64, 300), (1500, 1), (0, 1), (31, 2), (200, 90), (999, 1)]
    run_attention(ops, emu, dtype, 14, 2, 64, 64, window, spec, seed=90, amplify=(2, 100 if window is None else 1480, 30.0))
    run_attention(ops, emu, dtype, 6, 3, 48, 16, window, spec[:5], seed=91)
    run_attention(ops, emu, dtype, 8, 1, 128, 32, window, spec[:4], seed=92)


@pytest.mark.parametrize("window", [None, 40])
@pytest.mark.parametrize("cus", [8, 16, 30, 60, 80, 100, 1000])
@pytest.mark.parametrize("nq,nkv,d,page", [(14, 2, 64, 64), (6, 3, 48, 16), (8, 1, 128, 32), (2, 1, 256, 16)])
def test_attention_tilings_of_many_rows(ops, emu, window, cus, nq, nkv, d, page, dtype=torch.bfloat16):
    """The kernel variants for many tiles of rows (tiles of 128 rows, of 64, of 64 in
    pairs, keys split over the waves of a block) are chosen by the tiles per compute
    unit: told of fewer units than the chip has, a step of a few hundred rows takes
    each of them."""
    real = ops.num_cus
    ops.num_cus = cus
    try:
        run_attention(ops, emu, dtype, nq, nkv, d, page, window, [(0, 300), (0, 200)], seed=93,
                      amplify=(0, 70, 30.0))
        # behind a history (never in pairs), and one request decoding beside
        run_attention(ops, emu, dtype, nq, nkv, d, page, window, [(500, 300), (64, 200), (900, 1)], seed=94,
                      amplify=(0, 130 if window is None else 770, 30.0))
    finally:
        ops.num_cus = real


@pytest.mark.parametrize("window", [None, 40])
@pytest.mark.parametrize("cus", [8, 1000])
@pytest.mark.parametrize("nq,nkv,d,page", [(14, 2, 64, 64), (6, 3, 48, 16), (8, 1, 128, 32), (2, 1, 256, 16)])
def test_attention_tilings_of_many_rows_float32(ops, emu, window, cus, nq, nkv, d, page):
    """The float32 kernel's two launches for many rows: a wave per tile of rows, and (told
    of a very large chip, behind a history) the waves of a block splitting a tile's keys."""
    test_attention_tilings_of_many_rows(ops, emu, window, cus, nq, nkv, d, page, dtype=torch.float32)


@pytest.mark.parametrize("window", [None, 40])
@pytest.mark.parametrize("path", [1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("nq,nkv,d,page", [(14, 2, 64, 64), (6, 3, 48, 16), (8, 1, 128, 32), (3, 1, 96, 16),
                                           (4, 2, 16, 16), (5, 5, 112, 32), (2, 1, 256, 16)])
def test_attention_every_launch_of_many_rows(ops, emu, window, path, nq, nkv, d, page):
    """Each launch for steps of many rows, fixed from outside whatever the rule would take:
    keys split over the waves of a block, tiles of 32 and of 16 rows per wave, late and
    early tiles in pairs, and the last two with two groups of waves that take the staged
    keys in turn and merge at the end (a tile of rows whose second group sees no key at all,
    a history that ends inside the first group's keys)."""
    with ops.debug.force(attention_path=(d, path)):
        run_attention(ops, emu, torch.bfloat16, nq, nkv, d, page, window, [(0, 300), (0, 70), (0, 129)], seed=96,
                      amplify=(0, 70, 30.0))
        run_attention(ops, emu, torch.bfloat16, nq, nkv, d, page, window, [(500, 300), (64, 200), (900, 1)], seed=97,
                      amplify=(0, 130 if window is None else 770, 30.0))
        if path <= 2:      # float32 has these two: the waves of a block split the keys, or a wave per tile
            run_attention(ops, emu, torch.float32, nq, nkv, d, page, window, [(0, 300), (0, 70), (0, 129)], seed=96,
                          amplify=(0, 70, 30.0))
            run_attention(ops, emu, torch.float32, nq, nkv, d, page, window, [(500, 300), (64, 200), (900, 1)],
                          seed=97, amplify=(0, 130 if window is None else 770, 30.0))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("start", [0, 3000])
def test_attention_of_a_long_portion(ops, emu, start, dtype):
    """2,048 tokens of a prompt at the 0.5B head counts, at its start and behind a
    history: enough tiles for the whole chip, as in a prefill step of the engine."""
    run_attention(ops, emu, dtype, 14, 2, 64, 64, None, [(start, 2048)], seed=95, amplify=(0, 1033, 30.0))


def make_cache(num_pages, nkv, page, d, dtype, seed):
    k = rnd((num_pages, nkv, page, d), dtype, seed)
    v = rnd((num_pages, nkv, d, page), dtype, seed + 1)
    return k, v


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,d,page", [(4, 2, 16, 16), (3, 1, 32, 32), (14, 2, 64, 64), (6, 3, 48, 16),
                                           (8, 8, 128, 64)])
def test_rope_kv_write(ops, emu, dtype, nq, nkv, d, page):
    rows_per, reqs, num_pages = [5, 1, 9], 3, 12
    starts = [3, 40, 0]
    rows = sum(rows_per)
    qkv = rnd((rows, (nq + 2 * nkv) * d), dtype, 20)
    positions = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, rows_per)]).int()
    row_req = torch.cat([torch.full((n,), b) for b, n in enumerate(rows_per)]).int()
    table = torch.full((reqs, 8), -1, dtype=torch.int32)
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(21)).int()
    at = 0
    for b in range(reqs):
        need = (starts[b] + rows_per[b] + page - 1) // page
        table[b, :need] = perm[at:at + need]
        at += need
    theta = 1e6
    inv_freq = (1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float64) / d))).float()
    kc, vc = make_cache(num_pages, nkv, page, d, dtype, 22)
    want_qkv, want_k, want_v = qkv.clone(), kc.clone(), vc.clone()
    emu.rope_kv_write(want_qkv, nq, nkv, d, inv_freq, positions, row_req, table, page, want_k, want_v)
    got_qkv, got_k, got_v = qkv.to(DEV), kc.to(DEV), vc.to(DEV)
    ops.rope_kv_write(got_qkv, nq, nkv, d, inv_freq.to(DEV), positions.to(DEV), row_req.to(DEV),
                      table.to(DEV), page, got_k, got_v)
    close(got_qkv[:, :nq * d], want_qkv[:, :nq * d], dtype, "rope q", 4.0)
    close(got_k, want_k, dtype, "key cache", 4.0)
    close(got_v, want_v, dtype, "value cache", 4.0)
    # untouched places of the cache stay bit-identical
    untouched = (want_k == kc)
    assert torch.equal(got_k.cpu()[untouched], kc[untouched])


def run_attention(ops, emu, dtype, nq, nkv, d, page, window, reqs_spec, seed=30, scale=None, amplify=None):
    """reqs_spec: list of (start_pos, q_len)."""
    reqs = len(reqs_spec)
    rows = sum(n for _, n in reqs_spec)
    max_ctx = max(s + n for s, n in reqs_spec)
    pages_per = (max_ctx + page - 1) // page
    num_pages = reqs * pages_per + 3
    qkv = rnd((rows, (nq + 2 * nkv) * d), dtype, seed)
    kc, vc = make_cache(num_pages, nkv, page, d, dtype, seed + 1)
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(seed + 2)).int()
    table = torch.full((reqs, pages_per), -1, dtype=torch.int32)
    q_start, start_pos = [0], []
    at = 0
    for b, (s, n) in enumerate(reqs_spec):
        need = (s + n + page - 1) // page
        table[b, :need] = perm[at:at + need]
        at += need
        q_start.append(q_start[-1] + n)
        start_pos.append(s)
    if amplify is not None:
        # one far key stands out: scale query and that key so its score dominates
        b, key_pos, factor = amplify
        pg, off = int(table[b, key_pos // page]), key_pos % page
        kc[pg, :, off, :] *= factor
    # positions past each request's end hold garbage that must not leak in
    for b, (s, n) in enumerate(reqs_spec):
        end = s + n
        if end % page:
            pg = int(table[b, end // page])
            kc[pg, :, end % page:, :] = 1e4
            vc[pg, :, :, end % page:] = -1e4
    # what was set up above by key and number goes into the order the cache keeps
    kc, vc = cache_layout.keys_to_cache_order(kc), cache_layout.values_to_cache_order(vc)
    q_start_t = torch.tensor(q_start, dtype=torch.int32)
    start_pos_t = torch.tensor(start_pos, dtype=torch.int32)
    scale = scale if scale is not None else 1 / math.sqrt(d)
    want = torch.zeros(rows, nq * d, dtype=dtype)
    emu.paged_attention(qkv, nq, nkv, d, kc, vc, table, page, q_start_t, start_pos_t, reqs,
                        max(n for _, n in reqs_spec), max_ctx, window, scale, want)
    got = torch.zeros(rows, nq * d, dtype=dtype, device=DEV)
    ops.paged_attention(qkv.to(DEV), nq, nkv, d, kc.to(DEV), vc.to(DEV), table.to(DEV), page,
                        q_start_t.to(DEV), start_pos_t.to(DEV), reqs, max(n for _, n in reqs_spec),
                        max_ctx, window, scale, got)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    err = (got.float().cpu() - want.float()).abs().max().item()
    assert err <= tol * max(1.0, want.float().abs().max().item()), f"attention error {err}"

    # the same step described as the engine describes it (which requests are short): a
    # mixed step is then served by two launches, or by one that runs both kinds of blocks
    limit = ops.attention_short_limit(nq, nkv, dtype, max(n for _, n in reqs_spec))
    short_reqs = [(s, n) for s, n in reqs_spec if n <= limit]
    short = None
    if 0 < len(short_reqs) < reqs:
        row_req = torch.cat([torch.full((n,), b) for b, (_, n) in enumerate(reqs_spec)]).int().to(DEV)
        short = (row_req, limit, len(short_reqs), max(s + n for s, n in short_reqs))
    got2 = torch.zeros(rows, nq * d, dtype=dtype, device=DEV)
    ops.paged_attention(qkv.to(DEV), nq, nkv, d, kc.to(DEV), vc.to(DEV), table.to(DEV), page,
                        q_start_t.to(DEV), start_pos_t.to(DEV), reqs, max(n for _, n in reqs_spec),
                        max_ctx, window, scale, got2, short)
    err = (got2.float().cpu() - want.float()).abs().max().item()
    assert err <= tol * max(1.0, want.float().abs().max().item()), f"attention error {err} (described step)"
    # key splits are merged by the last block to arrive; the same with the kernel of its own,
    # and the arrival counters are back at zero whoever merged
    if dtype == torch.bfloat16:
        # (and a mixed step in a launch for each kind of request where one launch would serve both)
        for who in (("attention_merge_kernel",), ("attention_merge_in_place",), ("attention_two_launches",),
                    ("attention_one_launch",), ("attention_one_launch", "attention_merge_kernel"),
                    ("attention_one_launch", "attention_merge_in_place")):
            got3 = torch.zeros(rows, nq * d, dtype=dtype, device=DEV)
            with ops.debug.force(**{w: d for w in who}):
                ops.paged_attention(qkv.to(DEV), nq, nkv, d, kc.to(DEV), vc.to(DEV), table.to(DEV), page,
                                    q_start_t.to(DEV), start_pos_t.to(DEV), reqs, max(n for _, n in reqs_spec),
                                    max_ctx, window, scale, got3, short)
            err = (got3.float().cpu() - want.float()).abs().max().item()
            assert err <= tol * max(1.0, want.float().abs().max().item()), f"attention error {err} ({who})"
    assert int(ops.arrived.abs().sum()) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d", [16, 32, 48, 64, 80, 96, 112, 128, 256])
def test_attention_head_sizes(ops, emu, dtype, d):
    run_attention(ops, emu, dtype, 4, 2, d, 16, None, [(0, 37), (21, 1), (5, 12)])
    run_attention(ops, emu, dtype, 4, 2, d, 64, None, [(100, 150), (300, 1)])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv", [(3, 1), (14, 2), (7, 7), (5, 1), (40, 8), (20, 1)])
def test_attention_groups(ops, emu, dtype, nq, nkv):
    run_attention(ops, emu, dtype, nq, nkv, 32, 32, None, [(0, 50), (63, 1), (10, 3)])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("length", [31, 32, 33, 63, 64, 65, 127, 129, 513])
def test_attention_decode_lengths(ops, emu, dtype, length):
    """One decoded token over `length` cached keys (the lengths of the reference's
    attention tests, rust/engine/src/runner/model/qwen2/engine.rs:3209-3435)."""
    run_attention(ops, emu, dtype, 14, 2, 64, 64, None, [(length - 1, 1)])
    run_attention(ops, emu, dtype, 4, 2, 64, 16, None, [(length - 1, 1), (7, 1)])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 5, 24, 64, 1000])
def test_attention_window(ops, emu, dtype, window):
    run_attention(ops, emu, dtype, 3, 1, 32, 16, window, [(0, 70), (100, 1), (33, 9)])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_far_key_among_hundreds(ops, emu, dtype):
    """A single far key carries the whole answer: a kernel that skips, repeats or
    mis-places a key block cannot hide behind averaged random values."""
    run_attention(ops, emu, dtype, 4, 2, 64, 64, None, [(900, 1)], amplify=(0, 3, 30.0))
    run_attention(ops, emu, dtype, 4, 2, 64, 16, None, [(0, 700)], amplify=(0, 130, 30.0))
    run_attention(ops, emu, dtype, 14, 2, 64, 64, None, [(4000, 1), (2000, 1)], amplify=(1, 1999, 30.0))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d,length,key", [(64, 9000, 8000), (128, 5000, 70), (64, 20001, 11), (64, 40000, 33000)])
def test_attention_one_request_over_a_long_history(ops, emu, d, length, key, dtype):
    """One decoded token of a single request: its keys are split over as many blocks
    as the merge takes (from 35 to the limit of 128 here), and one key far from both ends
    carries the answer."""
    run_attention(ops, emu, dtype, 4, 1, d, 64, None, [(length - 1, 1)], amplify=(0, key, 30.0))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("splits", [1, 3, 16, 17, 50, 64, 65, 128])
def test_attention_merge_of_any_number_of_splits(ops, emu, splits, dtype):
    """The number of key splits is fixed from outside: one wave merges up to sixteen,
    four waves more, a lane holds the weights of two; splits past the end of a short
    history have no keys at all and must count for nothing."""
    for d, length in ((64, 700), (128, 3000), (48, 90)):
        with ops.debug.force(attention_splits=(d, splits)):
            run_attention(ops, emu, dtype, 6, 2, d, 16, None, [(length - 1, 1), (40, 1), (length // 2, 2)],
                          seed=96, amplify=(0, length // 3, 30.0))


@pytest.mark.parametrize("one_pass", [True, False])
@pytest.mark.parametrize("vocab", [1, 255, 256, 257, 4095, 4097, 8193, 151936])
def test_argmax(ops, emu, vocab, one_pass):
    """Vocabulary sizes and special rows of the reference's argmax tests
    (rust/engine/src/runner/model/qwen2/engine.rs:2285-2358); in one kernel whose last block
    picks among the blocks' results (three times in a row: its counters must come back to
    zero), and in two kernels."""
    g = torch.Generator().manual_seed(vocab)
    logits = torch.randn(5, vocab, generator=g)
    logits[1, vocab - 1] = 100.0                      # maximum at the last index
    if vocab > 300:
        logits[2, 7] = logits[2, 290] = 50.0          # tie across threads: smallest index
    logits[3, :] = float("-inf")                      # all -inf: index 0
    logits[4, :] = float("nan")                       # all NaN: -1
    want = torch.zeros(5, dtype=torch.int32)
    emu.argmax(logits, want)
    on_gpu = logits.to(DEV)
    for _ in range(3):
        got = torch.full((5,), -9, dtype=torch.int32, device=DEV)
        ops.argmax(on_gpu, got, one_pass=one_pass)
        assert got.cpu().tolist() == want.tolist()
    assert int(ops.arrived.abs().sum()) == 0
    assert want[1] == vocab - 1 and want[3] == 0 and want[4] == -1
    if vocab > 300:
        assert want[2] == 7


def test_sample_temperature(ops, emu):
    vocab = 1000
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(64, vocab, generator=g) * 3
    temps = torch.full((64,), 0.8)
    temps[:4] = 0.0
    u = torch.rand(64, generator=g)
    got = torch.zeros(64, dtype=torch.int32, device=DEV)
    ops.sample(logits.to(DEV), temps.to(DEV), u.to(DEV), got)
    got = got.cpu()
    for b in range(64):
        if temps[b] == 0:
            assert got[b] == logits[b].argmax()
            continue
        p = torch.softmax(logits[b].double() / 0.8, dim=0)
        cdf = torch.cumsum(p, dim=0)
        t = int(got[b])
        lo = 0.0 if t == 0 else float(cdf[t - 1])
        assert lo - 1e-4 <= float(u[b]) <= float(cdf[t]) + 1e-4, (b, t, lo, float(u[b]), float(cdf[t]))
    # a 4-token vocabulary: the histogram of many draws follows softmax(logits / t)
    small = torch.tensor([[1.0, 0.0, -1.0, 2.0]]).repeat(4096, 1)
    u = torch.rand(4096, generator=g)
    out = torch.zeros(4096, dtype=torch.int32, device=DEV)
    ops.sample(small.to(DEV), torch.full((4096,), 0.5).to(DEV), u.to(DEV), out)
    hist = torch.bincount(out.cpu().long(), minlength=4).double() / 4096
    want = torch.softmax(small[0].double() / 0.5, dim=0)
    assert (hist - want).abs().max() < 0.03


def test_refused_sizes(ops):
    from llm_inference_lab_amd.config.errors import UnsupportedSizeError
    with pytest.raises(UnsupportedSizeError):
        ops.check_attention_sizes(4, 2, 24, torch.bfloat16)
    with pytest.raises(UnsupportedSizeError):
        ops.check_attention_sizes(4, 2, 272, torch.bfloat16)
    with pytest.raises(UnsupportedSizeError, match="multiple of 8"):
        ops.check_product_sizes(100, torch.bfloat16, "test")
    ops.check_product_sizes(100, torch.float32, "test")
    x = torch.zeros(2, 100, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(8, 100, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(UnsupportedSizeError):
        ops.prepare_weight(w)
    with pytest.raises(TypeError, match="prepare_weight"):      # bfloat16 weights are packed first
        ops.linear(x[:, :96].contiguous(), w[:, :96].contiguous(),
                   torch.zeros(2, 8, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize("n,k", [(16, 32), (90, 96), (65, 104), (896, 4864), (257, 136)])
def test_pack_weight_layout(ops, n, k):
    """Tile t of strip s holds W[16 s + l % 16, 32 t + 8 (l / 16) .. + 7] at 8 l; zeros past n and k."""
    w = rnd((n, k), torch.bfloat16, 91)
    packed = ops.prepare_weight(w.to(DEV))
    assert packed.shape == (n, k)
    strips, tiles = (n + 15) // 16, (k + 31) // 32
    padded = torch.zeros(strips * 16, tiles * 32, dtype=torch.bfloat16)
    padded[:n, :k] = w
    want = padded.view(strips, 16, tiles, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(-1)
    assert torch.equal(packed.data.cpu(), want)


@pytest.mark.parametrize("page,d", [(16, 16), (16, 48), (32, 32), (64, 64), (64, 128), (128, 80)])
def test_cache_order_round_trip(page, d):
    """The index maps are permutations of the page, and undo each other."""
    k = rnd((3, 2, page, d), torch.float32, 71)
    v = rnd((3, 2, d, page), torch.float32, 72)
    ki, vi = cache_layout.key_index(page, d), cache_layout.value_index(page, d)
    assert sorted(ki.reshape(-1).tolist()) == list(range(page * d))
    assert sorted(vi.reshape(-1).tolist()) == list(range(page * d))
    assert torch.equal(cache_layout.keys_from_cache_order(cache_layout.keys_to_cache_order(k)), k)
    assert torch.equal(cache_layout.values_from_cache_order(cache_layout.values_to_cache_order(v)), v)
    # a 16-key block is 16 * d consecutive numbers, for keys and for values
    assert int(ki[:16].max()) == 16 * d - 1 and int(vi[:, :16].max()) == 16 * d - 1


@pytest.mark.parametrize("m,n,k,splits", [(8, 896, 4864, 4), (1, 896, 896, 3), (16, 90, 512, 2), (5, 130, 264, 1),
                                          (40, 896, 512, 2), (64, 130, 264, 3), (200, 896, 4864, 4),
                                          (577, 300, 1160, 3), (130, 64, 72, 2)])
def test_linear_partials_and_pending(ops, emu, m, n, k, splits):
    """A product left in pieces along K; the pieces added on the fly where the rows are
    read (fused norm + product), folded in where a product adds into them, or folded
    by the stand-alone kernel: each against the same sum done at once."""
    bf = torch.bfloat16
    x, w = rnd((m, k), bf, 81), rnd((n, k), bf, 82, 0.1)
    parts = torch.zeros(ops.MAX_SPLITS, m, n, device=DEV)
    pending = ops.linear_partials(x.to(DEV), ops.prepare_weight(w.to(DEV)), parts, splits)
    want_parts = torch.zeros(ops.MAX_SPLITS, m, n)
    emu.linear_partials(x, w, want_parts, splits)
    close(parts[:splits], want_parts[:splits], torch.float32, "pieces", want_parts.abs().max().item())
    whole = x.float() @ w.float().t()
    close(parts[:splits].sum(0), whole, torch.float32, "sum of pieces", whole.abs().max().item())
    # stand-alone fold
    resid = rnd((m, n), torch.float32, 83)
    got = resid.clone().to(DEV)
    ops.add_pending(got, pending)
    close(got, resid + want_parts[:splits].sum(0), torch.float32, "fold", 4.0)
    # fold with the next product into the same rows
    x2, w2 = rnd((m, 96), bf, 84), rnd((n, 96), bf, 85, 0.1)
    got = resid.clone().to(DEV)
    ops.linear_residual(x2.to(DEV), ops.prepare_weight(w2.to(DEV)), got, pending=pending)
    want = resid + want_parts[:splits].sum(0) + x2.float() @ w2.float().t()
    close(got, want, torch.float32, "fold with a product", want.abs().max().item())
    # folded in by a stand-alone norm of the rows
    nw32 = 1 + 0.1 * rnd((n,), torch.float32, 88)
    got, normed = resid.clone().to(DEV), torch.empty(m, n, dtype=bf, device=DEV)
    ops.rmsnorm(got, nw32.to(DEV), 1e-6, normed, pending=pending)
    whole_rows = resid + want_parts[:splits].sum(0)
    close(got, whole_rows, torch.float32, "fold under a norm", 4.0)
    want_n = torch.empty(m, n, dtype=bf)
    emu.rmsnorm(whole_rows, nw32, 1e-6, want_n)
    close(normed, want_n, bf, "norm of the folded rows", 4.0)
    # added on the fly by a fused norm + product that reads the rows (n must fit the norm: use n wide rows)
    if n % 8 == 0 and m <= 64:
        nw = (1 + 0.1 * rnd((n,), torch.float32, 86)).to(bf)
        w3 = rnd((48, n), bf, 87, 0.1)
        logits = torch.zeros(m, 48, device=DEV)
        ops.fused_norm_logits(resid.to(DEV), None, nw.to(DEV), 1e-6, ops.prepare_weight(w3.to(DEV)), logits,
                              pending=pending)
        want_l = torch.zeros(m, 48)
        emu.fused_norm_logits(resid, None, nw, 1e-6, w3, want_l,
                              pending=type(pending)(want_parts, splits))
        close(logits, want_l, torch.float32, "pending under a fused norm", want_l.abs().max().item() * 4)


def test_bounded_wait_of_the_measured_grid_barrier_gives_up():
    """The benchmark's barrier loop (csrc/measure.hip) waits for all blocks at a counter; the
    wait is bounded.  Told to give up at once (a spin limit of 0) with a counter that can
    never fill (it starts far below zero), every block sets the flag and leaves; with room to
    spin and a counter at zero all rounds complete and the flag stays clear."""
    import ctypes
    from llm_inference_lab_amd.kernels import build
    lib = ctypes.CDLL(build.measure_library())
    lib.llmlab_measure_barrier.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_long, ctypes.c_void_p]
    stream = torch.cuda.current_stream(DEV).cuda_stream
    flags = torch.tensor([-1000000, 0], dtype=torch.int32, device=DEV)
    assert lib.llmlab_measure_barrier(64, 3, flags.data_ptr(), flags.data_ptr() + 4, 0, stream) == 0
    torch.cuda.synchronize(DEV)
    assert flags.cpu().tolist() == [-1000000 + 64, 1]
    flags = torch.zeros(2, dtype=torch.int32, device=DEV)
    assert lib.llmlab_measure_barrier(64, 5, flags.data_ptr(), flags.data_ptr() + 4, 1 << 22, stream) == 0
    torch.cuda.synchronize(DEV)
    assert flags.cpu().tolist() == [5 * 64, 0]
