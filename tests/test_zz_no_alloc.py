"""The entry point that allocates nothing (``llmlab_argmax_static``, csrc/no_alloc.h)
against ``llmlab_argmax``: called through ctypes twice in a row, the second time with
a smaller input, so that what the first call left in the library's device array would
show if the second read it; then a size beyond the array's, which must be refused."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _library():
    from llm_inference_lab_amd.kernels import build
    lib = ctypes.CDLL(build.core_library())
    vp, ci, cl, cs = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_size_t
    lib.llmlab_last_error.restype = ctypes.c_char_p
    lib.llmlab_argmax.argtypes = [vp, cl, ci, ci, vp, vp, cs, vp, cs, vp]
    lib.llmlab_argmax.restype = ci
    lib.llmlab_argmax_static.argtypes = [vp, cl, ci, ci, vp, vp]
    lib.llmlab_argmax_static.restype = ci
    return lib


def _both(lib, logits, workspace):
    rows, vocab = logits.shape
    stream = torch.cuda.current_stream(DEV).cuda_stream
    want = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
    got = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
    code = lib.llmlab_argmax(logits.data_ptr(), logits.stride(0), rows, vocab, want.data_ptr(),
                             workspace.data_ptr(), workspace.numel(), None, 0, stream)     # (its two kernels)
    assert code == 0, lib.llmlab_last_error()
    code = lib.llmlab_argmax_static(logits.data_ptr(), logits.stride(0), rows, vocab, got.data_ptr(),
                                    stream)
    assert code == 0, lib.llmlab_last_error()
    torch.cuda.synchronize(DEV)
    return got.cpu(), want.cpu()


def test_argmax_static_matches_argmax_on_two_calls_in_a_row():
    torch.cuda.set_device(DEV)
    lib = _library()
    workspace = torch.empty(1 << 16, dtype=torch.float32, device=DEV)
    gen = torch.Generator().manual_seed(5)
    # first call: many rows, a vocabulary of 19 chunks with a partial last one
    big = torch.randn((48, 151936), generator=gen)
    big[3, 151935] = 9.0                    # the winner in the last, partial chunk
    big[4, 8192] = big[4, 70000] = 8.0      # a tie across chunks goes to the smaller index
    big[5, :] = float("nan")                # nothing to choose
    got, want = _both(lib, big.to(DEV), workspace)
    assert torch.equal(got, want)
    assert got[3] == 151935 and got[4] == 8192 and got[5] == -1
    assert torch.equal(got[6:], big[6:].argmax(dim=1).int())
    # second call: fewer rows and chunks; its partial results overlap what the first left
    small = torch.randn((5, 20000), generator=gen)
    small[1, 19999] = 9.0
    small[2, :] = float("nan")
    got, want = _both(lib, small.to(DEV), workspace)
    assert torch.equal(got, want)
    assert got[1] == 19999 and got[2] == -1
    assert got[0] == small[0].argmax() and got[3] == small[3].argmax()


def test_argmax_static_refuses_what_its_array_cannot_hold():
    torch.cuda.set_device(DEV)
    lib = _library()
    rows, vocab = 4100, 8192 * 8 + 1          # 4100 * 9 partial results > 32768
    logits = torch.zeros((1, vocab), dtype=torch.float32, device=DEV)     # never read: refused first
    out = torch.zeros(rows, dtype=torch.int32, device=DEV)
    code = lib.llmlab_argmax_static(logits.data_ptr(), vocab, rows, vocab, out.data_ptr(),
                                    torch.cuda.current_stream(DEV).cuda_stream)
    assert code != 0
    assert b"static array" in lib.llmlab_last_error()
