"""The kernel set of the engine: thin, checked ctypes calls into the HIP
libraries.  There is no other implementation on the product path: without a
GPU, or if a library cannot be built or loaded, constructing ``HipOps`` raises.

Every call checks on the host that dtypes, shapes, strides and devices are what
the kernel and its grid assume before it launches anything; a size that the
kernels do not take is refused with ``UnsupportedSizeError``.  Kernels run on
the current PyTorch stream, so they can be captured into a HIP graph.
"""
from __future__ import annotations

import ctypes
import dataclasses
from typing import Dict, Optional

import torch

from ..config.errors import UnsupportedSizeError
from ..parts.base import PendingSums
from . import build
from .debug import DispatchRules, KernelDebug

DT_F32, DT_BF16 = 0, 1
EPI_STORE, EPI_RESID, EPI_F32, EPI_SWIGLU, EPI_QKV, EPI_PART = 0, 1, 2, 3, 4, 5

_c_int, _c_long, _c_float, _c_size, _c_ptr = (ctypes.c_int, ctypes.c_long, ctypes.c_float,
                                              ctypes.c_size_t, ctypes.c_void_p)


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return DT_F32
    if t.dtype == torch.bfloat16:
        return DT_BF16
    raise TypeError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}")


class KernelError(RuntimeError):
    pass


_NO_HEADS = (None, None, None, None, 0, 0, None, None, 0, 0, 0)     # a few-row product without the q/k/v epilogue


class PackedWeight:
    """A bfloat16 matrix [n, k] in the order the matrix cores read it: strips of 16
    rows, a strip a run of 1 KB tiles (16 rows x 32 columns, one MFMA B operand,
    lane l owning 16 bytes), zero-padded to whole tiles.  Made by
    ``HipOps.prepare_weight``; the product kernels take nothing else in bfloat16."""

    __slots__ = ("data", "shape", "dtype", "device")

    def __init__(self, data: torch.Tensor, n: int, k: int):
        self.data = data
        self.shape = (n, k)
        self.dtype = data.dtype
        self.device = data.device

    def data_ptr(self) -> int:
        return self.data.data_ptr()

    def is_contiguous(self) -> bool:
        return True

    def numel(self) -> int:
        return self.shape[0] * self.shape[1]

    def element_size(self) -> int:
        return self.data.element_size()


class LaunchRecord:
    """The calls into the kernel libraries that a part made while it was recorded, so that
    the same part under the same conditions can make them again without its Python code:
    ``calls[i]`` is ``(function, argument list, library)``, or ``(None, callable, None)``
    for a call that depends on the step's data and is made anew through its closure
    (``HipOps.live``).  ``dry``: nothing is launched while recording (a recorded sequence is
    only compared with one kept from before)."""

    __slots__ = ("calls", "dry")

    def __init__(self, dry: bool = False):
        self.calls = []
        self.dry = dry

    def same_as(self, other: "LaunchRecord") -> bool:
        if len(self.calls) != len(other.calls):
            return False
        for (fa, aa, _), (fb, ab, _) in zip(self.calls, other.calls):
            if (fa is None) != (fb is None):
                return False
            if fa is not None and (fa is not fb or list(aa[:-1]) != list(ab[:-1])):     # (the last is the stream)
                return False
        return True


class AttentionCall:
    """An attention call with its unchanging arguments checked and laid out
    (``HipOps.prepare_attention``)."""

    __slots__ = ("ops", "lib", "args", "most_requests", "most_context", "row_req", "heads", "dtype")
    N_REQS, MAX_Q, MAX_CTX, ROW_REQ, SHORT_LEN, N_SHORT, SHORT_CTX, STREAM = 12, 13, 14, 23, 24, 25, 26, 29

    def __init__(self, ops, lib, args, most_requests, most_context, row_req, heads, dtype):
        self.ops, self.lib, self.args = ops, lib, args
        self.most_requests, self.most_context, self.row_req = most_requests, most_context, row_req
        self.heads, self.dtype = heads, dtype

    def launch(self, n_reqs: int, max_q_len: int, max_ctx_len: int, short=None) -> None:
        if n_reqs > self.most_requests:
            raise ValueError("attention: request arrays are shorter than the number of requests")
        if max_ctx_len > self.most_context:
            raise ValueError("attention: the block table is too narrow for the longest context")
        a = self.args
        a[self.N_REQS], a[self.MAX_Q], a[self.MAX_CTX] = n_reqs, max_q_len, max_ctx_len
        if short is not None:
            _, short_len, n_short, short_ctx = short
            if (short_len != self.ops.attention_short_limit(self.heads[0], self.heads[1], self.dtype, max_q_len)
                    or not 0 < n_short < n_reqs or short_ctx > max_ctx_len or self.row_req is None):
                raise ValueError("attention: the description of the step's short requests does not fit")
            a[self.ROW_REQ], a[self.SHORT_LEN], a[self.N_SHORT], a[self.SHORT_CTX] = self.row_req, short_len, n_short, short_ctx
        else:
            a[self.ROW_REQ], a[self.SHORT_LEN], a[self.N_SHORT], a[self.SHORT_CTX] = None, 0, 0, 0
        a[self.STREAM] = self.ops._stream()
        self.ops._call(self.lib.llmlab_paged_attention, *a, lib=self.lib)


class HipOps:
    WORKSPACE_FLOATS = 16 * 1024 * 1024      # 64 MiB of float32 scratch (split partial sums)
    ARRIVED_INTS = 64 * 1024                 # arrival counters: one per (request, kv head) of a step

    def __init__(self, device="cuda:0"):
        if not torch.cuda.is_available():
            raise RuntimeError(
                "no GPU is visible: the engine runs on hand-written HIP kernels for gfx950 "
                "and has no CPU path")
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError(f"the kernels need a GPU device, got '{device}'")
        torch.cuda.set_device(self.device)
        if self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        self._core = self._load(build.core_library())
        self._declare_core()
        if self._core.llmlab_abi_version() != 6:
            raise RuntimeError("kernel library and Python bindings disagree on the interface")
        self._attn: Dict[int, ctypes.CDLL] = {}
        self._shared: Dict[int, tuple] = {}
        self.num_cus = int(torch.cuda.get_device_properties(self.device).multi_processor_count)
        self.workspace = torch.empty(self.WORKSPACE_FLOATS, dtype=torch.float32, device=self.device)
        # Counters by which blocks of one kernel find out which of them is the last to arrive
        # (the key splits of decode attention, the pieces of the argmax).  Zero between
        # launches: the block that reads the full count sets its counter back.
        self.arrived = torch.zeros(self.ARRIVED_INTS, dtype=torch.int32, device=self.device)
        self.loaded_libraries = [self._core._name]
        self.calls_made = 0          # calls into the kernel libraries so far
        self._record: Optional[LaunchRecord] = None
        self.debug_epoch = 0         # counts the changes of forced kernel choices (kernels/debug.py)
        self.rules = DispatchRules()         # the measured thresholds of the dispatch, in one place
        self.debug = KernelDebug(self)       # forcing kernel choices from outside (tests, measurements)

    # ---------------------------------------------------------------- loading
    @staticmethod
    def _load(path: str) -> ctypes.CDLL:
        try:
            return ctypes.CDLL(path)
        except OSError as e:
            raise RuntimeError(f"cannot load the kernel library {path}: {e}") from None

    def _declare_core(self) -> None:
        c = self._core
        c.llmlab_last_error.restype = ctypes.c_char_p
        c.llmlab_abi_version.restype = _c_int
        c.llmlab_embed.argtypes = [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr]
        c.llmlab_rmsnorm.argtypes = [_c_ptr, _c_ptr, _c_int, _c_float, _c_ptr, _c_int, _c_ptr, _c_int,
                                     _c_int, _c_ptr, _c_int, _c_size, _c_ptr]
        c.llmlab_rope_kv_write.argtypes = [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                           _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr,
                                           _c_ptr, _c_ptr]
        c.llmlab_rope_inplace.argtypes = [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_long, _c_long,
                                          _c_ptr, _c_ptr, _c_ptr]
        c.llmlab_linear.argtypes = [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_int,
                                    _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr]
        c.llmlab_sample.argtypes = [_c_ptr, _c_long, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr]
        c.llmlab_gather_tokens.argtypes = [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr]
        c.llmlab_gather_tokens.restype = _c_int
        c.llmlab_packed_elements.argtypes = [_c_int, _c_int]
        c.llmlab_packed_elements.restype = _c_long
        c.llmlab_pack_weight.argtypes = [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr]
        c.llmlab_pack_weight.restype = _c_int
        c.llmlab_argmax.argtypes = [_c_ptr, _c_long, _c_int, _c_int, _c_ptr, _c_ptr, _c_size, _c_ptr, _c_size,
                                    _c_ptr]
        c.llmlab_argmax.restype = _c_int
        c.llmlab_linear_qkv.argtypes = [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int,
                                        _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr,
                                        _c_int, _c_int, _c_int, _c_int, _c_ptr]
        c.llmlab_linear_tile.argtypes = [_c_int, _c_int, _c_int, _c_int]
        c.llmlab_linear_tile.restype = _c_int
        c.llmlab_linear_partials.argtypes = [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int,
                                             _c_int, _c_int, _c_size, _c_int, _c_ptr]
        c.llmlab_qkv_from_pieces.argtypes = [_c_ptr, _c_int, _c_size, _c_int, _c_ptr, _c_int, _c_int, _c_int,
                                             _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                                             _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr]
        c.llmlab_qkv_from_pieces.restype = _c_int
        c.llmlab_linear_plan.argtypes = [_c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr]
        c.llmlab_linear_plan.restype = None
        c.llmlab_skinny_linear.argtypes = [
            _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_float, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr,
            _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
            _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int,
            _c_ptr, _c_int, _c_int, _c_size, _c_int, _c_size, _c_ptr]
        c.llmlab_add_pending.argtypes = [_c_ptr, _c_ptr, _c_int, _c_size, _c_int, _c_int, _c_ptr]
        c.llmlab_add_pending.restype = _c_int
        for fn in (c.llmlab_embed, c.llmlab_rmsnorm, c.llmlab_rope_kv_write, c.llmlab_rope_inplace,
                   c.llmlab_linear, c.llmlab_sample, c.llmlab_skinny_linear,
                   c.llmlab_linear_partials, c.llmlab_linear_qkv):
            fn.restype = _c_int

    def _attention_lib(self, head_dim: int) -> ctypes.CDLL:
        lib = self._attn.get(head_dim)
        if lib is None:
            lib = self._load(build.attention_library(head_dim))
            lib.llmlab_last_error.restype = ctypes.c_char_p
            lib.llmlab_attention_head_dim.restype = _c_int
            if lib.llmlab_attention_head_dim() != head_dim:
                raise RuntimeError(f"attention library for head size {head_dim} reports "
                                   f"{lib.llmlab_attention_head_dim()}")
            lib.llmlab_paged_attention.argtypes = [
                _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr,
                _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_float, _c_ptr, _c_int, _c_ptr, _c_size,
                _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_size, _c_ptr]
            lib.llmlab_paged_attention.restype = _c_int
            self._attn[head_dim] = lib
            self.loaded_libraries.append(lib._name)
        return lib

    def check_attention_sizes(self, num_heads: int, num_kv_heads: int, head_dim: int, dtype) -> None:
        if head_dim % 16 != 0 or not 16 <= head_dim <= 256:
            raise UnsupportedSizeError(
                f"attention kernels take head sizes that are multiples of 16 from 16 to 256, "
                f"got {head_dim} (in float32 too: the pages of keys and values are laid out in "
                f"blocks of 16 numbers of a head for both dtypes, and the kernels are compiled "
                f"per head size)")
        if num_heads % num_kv_heads != 0:
            raise UnsupportedSizeError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        self._attention_lib(head_dim)

    def check_product_sizes(self, inner: int, dtype, what: str) -> None:
        """Refuse at load time what the matrix product kernels do not take."""
        if dtype == torch.bfloat16 and inner % 8 != 0:
            raise UnsupportedSizeError(
                f"{what}: bfloat16 matrix products need an inner size that is a multiple of 8, "
                f"got {inner} (the float32 path takes any size)")

    def prepare_weight(self, w: torch.Tensor, shared: bool = False):
        """What the product kernels take for the matrix ``w`` [n, k]: float32 as it is,
        bfloat16 packed in fragment order (a copy; ``w`` itself is not kept).

        ``shared``: parts that may be bound to one and the same tensor (an embedding
        and an output head with tied weights) get one packed copy between them;
        the model calls ``release_shared()`` when all its parts are bound."""
        if shared and id(w) in self._shared:
            return self._shared[id(w)][1]
        packed = self._prepare(w)
        if shared:
            self._shared[id(w)] = (w, packed)       # w is held so that its id stays its own
        return packed

    def release_shared(self) -> None:
        self._shared.clear()

    def _prepare(self, w: torch.Tensor):
        self._need(w, "weight")
        if w.dim() != 2:
            raise ValueError(f"a weight matrix has two dimensions, got {tuple(w.shape)}")
        if w.dtype == torch.float32:
            return w
        if w.dtype != torch.bfloat16:
            raise TypeError(f"weights are float32 or bfloat16, got {w.dtype}")
        n, k = w.shape
        self.check_product_sizes(k, w.dtype, "weight matrix")
        data = torch.empty(self._core.llmlab_packed_elements(n, k), dtype=torch.bfloat16, device=self.device)
        self._call(self._core.llmlab_pack_weight, self._ptr(w), self._ptr(data), n, k, self._stream())
        return PackedWeight(data, n, k)

    def _weight(self, w, name: str):
        """The weight operand of a product: packed if bfloat16."""
        if isinstance(w, PackedWeight):
            if w.device != self.device:
                raise ValueError(f"{name} is on {w.device}, the kernels run on {self.device}")
            return w
        self._need(w, name)
        if w.dtype == torch.bfloat16:
            raise TypeError(f"{name}: bfloat16 weights go through prepare_weight() once, when the "
                            f"part is bound; the product kernels read the packed order only")
        return w

    # ---------------------------------------------------------------- helpers
    def _stream(self):
        # the raw handle of the current stream (under graph capture: the capturing one);
        # asked for at every launch, so by the short way where torch has one
        raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        if raw is not None:
            return raw(self.device.index)
        return torch.cuda.current_stream(self.device).cuda_stream

    def _call(self, fn, *args, lib=None) -> None:
        """One call into the kernel libraries; a failure raises with the library's message."""
        self.calls_made += 1
        if self._record is not None:
            self._record.calls.append((fn, list(args), lib))
            if self._record.dry:
                return
        code = fn(*args)
        if code != 0:
            self._check(code, lib)

    # ------------------------------------------------- recorded launch sequences
    def begin_recording(self, dry: bool = False) -> LaunchRecord:
        """From now until ``end_recording`` every call into the kernel libraries is also
        written down (``engine/model.py`` keeps the sequences of its blocks and replays
        them for steps of the same shape)."""
        if self._record is not None:
            raise RuntimeError("a recording is already under way")
        self._record = LaunchRecord(dry)
        return self._record

    def end_recording(self) -> Optional[LaunchRecord]:
        record, self._record = self._record, None
        return record

    def live(self, launch) -> None:
        """``launch()`` makes calls whose arguments depend on the step's data (how many
        requests, how long their histories): while a sequence is recorded it is written
        down as a closure, to be called anew at every replay, and its own calls are not."""
        record = self._record
        if record is None:
            launch()
            return
        record.calls.append((None, launch, None))
        if record.dry:
            return
        self._record = None
        try:
            launch()
        finally:
            self._record = record

    def replay(self, record: LaunchRecord) -> None:
        """Make a recorded sequence of calls again, on the current stream."""
        stream = self._stream()
        for fn, args, lib in record.calls:
            if fn is None:
                args()
                continue
            args[-1] = stream
            self.calls_made += 1
            code = fn(*args)
            if code != 0:
                self._check(code, lib)

    def fingerprint(self):
        """What the host-side choices of the kernel set depend on beside the shapes."""
        return (self.num_cus, self.debug_epoch, dataclasses.astuple(self.rules))

    def _check(self, code: int, lib=None) -> None:
        if code != 0:
            msg = (lib or self._core).llmlab_last_error()
            raise KernelError(msg.decode() if msg else f"kernel call failed with code {code}")

    def _need(self, t: torch.Tensor, name: str, dtype=None, contiguous=True) -> torch.Tensor:
        if t.device != self.device:
            raise ValueError(f"{name} is on {t.device}, the kernels run on {self.device}")
        if dtype is not None and t.dtype != dtype:
            raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
        if contiguous and not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
        return t

    @staticmethod
    def _ptr(t: Optional[torch.Tensor]):
        # (a plain integer: ctypes makes the pointer argument of it, None is the null pointer)
        return t.data_ptr() if t is not None else None

    def synchronize(self) -> None:
        torch.cuda.synchronize(self.device)

    # ------------------------------------------------------------ elementwise
    def embed(self, table, ids, out) -> None:
        """Rows of ``table`` (float32, bfloat16, or bfloat16 packed by prepare_weight)."""
        packed = isinstance(table, PackedWeight)
        if not packed:
            self._need(table, "embedding table")
        self._need(ids, "token ids", torch.int32)
        self._need(out, "embedding output", torch.float32)
        rows, hidden = out.shape
        if ids.numel() != rows or table.shape[1] != hidden:
            raise ValueError(f"embed: ids {tuple(ids.shape)}, table {tuple(table.shape)}, "
                             f"out {tuple(out.shape)} do not fit")
        self._call(self._core.llmlab_embed, self._ptr(table), _dt(table), 1 if packed else 0,
                                            self._ptr(ids), self._ptr(out), rows, hidden, table.shape[0],
                                            self._stream())

    def gather_tokens(self, dst, dst_index, src, src_index, n) -> None:
        """dst[dst_index[i]] = src[src_index[i]] for i < n (all int32 on the GPU)."""
        for t, name in ((dst, "dst"), (dst_index, "dst_index"), (src, "src"), (src_index, "src_index")):
            self._need(t, f"gather_tokens {name}", torch.int32)
        if dst_index.numel() < n or src_index.numel() < n:
            raise ValueError("gather_tokens: index arrays are shorter than the count")
        self._call(self._core.llmlab_gather_tokens, self._ptr(dst), self._ptr(dst_index), self._ptr(src),
                                                    self._ptr(src_index), int(n), self._stream())

    def rmsnorm(self, x, weight, eps, out, rows=None, pending=None) -> None:
        """``out[i] = norm(x[rows[i]])``.  ``pending`` (all rows in order only): the pieces are
        folded into ``x`` on the way, ``x += sum_s parts[s]``, and the whole rows are normed."""
        self._need(x, "norm input", torch.float32)
        self._need(weight, "norm weight")
        self._need(out, "norm output")
        hidden = x.shape[1]
        n_out = out.shape[0]
        if weight.numel() != hidden or out.shape[1] != hidden:
            raise ValueError(f"rmsnorm: x {tuple(x.shape)}, weight {tuple(weight.shape)}, "
                             f"out {tuple(out.shape)} do not fit")
        if rows is None:
            if n_out != x.shape[0]:
                raise ValueError("rmsnorm: output rows differ from input rows")
        else:
            self._need(rows, "norm row indices", torch.int32)
            if rows.numel() != n_out:
                raise ValueError("rmsnorm: one row index per output row")
        pend = (None, 0, 0)
        if pending is not None:
            p = pending.parts
            if rows is not None or p.shape[1] != n_out or p.shape[2] != hidden or not p[0].is_contiguous():
                raise ValueError("rmsnorm: pending sums go with all rows in order and the same shape")
            pend = (self._ptr(p), pending.splits, p.stride(0))
        self._call(self._core.llmlab_rmsnorm, self._ptr(x), self._ptr(weight), _dt(weight), float(eps),
                                              self._ptr(out), _dt(out), self._ptr(rows), n_out, hidden,
                                              pend[0], pend[1], pend[2], self._stream())

    # ----------------------------------------------------------------- linear
    def _linear(self, x, w, out, bias, epilogue, n_out, pending: Optional[PendingSums] = None) -> None:
        self._need(x, "linear input")
        w = self._weight(w, "linear weight")
        if x.dtype != w.dtype:
            raise TypeError(f"linear: input is {x.dtype} but the weight is {w.dtype}")
        if out.device != self.device or out.stride(-1) != 1:
            raise ValueError("linear: output must be on the GPU with unit column stride")
        m, k = x.shape
        n = w.shape[0]
        if w.shape[1] != k or out.shape[0] != m or out.shape[1] != n_out:
            raise ValueError(f"linear: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} "
                             f"do not fit")
        if x.dtype == torch.bfloat16 and k % 8 != 0:
            raise UnsupportedSizeError(
                f"bfloat16 matrix products need an inner size that is a multiple of 8, got {k}")
        want_out = x.dtype if epilogue in (EPI_STORE, EPI_SWIGLU) else torch.float32
        if out.dtype != want_out:
            raise TypeError(f"linear: output must be {want_out}, got {out.dtype}")
        if bias is not None:
            self._need(bias, "linear bias")
            if bias.numel() != n:
                raise ValueError("linear: bias length differs from the output width")
        ldo = out.stride(0) if m > 1 else max(out.stride(0), n_out)
        # few rows: the block kernel that splits K inside a block; from 17 rows on only
        # for narrow outputs (the tiled kernel has too few tiles there), measured
        if x.dtype == torch.bfloat16 and (m <= 16 or (n < 8192 and self.few_rows_take(m, n, k))):
            self._skinny(x, False, None, None, 0.0, w, bias, epilogue, out, m, n, k, ldo, n_out,
                         pending=pending)
            return
        if pending is not None:
            self.add_pending(out, pending)
        self._call(self._core.llmlab_linear,
            self._ptr(x), self._ptr(w), _dt(x), epilogue, self._ptr(out), self._ptr(bias),
            _dt(bias) if bias is not None else 0, m, n, k, ldo, n_out, self.num_cus, self._stream())

    def linear(self, x, w, out, bias=None) -> None:
        self._linear(x, w, out, bias, EPI_STORE, w.shape[0])

    def linear_residual(self, x, w, resid, bias=None, pending: Optional[PendingSums] = None) -> None:
        """``resid += x w^T (+ bias)``, and the pending pieces of ``resid`` with it."""
        self._linear(x, w, resid, bias, EPI_RESID, w.shape[0], pending)

    def linear_logits(self, x, w, out) -> None:
        self._linear(x, w, out, None, EPI_F32, w.shape[0])

    def linear_swiglu(self, x, w_gate_up, out) -> None:
        inter = out.shape[1]
        if w_gate_up.shape[0] != 2 * ((inter + 15) // 16 * 16):
            raise ValueError(f"linear_swiglu: {w_gate_up.shape[0]} interleaved rows do not belong "
                             f"to {inter} outputs")
        self._linear(x, w_gate_up, out, None, EPI_SWIGLU, inter)

    # ----------------------------------------------- few rows: fused kernels
    FUSED_MAX_ROWS = 1024         # most rows the few-row kernels take at all
    FEW_ROWS = 64                 # up to here a product may take them whatever its matrix
    FUSE_TILE_ROWS = 16           # the few-row kernels cut the rows into tiles of so many

    def few_rows_take(self, rows: int, outer: int, inner: int) -> bool:
        """Whether a plain product of ``rows`` rows with an ``[outer, inner]`` matrix goes to the
        few-row kernels: always up to 64 rows; beyond, up to ``rules.few_rows_max`` rows while
        the matrix, read once per tile of 16 rows, stays below ``rules.few_rows_read_bytes``."""
        if rows <= self.FEW_ROWS:
            return True
        tiles = (rows + self.FUSE_TILE_ROWS - 1) // self.FUSE_TILE_ROWS
        return (rows <= min(self.rules.few_rows_max, self.FUSED_MAX_ROWS)
                and 2.0 * outer * inner * tiles < self.rules.few_rows_read_bytes)
    STAGE_BYTES = 118 * 1024      # most LDS the staged rows of a fused kernel may take

    def can_fuse(self, rows: int, dtype, inner: int, outer: Optional[int] = None) -> bool:
        """Whether the fused few-row kernels take this step: bfloat16, few rows, a tile
        of rows (``inner`` wide) fits the staging buffer in LDS, and beyond one tile the
        matrix (``outer`` rows) is a small one."""
        if dtype != torch.bfloat16 or not 0 < rows <= min(max(self.FEW_ROWS, self.rules.few_rows_max), self.FUSED_MAX_ROWS):
            return False
        tiles = (rows + self.FUSE_TILE_ROWS - 1) // self.FUSE_TILE_ROWS
        limit = self.rules.fuse_read_bytes if rows <= self.FEW_ROWS else self.rules.few_rows_read_bytes
        if tiles > 1 and (outer is None or 2.0 * outer * inner * tiles >= limit):
            return False
        return min(rows, self.FUSE_TILE_ROWS) * ((inner + 31) // 32 * 32 + 8) * 2 <= self.STAGE_BYTES

    def _skinny(self, x, norm, x_rows, norm_w, eps, w, bias, epilogue, out, m, n, k, ldo, n_out,
                qkv=None, pending: Optional[PendingSums] = None, ksplit: int = 1,
                part_stride: int = 0) -> None:
        if pending is not None:
            p = pending.parts
            if (p.dtype != torch.float32 or p.dim() != 3 or p.stride(2) != 1 or p.device != self.device
                    or pending.splits > p.shape[0]):
                raise ValueError("pending sums: float32 [splits, rows, width] on the GPU expected")
            width = x.shape[1] if norm else n
            if p.shape[2] != width:
                raise ValueError(f"pending sums are {p.shape[2]} wide, the rows they belong to {width}")
            pend = (self._ptr(p), pending.splits, p.stride(1), p.stride(0))
        else:
            pend = (None, 0, 0, 0)
        if qkv is None:
            heads = _NO_HEADS
        else:
            table, ptr = qkv["table"], self._ptr
            heads = (ptr(qkv["inv_freq"]), ptr(qkv["positions"]), ptr(qkv["row_req"]), ptr(table),
                     table.stride(0) if table is not None else 0, qkv["page_size"], ptr(qkv["k_cache"]),
                     ptr(qkv["v_cache"]), qkv["nq"], qkv["nkv"], qkv["d"])
        self._call(self._core.llmlab_skinny_linear,
            x.data_ptr(), 1 if norm else 0, self._ptr(x_rows), self._ptr(norm_w),
            _dt(norm_w) if norm_w is not None else 0, float(eps), w.data_ptr(), self._ptr(bias),
            _dt(bias) if bias is not None else 0, epilogue, out.data_ptr(), m, n, k, ldo, n_out,
            *heads, self.num_cus, pend[0], pend[1], pend[2], pend[3], int(ksplit),
            int(part_stride), self._stream())

    # --------------------------------------------- sums left in pieces (deferred)
    MAX_SPLITS = 8
    split_max_rows = 32           # most rows of a few-row product that is left in pieces

    def pieces_too_large_to_read_per_block(self, pending: Optional[PendingSums]) -> bool:
        """A fused kernel that takes pieces on adds them as it reads the rows, in every one
        of its blocks; beyond this size the norm kernel should fold them once instead
        (32 rows of width 3584 in 7 pieces, 3.2 MB: 12 us a layer more in the fused kernels)."""
        if pending is None:
            return False
        p = pending.parts
        return pending.splits * p.shape[1] * p.shape[2] * 4 > self.rules.pieces_per_block_bytes

    def pieces_by_tiles(self, rows: int, n: int, k: int) -> bool:
        """Whether a product left in pieces is cut by the tiled kernel (else by the few-row one)."""
        return rows > self.FEW_ROWS or (rows > self.FUSE_TILE_ROWS and 2.0 * n * k >= self.rules.tiled_pieces_bytes)

    def split_count(self, rows: int, dtype, n: int, k: int) -> int:
        """Into how many pieces along the inner size a few-row product ``[rows, k] x
        [n, k]^T`` should be cut so that it spreads over the chip: a narrow output
        gives too few blocks otherwise, and a compute unit draws only so much from
        memory.  1: do not cut."""
        if dtype != torch.bfloat16 or rows <= 0:
            return 1
        if self.pieces_by_tiles(rows, n, k):
            # many rows, tiled kernel: its own estimate (rounds of blocks over the chip times
            # the K tiles of a block, plus a write and a read of the result for every piece)
            if k % 8:
                return 1
            if self.rules.forced_tiled_pieces:
                return max(1, min(self.rules.forced_tiled_pieces, (k + 63) // 64, self.MAX_SPLITS))
            return self._linear_plan(rows, n, k)[0]
        if rows > self.split_max_rows:
            return 1
        strips, steps = (n + 15) // 16, (k + 31) // 32
        most = min(steps // self.rules.min_steps_per_split, self.MAX_SPLITS)
        if strips > self.num_cus and rows <= self.FUSE_TILE_ROWS:
            # a wide output whose strips do not go evenly over the units (320 strips on 256
            # units: the busiest unit streams two, the chip waits for it): cut so that the
            # blocks fill whole rounds (5120 x 27648 at 8 rows: 70 us whole, 53 in 4 pieces)
            def waste(p):
                rounds = strips * p / self.num_cus
                return -(-strips * p // self.num_cus) / rounds
            if waste(1) < self.rules.uneven_rounds_waste:
                return 1
            for p in range(2, max(most, 1) + 1):
                if waste(p) <= 1.07:       # (3 pieces, 3.75 rounds, do as well as 4 and cost the next reader less)
                    return p
            return 1
        want = self.num_cus // max(strips, 1)
        return max(1, min(want, most))

    def _linear_plan(self, rows: int, n: int, k: int):
        """(pieces, tile) for a many-row product that adds into float32 rows."""
        out = (_c_int * 2)()
        self._core.llmlab_linear_plan(rows, n, k, self.num_cus, self.MAX_SPLITS, self.rules.min_tiles_per_split, out)
        return out[0], out[1]

    def linear_partials(self, x, w, parts: torch.Tensor, splits: int, bias=None) -> PendingSums:
        """``parts[s] = x[:, K_s] w[:, K_s]^T`` for the ``splits`` pieces ``K_s`` of the inner
        size (bias in piece 0): the product without the final sum."""
        self._need(x, "linear input", torch.bfloat16)
        w = self._weight(w, "linear weight")
        m, k = x.shape
        n = w.shape[0]
        if (w.shape[1] != k or parts.dtype != torch.float32 or parts.dim() != 3 or parts.shape[0] < splits
                or parts.shape[1] != m or parts.shape[2] != n or parts.stride(2) != 1
                or parts.device != self.device):
            raise ValueError(f"linear_partials: x {tuple(x.shape)}, w {tuple(w.shape)}, "
                             f"parts {tuple(parts.shape)} for {splits} pieces do not fit")
        if not 1 <= splits <= self.MAX_SPLITS:
            raise ValueError(f"linear_partials: {splits} pieces")
        if not self.pieces_by_tiles(m, n, k):
            self._skinny(x, False, None, None, 0.0, w, bias, EPI_PART, parts, m, n, k, parts.stride(1), n,
                         ksplit=splits, part_stride=parts.stride(0))
        else:
            if bias is not None:
                self._need(bias, "bias")
            self._call(self._core.llmlab_linear_partials,
                self._ptr(x), self._ptr(w), self._ptr(parts), self._ptr(bias),
                _dt(bias) if bias is not None else 0, m, n, k, parts.stride(1), splits, parts.stride(0),
                self._linear_plan(m, n, k)[1], self._stream())
        return PendingSums(parts, splits)

    def add_pending(self, x: torch.Tensor, pending: PendingSums) -> None:
        """``x += sum_s parts[s]``: fold the pieces into the float32 stream."""
        self._need(x, "residual stream", torch.float32)
        p = pending.parts
        rows, width = x.shape
        if p.shape[1] != rows or p.shape[2] != width or not p[0].is_contiguous():
            raise ValueError("add_pending: pieces and stream differ in shape")
        self._call(self._core.llmlab_add_pending, self._ptr(x), self._ptr(p), pending.splits, p.stride(0),
                                                  rows, width, self._stream())

    def _fused_common(self, x, norm_w, w, rows):
        self._need(x, "residual stream", torch.float32)
        self._need(norm_w, "norm weight")
        w = self._weight(w, "weight")
        if w.dtype != torch.bfloat16:
            raise TypeError("the fused few-row kernels are bfloat16 kernels")
        k = x.shape[1]
        if norm_w.numel() != k or w.shape[1] != k:
            raise ValueError(f"fused norm + product: x {tuple(x.shape)}, norm weight "
                             f"{tuple(norm_w.shape)}, w {tuple(w.shape)} do not fit")
        if k % 8 != 0:
            raise UnsupportedSizeError(
                f"bfloat16 matrix products need an inner size that is a multiple of 8, got {k}")
        if not 0 < rows <= self.FUSED_MAX_ROWS:
            raise ValueError(f"the fused kernels take 1..{self.FUSED_MAX_ROWS} rows, got {rows}")
        return w, k

    def _qkv_checks(self, what, rows, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions,
                    row_req, block_table, page_size, k_cache, v_cache, q_out) -> int:
        n = (num_heads + 2 * num_kv_heads) * head_dim
        if w_qkv.shape[0] != n or tuple(q_out.shape) != (rows, num_heads * head_dim):
            raise ValueError(f"{what}: weight or output shape does not fit the heads")
        self._need(q_out, "q output", torch.bfloat16)
        self._need(positions, "positions", torch.int32)
        if positions.numel() < rows:
            raise ValueError(f"{what}: one position per row")
        if b_qkv is not None and b_qkv.numel() != n:
            raise ValueError(f"{what}: bias length")
        if inv_freq is not None and (inv_freq.dtype != torch.float32 or inv_freq.numel() != head_dim // 2):
            raise ValueError(f"{what}: the frequency table must hold head_dim/2 float32 entries")
        if k_cache is not None:
            self._need(row_req, "row -> request map", torch.int32)
            self._need(block_table, "block table", torch.int32)
            pages = k_cache.shape[0]
            if (tuple(k_cache.shape) != (pages, num_kv_heads, page_size, head_dim)
                    or tuple(v_cache.shape) != (pages, num_kv_heads, head_dim, page_size)
                    or not k_cache.is_contiguous() or not v_cache.is_contiguous()
                    or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16
                    or row_req.numel() < rows):
                raise ValueError(f"{what}: cache tensors do not have the paged layout")
        return n

    def fused_norm_qkv(self, x, norm_w, eps, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim, inv_freq,
                       positions, row_req, block_table, page_size, k_cache, v_cache, q_out,
                       pending: Optional[PendingSums] = None) -> None:
        """q_out = rotate(norm(x) Wq^T + bq); rotated k and v of the new positions go to
        their pages (skipped when no cache is given).  ``pending``: pieces still owed to
        the rows of x, added while they are read (x itself is left as it is)."""
        rows = x.shape[0]
        w_qkv, k = self._fused_common(x, norm_w, w_qkv, rows)
        n = self._qkv_checks("fused_norm_qkv", rows, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim,
                             inv_freq, positions, row_req, block_table, page_size, k_cache, v_cache, q_out)
        self._skinny(x, True, None, norm_w, eps, w_qkv, b_qkv, EPI_QKV, q_out, rows, n, k,
                     q_out.shape[1], n,
                     dict(inv_freq=inv_freq, positions=positions, row_req=row_req, table=block_table,
                          page_size=page_size, k_cache=k_cache, v_cache=v_cache, nq=num_heads,
                          nkv=num_kv_heads, d=head_dim), pending=pending)

    QKV_ROPE_MAX_ROWS = 64        # up to here the few-row kernel, beyond it the tiled one
    QKV_PIECES_MAX_ROWS = 384     # up to here a large matrix may go through pieces along its inner size

    def can_fuse_qkv_rope(self, rows: int, dtype, head_dim: int, n: Optional[int] = None,
                          k: Optional[int] = None) -> bool:
        """Whether ``qkv_rope_cache`` takes this step: bfloat16, and a head that one block
        holds (few rows: the few-row kernel's block; more: the tile that a product ``[rows, k]
        x [n, k]^T`` gets, which a head must divide)."""
        if dtype != torch.bfloat16 or rows <= 0 or head_dim % 16 or head_dim < 16:
            return False
        if rows <= self.QKV_ROPE_MAX_ROWS:
            return head_dim <= (128 if rows > 32 else 256)
        if n is not None and k is not None and (self.few_rows_take(rows, n, k)
                                                or self._qkv_pieces_plan(rows, n, k) is not None):
            return True
        return (n is not None and k is not None
                and self._core.llmlab_linear_tile(rows, n, k, self.num_cus) % head_dim == 0)

    def _qkv_pieces_plan(self, rows: int, n: int, k: int):
        """``(pieces, tile)`` if q/k/v of these sizes goes through pieces along the inner size
        (then any head size does: the second kernel rotates whole rows), else None."""
        if not (self.rules.qkv_pieces_min_rows <= rows <= self.QKV_PIECES_MAX_ROWS and self.pieces_by_tiles(rows, n, k)):
            return None
        if rows > self.FEW_ROWS and self.few_rows_take(rows, n, k):
            return None
        pieces, tile = self._linear_plan(rows, n, k)
        if rows > self.FEW_ROWS and k >= 2 * 64 * self.rules.min_tiles_per_split:
            # (65 to 384 rows: two pieces at least.  4608 x 3584 at 192 / 256 rows: 24 / 31 us
            # against 33 / 39 whole; 2560 x 2048: 15 / 18.5 against 20.5; the estimate of
            # the plan, made for products that add into the stream, says one)
            pieces = max(pieces, 2)
        if self.rules.forced_tiled_pieces:
            pieces = max(1, min(self.rules.forced_tiled_pieces, (k + 63) // 64, self.MAX_SPLITS))
        if pieces > 1 and pieces * rows * n <= self.workspace.numel():
            return pieces, tile
        return None

    def qkv_rope_cache(self, h, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions,
                       row_req, block_table, page_size, k_cache, v_cache, q_out) -> None:
        """The same for activations ``h`` (bfloat16, already normed): product, bias, rotation
        and cache write in one kernel."""
        rows, k = h.shape
        self._need(h, "activations", torch.bfloat16)
        w_qkv = self._weight(w_qkv, "weight")
        n = w_qkv.shape[0]
        if w_qkv.shape[1] != k or k % 8 != 0 or not self.can_fuse_qkv_rope(rows, h.dtype, head_dim, n, k):
            raise ValueError(f"qkv_rope_cache: {rows} rows of {k}, heads of {head_dim} do not fit")
        self._qkv_checks("qkv_rope_cache", rows, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim,
                         inv_freq, positions, row_req, block_table, page_size, k_cache, v_cache, q_out)
        plan = self._qkv_pieces_plan(rows, n, k)
        if plan is not None:
            # some rows of a large matrix: a head per block leaves most of the chip idle, so
            # the product is cut along K by the tiled kernel and a second kernel sums the
            # pieces, rotates and writes the cache (64 rows of 7168 x 5120: 26 us against 52
            # in one kernel, of 4608 x 3584: 19 against 24; the same at 24 rows, slower below)
            pieces, tile = plan
            if b_qkv is not None:
                self._need(b_qkv, "bias")
            parts = self.workspace[:pieces * rows * n].view(pieces, rows, n)
            self._call(self._core.llmlab_linear_partials,
                self._ptr(h), self._ptr(w_qkv), self._ptr(parts), None, 0, rows, n, k, n, pieces,
                rows * n, tile, self._stream())
            self._call(self._core.llmlab_qkv_from_pieces,
                self._ptr(parts), pieces, rows * n, n, self._ptr(b_qkv),
                _dt(b_qkv) if b_qkv is not None else 0, rows, num_heads, num_kv_heads, head_dim,
                self._ptr(inv_freq), self._ptr(positions), self._ptr(row_req), self._ptr(block_table),
                block_table.stride(0) if block_table is not None else 0, int(page_size),
                self._ptr(k_cache), self._ptr(v_cache), self._ptr(q_out), q_out.stride(0), self._stream())
            return
        if rows <= self.QKV_ROPE_MAX_ROWS or self.few_rows_take(rows, n, k):
            self._skinny(h, False, None, None, 0.0, w_qkv, b_qkv, EPI_QKV, q_out, rows, n, k,
                         q_out.shape[1], n,
                         dict(inv_freq=inv_freq, positions=positions, row_req=row_req, table=block_table,
                              page_size=page_size, k_cache=k_cache, v_cache=v_cache, nq=num_heads,
                              nkv=num_kv_heads, d=head_dim))
            return
        if b_qkv is not None:
            self._need(b_qkv, "bias")
        self._call(self._core.llmlab_linear_qkv,
            self._ptr(h), self._ptr(w_qkv), self._ptr(b_qkv), _dt(b_qkv) if b_qkv is not None else 0,
            self._ptr(q_out), rows, n, k, q_out.stride(0), self._ptr(inv_freq), self._ptr(positions),
            self._ptr(row_req), self._ptr(block_table), block_table.stride(0) if block_table is not None else 0,
            int(page_size), self._ptr(k_cache), self._ptr(v_cache), num_heads, num_kv_heads, head_dim,
            self.num_cus, self._stream())

    def fused_norm_swiglu(self, x, norm_w, eps, w_gate_up, out, pending: Optional[PendingSums] = None) -> None:
        rows, inter = out.shape
        w_gate_up, k = self._fused_common(x, norm_w, w_gate_up, rows)
        self._need(out, "SwiGLU output", torch.bfloat16)
        if x.shape[0] != rows or w_gate_up.shape[0] != 2 * ((inter + 15) // 16 * 16):
            raise ValueError("fused_norm_swiglu: shapes do not fit")
        self._skinny(x, True, None, norm_w, eps, w_gate_up, None, EPI_SWIGLU, out, rows,
                     w_gate_up.shape[0], k, out.shape[1], inter, pending=pending)

    def fused_norm_logits(self, x, rows_index, norm_w, eps, w, out, pending: Optional[PendingSums] = None) -> None:
        """out[i] = norm(x[rows_index[i]]) W^T in float32."""
        rows, vocab = out.shape
        w, k = self._fused_common(x, norm_w, w, rows)
        self._need(out, "logits", torch.float32)
        if w.shape[0] != vocab:
            raise ValueError("fused_norm_logits: weight rows differ from the vocabulary")
        if rows_index is not None:
            self._need(rows_index, "row indices", torch.int32)
            if rows_index.numel() < rows:
                raise ValueError("fused_norm_logits: one row index per output row")
        elif x.shape[0] != rows:
            raise ValueError("fused_norm_logits: rows differ")
        self._skinny(x, True, rows_index, norm_w, eps, w, None, EPI_F32, out, rows, vocab, k,
                     out.shape[1], vocab, pending=pending)

    # ------------------------------------------------------------------- rope
    def rope_inplace(self, x, positions, inv_freq) -> None:
        rows, heads, d = x.shape
        if x.stride(2) != 1:
            raise ValueError("rope: the head dimension must be contiguous")
        self._need(positions, "positions", torch.int32)
        self._need(inv_freq, "rotary frequencies", torch.float32)
        if inv_freq.numel() != d // 2 or positions.numel() < rows:
            raise ValueError("rope: frequency table or positions do not fit")
        self._call(self._core.llmlab_rope_inplace,
            self._ptr(x), _dt(x), rows, heads, d, x.stride(0), x.stride(1), self._ptr(inv_freq),
            self._ptr(positions), self._stream())

    def rope_kv_write(self, qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions, row_req,
                      block_table, page_size, k_cache, v_cache) -> None:
        self._need(qkv, "qkv", contiguous=False)
        rows = qkv.shape[0]
        if qkv.stride(1) != 1 or qkv.shape[1] != (num_heads + 2 * num_kv_heads) * head_dim:
            raise ValueError(f"rope_kv_write: qkv {tuple(qkv.shape)} does not hold {num_heads}+2*"
                             f"{num_kv_heads} heads of {head_dim}")
        self._need(positions, "positions", torch.int32)
        if positions.numel() < rows:
            raise ValueError("rope_kv_write: one position per row")
        if inv_freq is not None:
            self._need(inv_freq, "rotary frequencies", torch.float32)
            if inv_freq.numel() != head_dim // 2:
                raise ValueError("rope_kv_write: the frequency table must hold head_dim/2 entries")
        table_stride = 0
        if k_cache is not None:
            self._need(row_req, "row -> request map", torch.int32)
            self._need(block_table, "block table", torch.int32)
            if row_req.numel() < rows:
                raise ValueError("rope_kv_write: one request index per row")
            pages = k_cache.shape[0]
            if (tuple(k_cache.shape) != (pages, num_kv_heads, page_size, head_dim)
                    or tuple(v_cache.shape) != (pages, num_kv_heads, head_dim, page_size)
                    or not k_cache.is_contiguous() or not v_cache.is_contiguous()
                    or k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype):
                raise ValueError("rope_kv_write: cache tensors do not have the paged layout")
            table_stride = block_table.stride(0)
        self._call(self._core.llmlab_rope_kv_write,
            self._ptr(qkv), _dt(qkv), rows, qkv.stride(0) if rows > 1 else qkv.shape[1], num_heads,
            num_kv_heads, head_dim, self._ptr(inv_freq), self._ptr(positions), self._ptr(row_req),
            self._ptr(block_table), table_stride, page_size, self._ptr(k_cache), self._ptr(v_cache),
            self._stream())

    # -------------------------------------------------------------- attention
    def attention_short_limit(self, num_heads: int, num_kv_heads: int, dtype, max_q_len: int) -> int:
        """A mixed step (portions of prompts beside decoding requests) is served by two
        launches: its requests of a few tokens go to the one that splits their keys over
        the chip, the portions to the tiled one.  Returns the most tokens a request may
        bring to count as short in such a step, or 0 if the step is not divided."""
        group = num_heads // num_kv_heads
        if group <= 16 < max_q_len * group:
            return 16 // group
        return 0

    def paged_attention(self, qkv, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_table,
                        page_size, q_start, start_pos, n_reqs, max_q_len, max_ctx_len, window, scale,
                        out, short=None) -> None:
        """``short``: ``(row_req, limit, count, longest)`` for a step in which ``count`` of the
        requests (not all) bring at most ``limit = attention_short_limit(...)`` tokens, the
        longest context among those being ``longest``."""
        self.prepare_attention(qkv, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_table, page_size,
                               q_start, start_pos, window, scale, out,
                               short[0] if short is not None else None).launch(n_reqs, max_q_len, max_ctx_len, short)

    def prepare_attention(self, qkv, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_table,
                          page_size, q_start, start_pos, window, scale, out, row_req=None) -> "AttentionCall":
        """Everything of an attention call that does not change while the same buffers serve
        the same number of rows, checked and laid out once; ``launch`` then takes what a step
        brings (how many requests, their longest portion and context, its short requests).
        ``q_start`` and ``start_pos`` may be longer than a step's requests; ``row_req`` is
        needed only if a step will name short requests."""
        lib = self._attention_lib(head_dim)
        rows = qkv.shape[0]
        self._need(qkv, "queries", contiguous=False)
        self._need(out, "attention output")
        self._need(block_table, "block table", torch.int32)
        self._need(q_start, "request row starts", torch.int32)
        self._need(start_pos, "request start positions", torch.int32)
        pages = k_cache.shape[0]
        if (tuple(k_cache.shape) != (pages, num_kv_heads, page_size, head_dim)
                or tuple(v_cache.shape) != (pages, num_kv_heads, head_dim, page_size)
                or not k_cache.is_contiguous() or not v_cache.is_contiguous()):
            raise ValueError("attention: cache tensors do not have the paged layout")
        if not (qkv.dtype == out.dtype == k_cache.dtype == v_cache.dtype):
            raise TypeError("attention: queries, cache and output must share one dtype")
        if qkv.stride(1) != 1 or qkv.shape[1] < num_heads * head_dim:
            raise ValueError("attention: the query rows are too narrow")
        if tuple(out.shape) != (rows, num_heads * head_dim):
            raise ValueError(f"attention: output {tuple(out.shape)} != ({rows}, {num_heads * head_dim})")
        if page_size < 16 or page_size & (page_size - 1):
            raise UnsupportedSizeError(f"page size {page_size} is not a power of two >= 16")
        if row_req is not None:
            self._need(row_req, "row -> request map", torch.int32)
            if row_req.numel() < rows:
                raise ValueError("attention: one request index per row")
        q_stride = qkv.stride(0) if rows > 1 else qkv.shape[1]
        args = [self._ptr(qkv), _dt(qkv), q_stride, num_heads, num_kv_heads, self._ptr(k_cache),
                self._ptr(v_cache), self._ptr(block_table), block_table.stride(0), page_size,
                self._ptr(q_start), self._ptr(start_pos), 0, 0, 0,
                int(window) if window else 0, float(scale), self._ptr(out), out.stride(0) if rows > 1 else
                out.shape[1], self._ptr(self.workspace), self.workspace.numel(), rows, self.num_cus,
                None, 0, 0, 0, self._ptr(self.arrived), self.arrived.numel(), None]
        return AttentionCall(self, lib, args, most_requests=min(q_start.numel() - 1, start_pos.numel(), block_table.shape[0]),
                             most_context=block_table.shape[1] * page_size, row_req=self._ptr(row_req),
                             heads=(num_heads, num_kv_heads), dtype=qkv.dtype)

    # --------------------------------------------------------------- sampling
    def argmax(self, logits, out, one_pass: bool = True) -> None:
        """``out[r]`` = the largest logit's index (the smallest among equals; -1 for a row
        without a finite value).  ``one_pass=False``: in two kernels, without the counters."""
        self._need(logits, "logits", torch.float32, contiguous=False)
        self._need(out, "chosen tokens", torch.int32)
        rows, vocab = logits.shape
        if logits.stride(1) != 1 or out.numel() < rows:
            raise ValueError("argmax: logits rows must be contiguous and out must hold one token per row")
        self._call(self._core.llmlab_argmax,
            self._ptr(logits), logits.stride(0) if rows > 1 else vocab, rows, vocab, self._ptr(out),
            self._ptr(self.workspace), self.workspace.numel(),
            self._ptr(self.arrived) if one_pass else None, self.arrived.numel(), self._stream())

    def sample(self, logits, temperatures, uniforms, out) -> None:
        self._need(logits, "logits", torch.float32, contiguous=False)
        self._need(out, "chosen tokens", torch.int32)
        rows, vocab = logits.shape
        if logits.stride(1) != 1 or out.numel() < rows:
            raise ValueError("sample: logits rows must be contiguous and out must hold one token per row")
        if temperatures is not None:
            self._need(temperatures, "temperatures", torch.float32)
            self._need(uniforms, "uniform numbers", torch.float32)
            if temperatures.numel() < rows or uniforms.numel() < rows:
                raise ValueError("sample: one temperature and one uniform number per row")
        self._call(self._core.llmlab_sample,
            self._ptr(logits), logits.stride(0) if rows > 1 else vocab, rows, vocab,
            self._ptr(temperatures), self._ptr(uniforms), self._ptr(out), self._stream())
