"""Plain PyTorch references of the kernel set, op by op, on the engine's own
buffers and layouts (paged cache, block tables, interleaved gate/up rows).

Two uses: the GPU tests compare each HIP kernel with the function of the same
name here, and the CPU tests plug this object into the engine in place of the
HIP kernels to exercise the cache manager, the step function and the scheduler
without a GPU.  It is test code, not a fallback: the product never loads it.
All arithmetic is float32 whatever the storage dtype.
"""
from __future__ import annotations

import math

import torch

from llm_inference_lab_amd.cache import layout as cache_layout
from llm_inference_lab_amd.parts import PendingSums


class EmuRecord:
    """The calls a part made while it was recorded (the counterpart of the product's
    ``LaunchRecord``): ``(bound method, (args, kwargs), None)`` or ``(None, closure, None)``."""

    def __init__(self, dry=False):
        self.calls = []
        self.dry = dry

    @staticmethod
    def _same(a, b):
        if isinstance(a, torch.Tensor) or isinstance(b, torch.Tensor):
            return (isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor) and a.data_ptr() == b.data_ptr()
                    and a.shape == b.shape and a.stride() == b.stride() and a.dtype == b.dtype)
        if isinstance(a, PendingSums) or isinstance(b, PendingSums):
            return (isinstance(a, PendingSums) and isinstance(b, PendingSums) and a.splits == b.splits
                    and EmuRecord._same(a.parts, b.parts))
        return a == b

    def same_as(self, other):
        if len(self.calls) != len(other.calls):
            return False
        for (fa, aa, _), (fb, ab, _) in zip(self.calls, other.calls):
            if (fa is None) != (fb is None):
                return False
            if fa is None:
                continue
            if fa is not fb or len(aa[0]) != len(ab[0]) or sorted(aa[1]) != sorted(ab[1]):
                return False
            if not all(self._same(x, y) for x, y in zip(aa[0], ab[0])):
                return False
            if not all(self._same(aa[1][k], ab[1][k]) for k in aa[1]):
                return False
        return True


class EmuOps:
    # the operations that do work on tensors: written down while a part is recorded, as the
    # product's kernel set writes down its calls into the kernel libraries
    RECORDED = ("embed", "gather_tokens", "rmsnorm", "linear", "linear_residual", "linear_partials",
                "add_pending", "linear_logits", "linear_swiglu", "fused_norm_qkv", "qkv_rope_cache",
                "fused_norm_swiglu", "fused_norm_logits", "rope_inplace", "rope_kv_write",
                "paged_attention", "argmax", "sample")

    def __init__(self, device="cpu", fuse=True):
        self.device = torch.device(device)
        self.calls = {}
        self.fuse = fuse
        import types
        self.rules = types.SimpleNamespace(min_steps_per_split=8)
        self._record = None
        self._depth = 0
        for name in self.RECORDED:
            setattr(self, name, self._recordable(getattr(self, name)))

    # ----------------------------------------------- recorded sequences of calls
    def _recordable(self, method):
        def call(*args, **kwargs):
            record = self._record
            if record is not None and self._depth == 0:      # (an operation's own inner calls are its business)
                record.calls.append((call, (args, kwargs), None))
                if record.dry:      # (nothing is computed; what the caller is handed back all the same)
                    return PendingSums(args[2], args[3]) if method.__name__ == "linear_partials" else None
            self._depth += 1
            try:
                return method(*args, **kwargs)
            finally:
                self._depth -= 1
        call.inner = method
        return call

    def begin_recording(self, dry=False):
        assert self._record is None
        self._record = EmuRecord(dry)
        return self._record

    def end_recording(self):
        record, self._record = self._record, None
        return record

    def live(self, launch):
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

    def replay(self, record):
        for fn, args, _ in record.calls:
            if fn is None:
                args()
            else:
                fn.inner(*args[0], **args[1])

    def fingerprint(self):
        plain = (int, float, str, bool, type(None))
        rules = tuple(sorted((k, v if isinstance(v, plain) else id(v)) for k, v in vars(self.rules).items()))
        return (self.fuse, rules, getattr(self, "num_cus", 0))

    def _count(self, name):
        self.calls[name] = self.calls.get(name, 0) + 1

    @property
    def calls_made(self):
        """Calls so far, as the kernel set of the product counts them."""
        return sum(self.calls.values())

    def check_attention_sizes(self, num_heads, num_kv_heads, head_dim, dtype):
        pass

    def check_product_sizes(self, inner, dtype, what):
        pass

    def synchronize(self):
        pass

    # ------------------------------------------------------------ elementwise
    def embed(self, table, ids, out):
        self._count("embed")
        out.copy_(table[ids.long()].float())

    def gather_tokens(self, dst, dst_index, src, src_index, n):
        self._count("gather_tokens")
        for i in range(n):
            dst[int(dst_index[i])] = src[int(src_index[i])]

    def rmsnorm(self, x, weight, eps, out, rows=None, pending=None):
        self._count("rmsnorm")
        if pending is not None:
            assert rows is None and pending.parts.shape[1:] == x.shape
            x += pending.parts[:pending.splits].float().sum(0)
        v = x.float() if rows is None else x.float()[rows.long()]
        inv = torch.rsqrt((v * v).sum(-1, keepdim=True) / v.shape[-1] + eps)
        out.copy_((v * inv * weight.float()).to(out.dtype))

    # ----------------------------------------------------------------- linear
    def linear(self, x, w, out, bias=None):
        self._count("linear")
        y = x.float() @ w.float().t()
        if bias is not None:
            y = y + bias.float()
        out.copy_(y.to(out.dtype))

    def linear_residual(self, x, w, resid, bias=None, pending=None):
        self._count("linear_residual")
        y = x.float() @ w.float().t()
        if bias is not None:
            y = y + bias.float()
        if pending is not None:
            resid.add_(self._owed(pending))
        resid.add_(y)

    # ---------------------------------------------------- sums left in pieces
    MAX_SPLITS = 8
    num_cus = 256

    @staticmethod
    def _owed(pending):
        return pending.parts[:pending.splits].sum(0) if pending is not None else 0.0

    def split_count(self, rows, dtype, n, k):
        if not self.fuse or dtype != torch.bfloat16 or not 0 < rows <= 64:
            return 1
        strips, steps = (n + 15) // 16, (k + 31) // 32
        return max(1, min(self.num_cus // max(strips, 1), steps // self.rules.min_steps_per_split, self.MAX_SPLITS))

    def linear_partials(self, x, w, parts, splits, bias=None):
        """Piece s covers the K steps from s * ceil(steps / splits) on; a step is 32 wide
        for up to 64 rows and 64 wide for more (the two kernels' K tiles)."""
        self._count("linear_partials")
        k = x.shape[1]
        width = 32 if x.shape[0] <= 64 else 64
        steps = (k + width - 1) // width
        per = (steps + splits - 1) // splits
        for s in range(splits):
            lo, hi = min(k, s * per * width), min(k, (s + 1) * per * width)
            parts[s] = x[:, lo:hi].float() @ w[:, lo:hi].float().t()
        if bias is not None:
            parts[0] += bias.float()
        return PendingSums(parts, splits)

    def add_pending(self, x, pending):
        self._count("add_pending")
        x.add_(self._owed(pending))

    def linear_logits(self, x, w, out):
        self._count("linear_logits")
        out.copy_(x.float() @ w.float().t())

    def linear_swiglu(self, x, w_gu, out):
        """w_gu rows alternate in runs of 16: gate rows of 16 outputs, then the
        up rows of the same outputs."""
        self._count("linear_swiglu")
        inter = out.shape[1]
        y = x.float() @ w_gu.float().t()                       # [M, 2*Ipad]
        y = y.view(x.shape[0], -1, 2, 16)
        gate = y[:, :, 0, :].reshape(x.shape[0], -1)[:, :inter]
        up = y[:, :, 1, :].reshape(x.shape[0], -1)[:, :inter]
        out.copy_((gate / (1.0 + torch.exp(-gate)) * up).to(out.dtype))

    # ------------------------------------------------- fused few-row kernels
    FUSED_MAX_ROWS = 64
    fuse_max_rows = 16

    def pieces_too_large_to_read_per_block(self, pending):
        return False

    def pieces_by_tiles(self, rows, n, k):
        return False

    def can_fuse(self, rows, dtype, inner, outer=None):
        return self.fuse and dtype == torch.bfloat16 and 0 < rows <= self.fuse_max_rows

    def prepare_weight(self, w, shared=False):
        return w

    def release_shared(self):
        pass

    def _normed(self, x, rows_index, norm_w, eps, n, pending=None):
        v = x.float() + self._owed(pending)
        v = v if rows_index is None else v[rows_index[:n].long()]
        inv = torch.rsqrt((v * v).sum(-1, keepdim=True) / v.shape[-1] + eps)
        # the kernel rounds x * w to bfloat16 and scales by inv_rms afterwards
        return (v * norm_w.float()).to(torch.bfloat16).float() * inv

    def fused_norm_qkv(self, x, norm_w, eps, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim, inv_freq,
                       positions, row_req, block_table, page_size, k_cache, v_cache, q_out, pending=None):
        self._count("fused_norm_qkv")
        rows = x.shape[0]
        y = self._normed(x, None, norm_w, eps, rows, pending) @ w_qkv.float().t()
        if b_qkv is not None:
            y = y + b_qkv.float()
        qkv = y.clone()                      # float32: the kernel rotates before it rounds
        self.rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions, row_req,
                           block_table, page_size, k_cache, v_cache)
        q_out.copy_(qkv[:, :num_heads * head_dim].to(q_out.dtype))

    def can_fuse_qkv_rope(self, rows, dtype, head_dim, n=None, k=None):
        return self.fuse and dtype == torch.bfloat16 and rows > 0 and head_dim % 16 == 0 and (
            rows <= 64 or (n is not None and 64 % head_dim == 0))

    def qkv_rope_cache(self, h, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions,
                       row_req, block_table, page_size, k_cache, v_cache, q_out):
        self._count("qkv_rope_cache")
        y = h.float() @ w_qkv.float().t()
        if b_qkv is not None:
            y = y + b_qkv.float()
        qkv = y.clone()                      # float32: the kernel rotates before it rounds
        self.rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions, row_req,
                           block_table, page_size, k_cache, v_cache)
        q_out.copy_(qkv[:, :num_heads * head_dim].to(q_out.dtype))

    def fused_norm_swiglu(self, x, norm_w, eps, w_gate_up, out, pending=None):
        self._count("fused_norm_swiglu")
        h = self._normed(x, None, norm_w, eps, x.shape[0], pending)
        self.linear_swiglu(h, w_gate_up, out)

    def fused_norm_logits(self, x, rows_index, norm_w, eps, w, out, pending=None):
        self._count("fused_norm_logits")
        out.copy_(self._normed(x, rows_index, norm_w, eps, out.shape[0], pending) @ w.float().t())

    # ------------------------------------------------------------------- rope
    @staticmethod
    def _rotate(x, positions, inv_freq):
        # x [rows, heads, d] float32
        half = x.shape[-1] // 2
        ang = positions.float()[:, None] * inv_freq.float()[None, :]
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        lo, hi = x[..., :half], x[..., half:]
        return torch.cat([lo * c - hi * s, hi * c + lo * s], dim=-1)

    def rope_inplace(self, x, positions, inv_freq):
        self._count("rope_inplace")
        x.copy_(self._rotate(x.float(), positions, inv_freq).to(x.dtype))

    def rope_kv_write(self, qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions, row_req,
                      block_table, page_size, k_cache, v_cache):
        self._count("rope_kv_write")
        rows = qkv.shape[0]
        qs, ks = num_heads * head_dim, num_kv_heads * head_dim
        q = qkv[:, :qs].float().view(rows, num_heads, head_dim)
        k = qkv[:, qs:qs + ks].float().view(rows, num_kv_heads, head_dim)
        v = qkv[:, qs + ks:].float().view(rows, num_kv_heads, head_dim)
        if inv_freq is not None:
            q = self._rotate(q, positions[:rows], inv_freq)
            k = self._rotate(k, positions[:rows], inv_freq)
            qkv[:, :qs] = q.reshape(rows, qs).to(qkv.dtype)
        if k_cache is None:
            return
        for r in range(rows):
            p = int(positions[r])
            page = int(block_table[int(row_req[r]), p // page_size])
            assert page >= 0, "write to a position without a page"
            off = p % page_size
            # the numbers of a page lie in the kernels' fragment order
            kflat = k_cache.view(k_cache.shape[0], num_kv_heads, -1)
            vflat = v_cache.view(v_cache.shape[0], num_kv_heads, -1)
            kflat[page][:, cache_layout.key_index(page_size, head_dim)[off]] = k[r].to(k_cache.dtype)
            vflat[page][:, cache_layout.value_index(page_size, head_dim)[:, off]] = v[r].to(v_cache.dtype)

    # -------------------------------------------------------------- attention
    def attention_short_limit(self, num_heads, num_kv_heads, dtype, max_q_len):
        return 0

    def paged_attention(self, qkv, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_table,
                        page_size, q_start, start_pos, n_reqs, max_q_len, max_ctx_len, window, scale,
                        out, short=None):
        self._count("paged_attention")
        group = num_heads // num_kv_heads
        qs = num_heads * head_dim
        for b in range(n_reqs):
            r0, r1 = int(q_start[b]), int(q_start[b + 1])
            sp = int(start_pos[b])
            end = sp + (r1 - r0)
            # the request's positions, read through its block table (a freed or
            # missing page reads as NaN, so a wrong access shows in the result)
            keys = torch.full((end, num_kv_heads, head_dim), float("nan"))
            vals = torch.full((end, num_kv_heads, head_dim), float("nan"))
            kidx = cache_layout.key_index(page_size, head_dim)
            vidx = cache_layout.value_index(page_size, head_dim)
            kflat = k_cache.view(k_cache.shape[0], num_kv_heads, -1)
            vflat = v_cache.view(v_cache.shape[0], num_kv_heads, -1)
            for j in range(end):
                pg = int(block_table[b, j // page_size])
                if pg >= 0:
                    keys[j] = kflat[pg][:, kidx[j % page_size]].float()
                    vals[j] = vflat[pg][:, vidx[:, j % page_size]].float()
            for r in range(r0, r1):
                p = sp + (r - r0)
                lo = 0 if window is None else max(0, p - window + 1)
                q = qkv[r, :qs].float().view(num_heads, head_dim)
                for h in range(num_heads):
                    kvh = h // group
                    s = (keys[lo:p + 1, kvh] @ q[h]) * scale
                    pr = torch.softmax(s, dim=0)
                    out[r, h * head_dim:(h + 1) * head_dim] = (pr @ vals[lo:p + 1, kvh]).to(out.dtype)

    # --------------------------------------------------------------- sampling
    def argmax(self, logits, out):
        self._count("argmax")
        for b in range(logits.shape[0]):
            row = logits[b]
            if torch.isnan(row).all():
                out[b] = -1
                continue
            row = torch.where(torch.isnan(row), torch.full_like(row, float("-inf")), row)
            m = row.max()
            out[b] = int((row == m).nonzero()[0, 0])

    def sample(self, logits, temperatures, uniforms, out):
        """temperature <= 0: argmax.  Else the smallest index whose cumulative
        probability under softmax(logits / t) reaches u * total."""
        self._count("sample")
        for b in range(logits.shape[0]):
            t = float(temperatures[b])
            if t <= 0.0:
                self.argmax(logits[b:b + 1], out[b:b + 1])
                continue
            z = logits[b].double() / t
            e = torch.exp(z - z.max())
            target = float(uniforms[b]) * float(e.sum())
            cum = torch.cumsum(e, dim=0)
            idx = int(torch.searchsorted(cum, torch.tensor(target, dtype=torch.float64)))
            out[b] = min(idx, logits.shape[1] - 1)
