"""Token selection on the GPU with host-side, counter-based random numbers.

The n-th token of a request is drawn with the uniform number ``u(seed, n)``, a
pure function of the request's seed and n.  The choice therefore does not depend
on which other requests shared the step, on how the prompt was cut, or on the
order of the batch.  The kernel takes the argmax where the temperature is 0 and
otherwise the smallest token whose cumulative probability under
``softmax(logits / temperature)`` reaches ``u``.  The reference selects with a
two-stage argmax only (rust/engine/src/runner/model/qwen2/kernels.rs:1488-1552).
"""
from __future__ import annotations

from typing import List, Sequence

import numpy as np
import torch

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform(seed: int, n: int) -> float:
    """The n-th uniform number in [0, 1) of the stream ``seed`` (24 bits, exact in float32)."""
    z = _splitmix64(_splitmix64(int(seed) & _MASK) ^ ((int(n) * 0xD1342543DE82EF95) & _MASK))
    return (z >> 40) / float(1 << 24)


class PendingTokens:
    """Tokens chosen on the GPU whose copy to the host may still be under way."""

    def __init__(self, device_tokens: torch.Tensor, host_tokens: torch.Tensor, event, rows: int):
        self.device_tokens = device_tokens      # int32 [rows] on the GPU: the next step may read it there
        self._host = host_tokens
        self._event = event
        self.rows = rows

    def tokens(self) -> List[int]:
        """Wait for the copy.  A row that held no finite logit gives -1."""
        if self._event is not None:
            self._event.synchronize()
        return self._host[:self.rows].tolist()

    def result(self) -> List[int]:
        """Wait for the copy; raises if a row held no finite logit."""
        tokens = self.tokens()
        for t in tokens:
            if t < 0:
                raise FloatingPointError("non-finite logits: no token can be chosen")
        return tokens


class Sampler:
    SLOTS = 2     # results of two steps can be alive: the one being read and the one in flight

    def __init__(self, ops, max_requests: int):
        self.ops = ops
        self.device = ops.device
        self._cuda = torch.device(self.device).type == "cuda"
        # Every slot has its own staging of the inputs (temperatures, uniform numbers) as
        # well as of the outputs: with one step of lookahead the host fills the next
        # step's numbers while the copy of this step's may not have run yet.
        self._host = [torch.zeros((2, max_requests), dtype=torch.float32, pin_memory=self._cuda)
                      for _ in range(self.SLOTS)]
        self._dev = [torch.zeros((2, max_requests), dtype=torch.float32, device=self.device)
                     for _ in range(self.SLOTS)]
        self._out = [torch.zeros(max_requests, dtype=torch.int32, device=self.device)
                     for _ in range(self.SLOTS)]
        self._out_host = [torch.zeros(max_requests, dtype=torch.int32, pin_memory=self._cuda)
                          for _ in range(self.SLOTS)]
        self._done = [None] * self.SLOTS      # recorded after a slot's last copy to the host
        self._views = {}
        self._slot = 0

    def sample_async(self, logits: torch.Tensor, temperatures: Sequence[float], seeds: Sequence[int],
                     counters: Sequence[int]) -> PendingTokens:
        """Choose one token per row of ``logits``; the tokens stay on the GPU and a copy
        to the host is started.  The buffers are reused after ``SLOTS`` further calls."""
        rows = logits.shape[0]
        self._slot = (self._slot + 1) % self.SLOTS
        slot = self._slot
        out, out_host = self._out[slot], self._out_host[slot]
        views = self._views.get((slot, rows))       # (slices of the slot's buffers: made once per batch size)
        if views is None:
            views = self._views[(slot, rows)] = (out[:rows], out_host[:rows])
        out_rows, out_host_rows = views
        if self._done[slot] is not None:
            # everything queued with this slot's buffers has run: they are free again
            self._done[slot].synchronize()
        if all(t <= 0.0 for t in temperatures):
            self.ops.argmax(logits, out_rows)
        else:
            host, dev = self._host[slot], self._dev[slot]
            h = host.numpy()
            h[0, :rows] = np.asarray(temperatures, dtype=np.float32)
            h[1, :rows] = np.asarray([uniform(s, c) for s, c in zip(seeds, counters)], dtype=np.float32)
            dev[:, :rows].copy_(host[:, :rows], non_blocking=True)
            self.ops.sample(logits, dev[0, :rows], dev[1, :rows], out_rows)
        event = None
        if self._cuda:
            out_host_rows.copy_(out_rows, non_blocking=True)
            event = self._done[slot] or torch.cuda.Event()        # (the slot's event, recorded anew)
            event.record()
            self._done[slot] = event
        else:
            out_host_rows.copy_(out_rows)
        return PendingTokens(out, out_host, event, rows)

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], seeds: Sequence[int],
               counters: Sequence[int]) -> List[int]:
        """One token per row of ``logits``.  Raises if a row holds no finite value."""
        return self.sample_async(logits, temperatures, seeds, counters).result()
