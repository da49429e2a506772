"""The engine: a model folder (or a configuration and a seed) becomes a model
bound to kernels, a cache manager and a step function.

Option names follow the reference's command line where it has them
(rust/engine/examples/qwen2.rs:38-73): ``dtype`` ("bf16" or "f32": weights,
activations and cache storage; reductions stay in 32 bits), ``model_dir``,
``max_batch_tokens`` (most uncached input tokens per step, shared by decode and
prefill, default 512).
"""
from __future__ import annotations

import os
import tempfile
from typing import Callable, Dict, List, Optional, Sequence

import torch

from .. import architectures  # noqa: F401  (registers the known architectures)
from ..cache.manager import CacheManager, GroupLayout, RequestCache, pages_for_tokens
from ..config.errors import ConfigError
from ..config.registry import get_architecture, read_config
from ..weights.loader import load_tensors, place_tensors
from ..weights.random_init import random_tensors, write_model_dir
from .model import CausalLM
from .step import StepEntry, StepFunction

_DTYPES = {
    "bf16": torch.bfloat16, "bfloat16": torch.bfloat16,
    "f32": torch.float32, "fp32": torch.float32, "float32": torch.float32,
}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ConfigError(f"dtype must be bfloat16 or float32, got {name}")
        return name
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise ConfigError(f"dtype must be one of {sorted(_DTYPES)}, got {name!r}") from None


def default_ops(device):
    """The HIP kernel set.  There is no other: without a GPU or without the
    compiled extension this raises."""
    from ..kernels.hip_ops import HipOps
    return HipOps(device)


class Engine:
    """Model + cache + step function on one GPU."""

    def __init__(self, model_dir: Optional[str] = None, *, config=None, seed: int = 0,
                 dtype="bf16", device: str = "cuda:0", ops=None, page_size: int = 64,
                 max_cache_tokens: Optional[int] = None, num_pages: Optional[int] = None,
                 max_requests: int = 64, max_batch_tokens: int = 512,
                 max_seq_len: Optional[int] = None, tensors=None, graph=False,
                 progress: Optional[Callable[[str], None]] = None):
        self.dtype = parse_dtype(dtype)
        if model_dir is not None:
            self.architecture, self.config = read_config(model_dir)
        elif config is not None:
            arch_name = getattr(config, "architecture", None) or getattr(config, "ARCHITECTURE")
            self.architecture, self.config = get_architecture(arch_name), config
        else:
            raise ValueError("give a model_dir or a config")
        self.spec = self.architecture.build_spec(self.config)
        if ops is None:
            # compile what this model needs before the GPU is first touched
            from ..kernels import build
            build.core_library()
            for dim in sorted({b.mixer.params["head_dim"] for b in self.spec.blocks
                               if "head_dim" in b.mixer.params}):
                build.attention_library(int(dim))
        self.ops = ops if ops is not None else default_ops(device)
        self.device = self.ops.device
        self.model = CausalLM(self.spec)
        expected = self.model.tensor_specs()
        if model_dir is not None:
            loaded = load_tensors(model_dir, expected, self.dtype, self.device, progress)
        elif tensors is not None:
            loaded = place_tensors(tensors, expected, self.dtype, self.device)
        else:
            loaded = place_tensors(random_tensors(expected, seed, torch.bfloat16), expected,
                                   self.dtype, self.device, "random weights")
        self.model.bind(loaded, self.ops, self.dtype)
        del loaded
        # ------------------------------------------------------------- cache
        self.page_size = int(page_size)
        self.max_requests = int(max_requests)
        self.max_batch_tokens = int(max_batch_tokens)
        self.max_seq_len = int(max_seq_len or self.spec.max_positions)
        self.max_seq_len = min(self.max_seq_len, self.spec.max_positions)
        groups, state_specs = self.model.cache_layout()
        if num_pages is None:
            tokens = max_cache_tokens if max_cache_tokens is not None else \
                self.max_requests * self.max_seq_len
            num_pages = pages_for_tokens(int(tokens), self.page_size)
            if max_cache_tokens is None:
                # nobody asked for a size: every request at full length, or what the
                # memory that the weights left free can hold, whichever is less
                num_pages = min(num_pages, self._pages_that_fit(groups))
        for g in groups:
            g.num_pages = int(num_pages)
        self.cache = CacheManager(groups, self.page_size, self.max_requests, self.max_seq_len,
                                  state_specs, self.dtype, self.device)
        self.model.attach_cache(self.cache)
        self.step_fn = StepFunction(self.model, self.cache, self.ops, self.max_batch_tokens,
                                    graph=self._graph_choice(graph))
        self._sampler = None
        self.last_scheduler = None

    CACHE_SHARE_OF_FREE_MEMORY = 0.9

    def _pages_that_fit(self, groups) -> int:
        """Pages (per group) that fit the GPU memory that is free now, leaving a tenth of
        it for scratch buffers; at least one request of full length."""
        if self.device.type != "cuda":
            return 1 << 40
        width = torch.empty((), dtype=self.dtype).element_size()
        page_bytes = sum(2 * len(g.entries) * g.spec.num_kv_heads * g.spec.head_dim * width
                         for g in groups) * self.page_size
        free, _ = torch.cuda.mem_get_info(self.device)
        fit = int(free * self.CACHE_SHARE_OF_FREE_MEMORY) // max(page_bytes, 1)
        return max(fit, pages_for_tokens(self.max_seq_len, self.page_size))

    # A decode step replayed from a HIP graph costs the host nothing, but the GPU about a
    # microsecond more at every kernel boundary than kernels launched one by one by a host
    # that runs ahead (measured: 4.05 against 3.90 ms a step at the 7B shape, 17.3 against
    # 16.9 at the 32B shape; 0.97 against 1.7 at the 0.5B shape, where the host cannot keep
    # up).  ``graph="auto"`` takes the graph unless the step's reading of the weights
    # clearly outlasts the host's launching of its kernels.
    HOST_SECONDS_PER_KERNEL = 12e-6
    STREAMED_BYTES_PER_SECOND = 4.2e12

    def _graph_choice(self, graph) -> bool:
        if graph != "auto":
            return bool(graph)
        kernels = 6 * len(self.spec.schedule) + 6
        host = kernels * self.HOST_SECONDS_PER_KERNEL
        gpu = self.model.weight_bytes_per_step() / self.STREAMED_BYTES_PER_SECOND
        return gpu < 1.25 * host

    # ------------------------------------------------------------- requests
    def open(self, request_id) -> RequestCache:
        """Give a new request a row in the cache manager."""
        return self.cache.admit(request_id)

    def close(self, request: RequestCache) -> None:
        """The request has ended: everything it holds is given back."""
        self.cache.release(request)

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        return self.step_fn(entries)

    # ------------------------------------------------------------ generation
    def scheduler(self, max_batch_tokens: Optional[int] = None, on_token=None, trace=None,
                  overlap: bool = True):
        """A scheduler over this engine (continuous batching, chunked prefill)."""
        from ..sampling.sampler import Sampler
        from .scheduler import Scheduler
        if self._sampler is None:
            self._sampler = Sampler(self.ops, self.max_requests)
        return Scheduler(self, self._sampler, max_batch_tokens or self.max_batch_tokens,
                         on_token=on_token, trace=trace, overlap=overlap)

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 8,
                 temperature: Optional[float] = None, seed: int = 0, eos_token_id=None,
                 sampling=None, max_batch_tokens: Optional[int] = None, on_token=None,
                 trace=None, overlap: bool = True) -> List[List[int]]:
        """Token ids in, generated token ids out, one list per prompt.  ``sampling``
        (one ``SamplingConfig`` or one per prompt) overrides the scalar options; the
        i-th prompt draws from the random stream ``seed + i``.  A request that the
        scheduler refuses raises its error here."""
        from ..sampling.params import SamplingConfig
        sched = self.scheduler(max_batch_tokens, on_token, trace, overlap)
        ids = []
        for i, prompt in enumerate(prompts):
            if sampling is None:
                cfg = SamplingConfig(temperature=temperature, max_new_tokens=max_new_tokens,
                                     eos_token_id=eos_token_id, seed=seed + i,
                                     do_sample=None if temperature is None else temperature > 0)
            else:
                cfg = sampling[i] if isinstance(sampling, (list, tuple)) else sampling
            ids.append(sched.add_request(prompt, cfg))
        done = sched.run()
        self.last_scheduler = sched
        for i in ids:
            if done[i].error is not None:
                raise done[i].error
        return [list(done[i].generated) for i in ids]

    # ------------------------------------------------------------------ info
    def weight_bytes_per_step(self) -> int:
        return self.model.weight_bytes_per_step()

    def metrics(self) -> Dict[str, object]:
        return {"steps": self.step_fn.steps, "rows": self.step_fn.rows_total,
                "cache": self.cache.metrics()}


def write_random_model(model_dir: str, config, seed: int, dtype=torch.bfloat16) -> str:
    """Random-weights mode: write ``config.json`` and ``model.safetensors``."""
    arch_name = getattr(config, "architecture", None) or getattr(config, "ARCHITECTURE")
    arch = get_architecture(arch_name)
    expected = CausalLM(arch.build_spec(config)).tensor_specs()
    return write_model_dir(model_dir, config, expected, seed, dtype)
