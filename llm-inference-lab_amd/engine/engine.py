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
                 progress: Optional[Callable[[str], None]] = None, strict_weights: bool = False):
        self.dtype = parse_dtype(dtype)
        if model_dir is not None:
            self.architecture, self.config = read_config(model_dir)
        elif config is not None:
            arch_name = getattr(config, "architecture", None) or getattr(config, "ARCHITECTURE")
            self.architecture, self.config = get_architecture(arch_name), config
        else:
            raise ValueError("give a model_dir or a config")
        self.spec = self.architecture.build_spec(self.config)
        # The model's end-of-sequence ids: those of generation_config.json if the folder
        # has one that names any, else config.json's (engine.rs:403-407).  A request's own
        # ids go before both.  The file's other fields are kept in ``generation_config``
        # for callers that want them as defaults; requests carry their own options, as in
        # the reference (model_runner.rs:612-614).
        from ..sampling.params import read_generation_config
        self.generation_config = read_generation_config(model_dir) if model_dir is not None else None
        self.eos_token_ids = tuple(self.spec.eos_token_ids)
        if self.generation_config is not None and self.generation_config.eos_token_id is not None:
            self.eos_token_ids = self.generation_config.eos_ids()
        self.model = CausalLM(self.spec)
        if ops is None:
            # compile what this model's parts ask for before the GPU is first touched
            from ..kernels import build
            build.core_library()
            for kind, parameter in self.model.kernel_libraries():
                build.library(kind, parameter)
        self.ops = ops if ops is not None else default_ops(device)
        self.device = self.ops.device
        expected = self.model.tensor_specs()
        if model_dir is not None:
            loaded = load_tensors(model_dir, expected, self.dtype, self.device, progress, strict_weights)
        elif tensors is not None:
            loaded = place_tensors(tensors, expected, self.dtype, self.device, strict=strict_weights)
        else:
            loaded = place_tensors(draw_random_tensors(self.architecture, self.config, expected, seed),
                                   expected, self.dtype, self.device, "random weights")
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
                                    graph=graph)
        self._sampler = None
        self.last_scheduler = None
        from .instruments import RequestInstruments
        from .profiling import ranges_from_environment
        self.request_instruments = RequestInstruments()
        self.model.ranges = ranges_from_environment()

    CACHE_SHARE_OF_FREE_MEMORY = 0.9

    def _pages_that_fit(self, groups) -> int:
        """Pages (per group) that fit the GPU memory that is free now, leaving a tenth of
        it for scratch buffers; at least one request of full length."""
        if self.device.type != "cuda":
            return 1 << 40
        page_bytes = sum(len(g.entries) * g.spec.bytes_per_token(self.dtype) for g in groups) * self.page_size
        free, _ = torch.cuda.mem_get_info(self.device)
        fit = int(free * self.CACHE_SHARE_OF_FREE_MEMORY) // max(page_bytes, 1)
        return max(fit, pages_for_tokens(self.max_seq_len, self.page_size))

    # ------------------------------------------------------------- requests
    def open(self, request_id) -> RequestCache:
        """Give a new request a row in the cache manager."""
        return self.cache.admit(request_id)

    def close(self, request: RequestCache) -> None:
        """The request has ended: everything it holds is given back."""
        self.cache.release(request)

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """One step; an entry that cannot run raises before anything has run."""
        return self.step_fn(entries)

    def run_step(self, entries: Sequence[StepEntry]):
        """One step with a result for every entry (``StepResult``): entries that cannot run
        carry their error, the others run as one batch."""
        return self.step_fn.run(entries)

    @property
    def step_instruments(self):
        return self.step_fn.instruments

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
        """Counters and histograms as one dictionary of numbers: the step function's (steps
        and input tokens by phase, host submit and step wall times, batch sizes, failed
        steps, token readback), the decode graphs', the scratch buffers', the cache's, and
        the requests' over every scheduler this engine has made."""
        fn = self.step_fn
        out = {"steps": fn.steps, "rows": fn.rows_total, "step": fn.instruments.snapshot(),
               "graphs": {"enabled": fn.use_graph, "captures": fn.graph_captures,
                          "replays": fn.graph_replays, "evictions": fn.graph_evictions,
                          "kept": len(fn._graphs), "decode_calls": fn.decode_calls},
               "scratch": {"bytes": fn.ctx.scratch_bytes, "allocations": fn.ctx.scratch_allocations},
               "launch_sequences": {"recorded": self.model.launches_recorded,
                                    "replayed": self.model.launches_replayed},
               "kernel_calls": getattr(self.ops, "calls_made", None),
               "requests": self.request_instruments.snapshot(),
               "cache": self.cache.metrics()}
        out["step"]["failed_steps"] = fn.failed_steps
        return out


def settle_collector() -> None:
    """For a process that serves: call once when the engine is built and has run a few steps.
    Collects what is garbage now and moves everything alive at this moment (the modules of
    the libraries, the model's parts, the kept launch sequences) out of the reach of
    Python's cyclic collector (``gc.freeze``), which from then on walks only what requests
    allocate.  Without it a full collection walks some 200,000 objects: 35 to 70 ms every
    few hundred steps of a large batch, a tenth of a second of a step's tail latency.  The
    setting is the process's, not the engine's: a library does not take it by itself."""
    import gc
    gc.collect()
    gc.freeze()


def draw_random_tensors(architecture, config, expected, seed: int, dtype=torch.bfloat16):
    """The (name, tensor) pairs of the random-weights mode: drawn by the architecture's own
    ``random_init(config, expected, seed, dtype)`` if its registry entry has one, else
    every tensor as the part that owns it says (``TensorSpec.init``)."""
    if architecture.random_init is not None:
        return architecture.random_init(config, expected, seed, dtype)
    return random_tensors(expected, seed, dtype)


def write_random_model(model_dir: str, config, seed: int, dtype=torch.bfloat16) -> str:
    """Random-weights mode: write ``config.json`` and ``model.safetensors``."""
    arch_name = getattr(config, "architecture", None) or getattr(config, "ARCHITECTURE")
    arch = get_architecture(arch_name)
    expected = CausalLM(arch.build_spec(config)).tensor_specs()
    return write_model_dir(model_dir, config, expected, seed, dtype,
                           tensors=draw_random_tensors(arch, config, expected, seed, dtype))
