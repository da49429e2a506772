"""Random-weights mode: a model folder from a configuration and a seed.

Every tensor is drawn as the part that owns it says (``TensorSpec.init``): matrices,
biases and other learned vectors from N(0, std), the weights of norms from 1 + N(0,
norm_std), in the order in which the model lists its tensors, each tensor from
its own generator seeded by (seed, index), so a tensor's values do not depend
on the sizes of the others.  The reference has no such mode for this
architecture; its test fixture uses a closed formula
(rust/engine/src/runner/model/qwen2/engine.rs:2379-2398) and its toy model
draws per-tensor seeded normals (rust/engine/src/runner/model/simple_mlp/engine.rs:231-245).
"""
from __future__ import annotations

import json
import os
from typing import Dict, Iterator, Tuple

import torch

from .loader import TensorSpec, INT_TABLE, INIT_NORMAL, INIT_NORM, INIT_ZEROS, INIT_ONES
from .safetensors_io import save_safetensors


def random_tensors(expected: Dict[str, TensorSpec], seed: int, dtype: torch.dtype = torch.bfloat16,
                   std: float = 0.02, norm_std: float = 0.1,
                   device="cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    """One tensor per expected name, drawn as its ``TensorSpec.init`` says.  ``device``: where
    they are drawn (a GPU's generator gives other numbers than the host's for the same
    seed; a model folder is always written from the host's)."""
    for index, (name, spec) in enumerate(expected.items()):
        gen = torch.Generator(device=device)
        gen.manual_seed((int(seed) * 1000003 + index * 7919 + 12345) % (2 ** 63 - 1))
        if spec.kind == INT_TABLE:
            yield name, torch.zeros(spec.shape, dtype=torch.int32, device=device)
            continue
        if spec.init == INIT_ZEROS:
            yield name, torch.zeros(spec.shape, dtype=dtype, device=device)
            continue
        if spec.init == INIT_ONES:
            yield name, torch.ones(spec.shape, dtype=dtype, device=device)
            continue
        values = torch.randn(spec.shape, generator=gen, dtype=torch.float32, device=device)
        if spec.init == INIT_NORM:
            values = 1.0 + norm_std * values
        elif spec.init == INIT_NORMAL:
            values = std * values
        else:
            raise ValueError(f"tensor '{name}': unknown way to draw it, init={spec.init!r}")
        yield name, values.to(dtype)


def write_model_dir(model_dir: str, config, expected: Dict[str, TensorSpec], seed: int,
                    dtype: torch.dtype = torch.bfloat16, std: float = 0.02,
                    norm_std: float = 0.1, tensors=None) -> str:
    """Write ``config.json`` and ``model.safetensors`` of a random model.  ``tensors``: the
    (name, tensor) pairs to write instead of ``random_tensors(expected, seed, ...)`` (an
    architecture's own way of drawing them)."""
    os.makedirs(model_dir, exist_ok=True)
    raw = config.to_dict()
    raw["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32",
                          torch.float16: "float16"}[dtype]
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw, f, indent=2)
    save_safetensors(os.path.join(model_dir, "model.safetensors"),
                     tensors if tensors is not None else random_tensors(expected, seed, dtype, std, norm_std),
                     metadata={"format": "pt", "seed": str(seed)})
    return model_dir
