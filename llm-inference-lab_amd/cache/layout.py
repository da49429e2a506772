"""The order of the numbers inside one page of one kv head.

The cache tensors keep their logical shapes (keys ``[..., P, d]``, values
``[..., d, P]``), but the ``P * d`` numbers of a (page, kv head) pair lie in the
order in which the attention kernels' matrix-core fragments read them, so that
every wave instruction reads consecutive memory:

* keys:   ``[16-key block][octet of d][key in block][8]``
* values: ``[16-key block][16-wide block of d][group of 4 keys][number in block][4]``

(the same formulas as ``kcache_index`` / ``vcache_index`` in ``csrc/common.h``).
The kernels never need this module; it serves tests, tools and anyone who wants
to look into a cache from Python.
"""
from __future__ import annotations

import torch


def key_index(page_size: int, d: int) -> torch.Tensor:
    """``[P, d]`` int64: where key ``k``'s number ``dd`` lies in the flat page."""
    k = torch.arange(page_size).view(-1, 1)
    dd = torch.arange(d).view(1, -1)
    return (((k >> 4) * (d >> 3) + (dd >> 3)) * 16 + (k & 15)) * 8 + (dd & 7)


def value_index(page_size: int, d: int) -> torch.Tensor:
    """``[d, P]`` int64: where number ``dd`` of the value of key ``k`` lies."""
    k = torch.arange(page_size).view(1, -1)
    dd = torch.arange(d).view(-1, 1)
    return ((((k >> 4) * (d >> 4) + (dd >> 4)) * 4 + ((k & 15) >> 2)) * 16 + (dd & 15)) * 4 + (k & 3)


def _scatter(logical: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    flat = logical.reshape(*logical.shape[:-2], -1)
    out = torch.empty_like(flat)
    out[..., index.reshape(-1).to(flat.device)] = flat
    return out.view(logical.shape)


def _gather(physical: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    flat = physical.reshape(*physical.shape[:-2], -1)
    return flat[..., index.reshape(-1).to(flat.device)].view(physical.shape)


def keys_to_cache_order(keys: torch.Tensor) -> torch.Tensor:
    """``[..., P, d]`` row-major keys -> the same shape in cache order."""
    return _scatter(keys, key_index(keys.shape[-2], keys.shape[-1]))


def keys_from_cache_order(keys: torch.Tensor) -> torch.Tensor:
    return _gather(keys, key_index(keys.shape[-2], keys.shape[-1]))


def values_to_cache_order(values: torch.Tensor) -> torch.Tensor:
    """``[..., d, P]`` transposed values -> the same shape in cache order."""
    return _scatter(values, value_index(values.shape[-1], values.shape[-2]))


def values_from_cache_order(values: torch.Tensor) -> torch.Tensor:
    return _gather(values, value_index(values.shape[-1], values.shape[-2]))
