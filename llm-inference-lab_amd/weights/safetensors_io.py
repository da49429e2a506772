"""Reader and writer of the safetensors container.

Layout of a file: 8 bytes (little-endian u64) = length N of the header, N
bytes of JSON mapping each tensor name to ``{"dtype", "shape",
"data_offsets": [begin, end]}`` (offsets relative to the end of the header),
then the raw little-endian tensor bytes.  Files are memory-mapped; a tensor's
bytes are touched only when it is asked for.  The reference reads the same
layouts through its loader (rust/engine/src/runner/loader.rs:151-192): one
``model.safetensors``, or an authoritative ``model.safetensors.index.json``
whose ``weight_map`` names the shard of every tensor.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    """One memory-mapped safetensors file."""

    def __init__(self, path: str):
        self.path = path
        self._file = open(path, "rb")
        size = os.fstat(self._file.fileno()).st_size
        if size < 8:
            raise ValueError(f"{path}: too short to be a safetensors file")
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        (header_len,) = struct.unpack("<Q", self._map[:8])
        if header_len > size - 8:
            raise ValueError(f"{path}: header length {header_len} exceeds the file size")
        try:
            header = json.loads(self._map[8:8 + header_len].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise ValueError(f"{path}: header is not valid JSON: {e}") from None
        self.metadata = header.pop("__metadata__", {})
        self._base = 8 + header_len
        self.entries: Dict[str, dict] = {}
        for name, info in header.items():
            dtype = info.get("dtype")
            if dtype not in _DTYPES:
                raise ValueError(f"{path}: tensor '{name}' has unsupported dtype {dtype!r}")
            begin, end = info["data_offsets"]
            count = 1
            for d in info["shape"]:
                count *= int(d)
            width = torch.empty((), dtype=_DTYPES[dtype]).element_size()
            if end - begin != count * width or self._base + end > size or begin < 0:
                raise ValueError(f"{path}: tensor '{name}' has inconsistent offsets")
            self.entries[name] = info

    def names(self) -> List[str]:
        return list(self.entries)

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(int(d) for d in self.entries[name]["shape"])

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self.entries[name]["dtype"]]

    def tensor(self, name: str) -> torch.Tensor:
        """The tensor's values, copied out of the mapping (CPU, stored dtype)."""
        info = self.entries[name]
        begin, end = info["data_offsets"]
        shape = self.shape(name)
        dtype = _DTYPES[info["dtype"]]
        if end == begin:
            return torch.empty(shape, dtype=dtype)
        flat = np.frombuffer(self._map, dtype=np.uint8, count=end - begin, offset=self._base + begin)
        return torch.from_numpy(flat.copy()).view(dtype).reshape(shape)

    def close(self) -> None:
        try:
            self._map.close()
        except BufferError:
            pass
        self._file.close()


class ModelFiles:
    """All tensors of a model folder, whichever file holds them."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        index_path = os.path.join(model_dir, "model.safetensors.index.json")
        single_path = os.path.join(model_dir, "model.safetensors")
        self._files: Dict[str, SafetensorsFile] = {}
        self._where: Dict[str, str] = {}
        if os.path.isfile(index_path):
            with open(index_path, "r", encoding="utf-8") as f:
                index = json.load(f)
            weight_map = index.get("weight_map")
            if not isinstance(weight_map, dict):
                raise ValueError(f"{index_path}: no 'weight_map'")
            for name, shard in weight_map.items():
                if (not isinstance(shard, str) or os.path.basename(shard) != shard
                        or not shard.endswith(".safetensors")):
                    raise ValueError(f"{index_path}: shard name {shard!r} is not a plain "
                                     f"relative *.safetensors file name")
                if shard not in self._files:
                    self._files[shard] = SafetensorsFile(os.path.join(model_dir, shard))
                if name not in self._files[shard].entries:
                    raise ValueError(f"{index_path}: tensor '{name}' is not in shard '{shard}'")
                self._where[name] = shard
        elif os.path.isfile(single_path):
            self._files["model.safetensors"] = SafetensorsFile(single_path)
            for name in self._files["model.safetensors"].names():
                self._where[name] = "model.safetensors"
        else:
            raise FileNotFoundError(
                f"{model_dir}: neither model.safetensors nor model.safetensors.index.json found")

    def names(self) -> List[str]:
        return list(self._where)

    def shape(self, name: str):
        return self._files[self._where[name]].shape(name)

    def dtype(self, name: str):
        return self._files[self._where[name]].dtype(name)

    def tensor(self, name: str) -> torch.Tensor:
        return self._files[self._where[name]].tensor(name)

    def close(self) -> None:
        for f in self._files.values():
            f.close()


def save_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]],
                     metadata: Dict[str, str] = None) -> None:
    """Write tensors (name, CPU tensor) in the order given."""
    items = [(name, t.detach().contiguous().cpu()) for name, t in tensors]
    header: Dict[str, dict] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    for name, t in items:
        if t.dtype not in _NAMES:
            raise ValueError(f"tensor '{name}': dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for _, t in items:
            if t.numel():
                f.write(t.reshape(-1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
