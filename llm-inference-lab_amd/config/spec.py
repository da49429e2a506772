"""Architecture-neutral description of a model as data.

An architecture's builder turns its typed configuration into a ``ModelSpec``:
what each block is made of (norm, mixer, feed-forward, position encoding, all
with their sizes and constants as plain fields and their tensor names as
strings) and the order in which blocks run.  The parts are built from these
records and never see the configuration they came from.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List, Optional, Tuple


@dataclasses.dataclass(frozen=True)
class PartSpec:
    """A part is chosen by ``kind`` (a name in the parts registry); ``params``
    holds its sizes and constants; ``tensors`` maps the part's own role names
    (for instance ``q_weight``) to tensor names in the model file."""

    kind: str
    params: Dict[str, Any] = dataclasses.field(default_factory=dict)
    tensors: Dict[str, str] = dataclasses.field(default_factory=dict)


@dataclasses.dataclass(frozen=True)
class BlockSpec:
    """One layer: a block kind (a name in the parts registry) and the parts it is made of,
    by the names that this kind gives them.  Which parts a block has and how they are
    arranged is the kind's business: ``prenorm`` takes ``norm1, mixer, norm2,
    feed_forward`` (norm, sublayer, residual add, twice); a kind with one norm and two
    parallel sublayers, with norms on both sides of a sublayer, or without a feed-forward
    names its own.  The block class receives the named ``PartSpec``s and ``params`` as
    keyword arguments."""

    kind: str
    parts: Dict[str, PartSpec] = dataclasses.field(default_factory=dict)
    params: Dict[str, Any] = dataclasses.field(default_factory=dict)


@dataclasses.dataclass(frozen=True)
class ScheduleEntry:
    """One run of a block.  ``block`` indexes ``ModelSpec.blocks`` (the same
    block may run more than once).  ``cache_of`` names an earlier schedule
    entry whose cache this run reads instead of keeping one of its own."""

    block: int
    cache_of: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: PartSpec
    blocks: Tuple[BlockSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: Tuple[int, ...] = ()

    def validate(self) -> None:
        for i, entry in enumerate(self.schedule):
            if not 0 <= entry.block < len(self.blocks):
                raise ValueError(f"schedule[{i}] names block {entry.block}, "
                                 f"but there are {len(self.blocks)} blocks")
            if entry.cache_of is not None:
                if not 0 <= entry.cache_of < i:
                    raise ValueError(f"schedule[{i}].cache_of must name an earlier entry")
                if self.schedule[entry.cache_of].cache_of is not None:
                    raise ValueError(f"schedule[{i}].cache_of names an entry that owns no cache")
