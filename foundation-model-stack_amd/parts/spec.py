"""A model described as data: which parts, with which constants, in which order.

An architecture is a function from its configuration to a ``ModelSpec``; the
generic ``DecoderModel`` is built from the spec alone.  Layers are chosen one
by one, so one model can mix different mixers and feed-forwards, and the order
in which layers run is a list of its own (``schedule``) that may name a layer
twice or let an entry read the cache of an earlier entry.
"""

from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional


@dataclasses.dataclass
class PartSpec:
    kind: str
    args: dict = dataclasses.field(default_factory=dict)


@dataclasses.dataclass
class LayerSpec:
    mixer: PartSpec
    feed_forward: PartSpec
    norm: Optional[PartSpec] = None  # the spec of every norm the block asks for ...
    block: PartSpec = dataclasses.field(default_factory=lambda: PartSpec("pre_norm"))
    position: Optional[str] = None  # key into ModelSpec.positions, handed to the mixer
    norms: Optional[List[PartSpec]] = None  # ... or one spec for each, in the order of the block's `norm_arguments`


@dataclasses.dataclass
class ScheduleEntry:
    layer: int  # index into ModelSpec.layers
    cache_of: Optional[int] = None  # earlier schedule entry whose cache this entry reads instead of owning one


@dataclasses.dataclass
class ModelSpec:
    vocab: int
    width: int
    max_seq_len: int
    layers: List[LayerSpec]
    final_norm: PartSpec
    embedding: PartSpec = dataclasses.field(default_factory=lambda: PartSpec("table"))
    head: PartSpec = dataclasses.field(default_factory=lambda: PartSpec("linear"))
    positions: Dict[str, PartSpec] = dataclasses.field(default_factory=dict)
    schedule: Optional[List[ScheduleEntry]] = None  # default: every layer once, in order
    tie_heads: bool = False
    # parameter name prefixes (the reference's names by default)
    embedding_name: str = "base_model.embedding"
    layer_name: str = "base_model.layers.{i}"
    final_norm_name: str = "base_model.dec_norm"
    head_name: str = "head"

    def resolved_schedule(self) -> List[ScheduleEntry]:
        if self.schedule is None:
            return [ScheduleEntry(i) for i in range(len(self.layers))]
        for n, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"schedule entry {n} names layer {entry.layer}, the model has {len(self.layers)}")
            if entry.cache_of is not None:
                if not 0 <= entry.cache_of < n:
                    raise ValueError(f"schedule entry {n} reads the cache of entry {entry.cache_of}, which does not run before it")
                if self.schedule[entry.cache_of].cache_of is not None:
                    raise ValueError(f"schedule entry {n} reads the cache of entry {entry.cache_of}, which owns none")
        return list(self.schedule)
