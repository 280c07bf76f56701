"""Architecture-neutral description of a decoder: what the parts are and in which
order they run.  An architecture's typed configuration (for instance
`Gemma2Config`) is turned into a `ModelSpec`; everything below the configuration
(model, cache manager, step function) reads only the `ModelSpec`.

The layer pattern follows simply/model_lib.py:2839-2844 (each block gets its kind
from a pattern) but as data: every layer carries its own part specs, and the order
in which layers run is a list of `ScheduleEntry`, which may name a layer twice or
let an entry read the cache that an earlier entry wrote.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Mapping


@dataclasses.dataclass(frozen=True)
class PartSpec:
    """One part: `kind` is a name in the part's registry, `params` are its sizes and
    constants, `tensors` maps the part's own parameter names to tensor names in the
    model folder."""

    kind: str
    params: Mapping[str, Any] = dataclasses.field(default_factory=dict)
    tensors: Mapping[str, str] = dataclasses.field(default_factory=dict)


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    """A block: an arrangement (`block.kind`) of a mixer, a feed-forward and norms."""

    block: PartSpec
    mixer: PartSpec
    feed_forward: PartSpec
    norms: Mapping[str, PartSpec] = dataclasses.field(default_factory=dict)


@dataclasses.dataclass(frozen=True)
class ScheduleEntry:
    """Run layer `layer`.  `cache_from` names an earlier schedule entry (by its index
    in the schedule) whose cache this entry reads instead of keeping its own."""

    layer: int
    cache_from: int | None = None


@dataclasses.dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    schedule: tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    max_position: int
    eos_token_ids: tuple[int, ...] = ()
    initializer_range: float = 0.02
    #: tensor names that a model folder may hold beside the expected ones, each with the expected tensor whose
    #: copy it must be (a tied head stored once more under its own name): checked for equality, then left unread
    copies: Mapping[str, str] = dataclasses.field(default_factory=dict)

    def validate(self) -> None:
        n = len(self.layers)
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < n:
                raise ValueError(f"schedule entry {i} names layer {e.layer}, but there are {n} layers")
            if e.cache_from is not None:
                if not 0 <= e.cache_from < i:
                    raise ValueError(
                        f"schedule entry {i} reads the cache of entry {e.cache_from}, which does not run before it")
                if self.schedule[e.cache_from].cache_from is not None:
                    raise ValueError(
                        f"schedule entry {i} reads the cache of entry {e.cache_from}, which itself has none")
        for name, of in self.copies.items():
            if name == of:
                raise ValueError(f"tensor {name!r} is declared a copy of itself")
