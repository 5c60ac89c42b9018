"""The data that describes a model before any weight is loaded.

An architecture turns its typed configuration into a :class:`ModelPlan`: for every
layer the kinds of its parts with their sizes and constants, the checkpoint
tensors each parameter comes from, and the order in which layers run.  Parts are
built from this data alone; none of them knows the architecture it serves.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


@dataclass(frozen=True)
class Source:
    """Where a parameter comes from in the checkpoint.

    ``how`` is ``"single"`` (one tensor), ``"stack"`` (a new leading dimension
    over ``names``) or ``"concat"`` (joined along dimension 0).
    """
    names: tuple[str, ...]
    how: str = "single"

    @staticmethod
    def single(name: str) -> "Source":
        return Source((name,), "single")

    @staticmethod
    def stack(names) -> "Source":
        return Source(tuple(names), "stack")

    @staticmethod
    def concat(names) -> "Source":
        return Source(tuple(names), "concat")


@dataclass
class PartSpec:
    """One part: its kind (a key of the part registry), its arguments and its tensors."""
    kind: str
    args: dict[str, Any] = field(default_factory=dict)
    tensors: dict[str, Source] = field(default_factory=dict)


@dataclass
class LayerSpec:
    """One layer: how its parts are arranged (``block``) and the parts themselves."""
    block: str
    parts: dict[str, PartSpec]


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  ``cache_of`` names an earlier entry whose cache this run reads
    instead of keeping its own."""
    layer: int
    cache_of: int | None = None


@dataclass
class ModelPlan:
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: list[LayerSpec]
    schedule: list[ScheduleEntry]
    final_norm: PartSpec
    embedding: Source
    lm_head: Source | None          # None: tied to the embedding
    max_positions: int
    stop_tokens: tuple[int, ...] = ()
    embedding_scale: float = 1.0            # the embedding rows are multiplied by it
    logit_softcap: float | None = None      # logits <- cap * tanh(logits / cap)

    def validate(self) -> None:
        n = len(self.layers)
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ValueError(f"logit_softcap must be positive, got {self.logit_softcap}")
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < n:
                raise ValueError(f"schedule entry {i} names layer {e.layer}, model has {n}")
            if e.cache_of is not None and not 0 <= e.cache_of < i:
                raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_of}, which does not run before it")
