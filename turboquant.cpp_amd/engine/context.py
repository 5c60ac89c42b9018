"""What a part sees of the running step: the packed batch, the cache, the activation type."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..cache.paged import KVView, PagedCache
from .batch import StepBatch


@dataclass
class StepContext:
    batch: StepBatch
    cache: PagedCache
    act: str                          # "float32" or "bfloat16": the type of activations and cache
    device: torch.device

    def kv(self, entry: int) -> KVView:
        """Keys and values of the schedule entry (or of the entry whose cache it reads)."""
        return self.cache.kv(entry)

    def state(self, entry: int) -> torch.Tensor:
        """The entry's fixed-size state, [slots, ...]; row ``slot`` belongs to the sequence in that slot."""
        return self.cache.state(entry)
