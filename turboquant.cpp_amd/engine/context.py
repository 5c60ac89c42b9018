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
    side_stream: "torch.cuda.Stream | None" = None   # a second stream for work that does not depend on the main line
    capturing: bool = False      # the step is being recorded for replay: what the host pays now it pays once
    # called with (schedule entry, the residual stream behind that entry [T, H] float32, the batch), for whoever wants
    # to look at activations layer by layer (the reference prints them under TQ_DEBUG, tq_transformer.c:2340-2344)
    layer_hook: "object | None" = None
    native: "object | None" = None      # the model's form for the step executor (engine/native.py), if it has one

    def kv(self, entry: int) -> KVView:
        """Keys and values of the schedule entry (or of the entry whose cache it reads)."""
        return self.cache.kv(entry)

    def fork(self):
        """Lets the side stream start from where the current stream is; returns it (None: run in line)."""
        if self.side_stream is None:
            return None
        self.side_stream.wait_stream(torch.cuda.current_stream())
        return self.side_stream

    def join(self) -> None:
        """The current stream waits for what the side stream has been given."""
        if self.side_stream is not None:
            torch.cuda.current_stream().wait_stream(self.side_stream)

    def state(self, entry: int) -> torch.Tensor:
        """The entry's fixed-size state, [slots, ...]; row ``slot`` belongs to the sequence in that slot."""
        return self.cache.state(entry)

    def state_rows(self, entry: int) -> torch.Tensor:
        """The state of the step's sequences, [sequences, ...], in the step's order: gathered through the slots on
        the device, so a captured step replays it for other slots."""
        from ..csrc import ops
        return ops.gather_rows(self.cache.state(entry), self.batch.slots_dev, self.act)

    def store_state_rows(self, entry: int, rows: torch.Tensor) -> None:
        """Puts the advanced state of the step's sequences back (the counterpart of ``state_rows``)."""
        from ..csrc import ops
        ops.scatter_rows(self.cache.state(entry), self.batch.slots_dev, rows.contiguous(), self.act)
