"""The tokens of one step, packed: what the step function hands to every part.

The reference's forward takes one token and one position (``tq_forward(model, state, token, pos)``,
/root/reference/src/engine/tq_transformer.c:2281).  A step here takes the next tokens of several
sequences at once, back to back in one array, each token with its position and the slot of its
sequence; a sequence contributes its whole prompt or one decoded token.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch


@dataclass
class StepBatch:
    slots: list[int]                  # slot of each sequence of the step
    n_new: list[int]                  # tokens each sequence brings
    start: list[int]                  # position of each sequence's first new token
    n_tokens: int
    tokens: torch.Tensor              # int32 [T]
    positions: torch.Tensor           # int32 [T]
    slot_of_token: torch.Tensor       # int32 [T]
    cu_seqlens: torch.Tensor          # int32 [B+1]: first token of each sequence in the packed arrays
    slots_dev: torch.Tensor           # int32 [B]
    start_dev: torch.Tensor           # int32 [B]
    want_rows: torch.Tensor           # int32 [R]: packed rows whose logits are wanted
    n_want: int
    fixed_max_end: int | None = None  # set when launches must not depend on the sequences' true lengths

    @property
    def n_seqs(self) -> int:
        return len(self.slots)

    @property
    def max_new(self) -> int:
        return max(self.n_new)

    @property
    def is_decode(self) -> bool:
        return self.max_new == 1

    @property
    def max_end(self) -> int:
        if self.fixed_max_end is not None:
            return self.fixed_max_end
        return max(s + n for s, n in zip(self.start, self.n_new))

    def runs(self) -> dict:
        """The step as runs of consecutive positions, one per sequence, for kernels that tile over tokens."""
        return {"cu_seqlens": self.cu_seqlens, "slots": self.slots_dev, "start": self.start_dev,
                "max_new": self.max_new, "max_end": self.max_end, "decode": self.is_decode}


def pack_step(slots, starts, token_lists, wants, device) -> StepBatch:
    """Packs per-sequence token lists into the arrays of a step and sends them to the device in one copy.

    ``wants[i]`` lists the places among sequence i's new tokens whose logits are asked for."""
    n_new = [len(t) for t in token_lists]
    B, T = len(slots), sum(n_new)
    R = sum(len(w) for w in wants)
    layout = [("tokens", T), ("positions", T), ("slot_of_token", T), ("cu_seqlens", B + 1), ("slots", B),
              ("start", B), ("want_rows", R)]
    total = sum(n for _, n in layout)
    host = np.empty(total, dtype=np.int32)
    views, o = {}, 0
    for name, n in layout:
        views[name] = host[o:o + n]
        o += n
    off = 0
    want_rows = []
    for i, (slot, start, toks, want) in enumerate(zip(slots, starts, token_lists, wants)):
        n = len(toks)
        views["tokens"][off:off + n] = toks
        views["positions"][off:off + n] = np.arange(start, start + n, dtype=np.int32)
        views["slot_of_token"][off:off + n] = slot
        views["cu_seqlens"][i] = off
        for w in want:
            if not 0 <= w < n:
                raise ValueError(f"wanted place {w} is outside the {n} tokens that sequence {i} brings")
            want_rows.append(off + w)
        off += n
    views["cu_seqlens"][B] = off
    views["slots"][:] = slots
    views["start"][:] = starts
    views["want_rows"][:] = want_rows
    dev = torch.from_numpy(host)
    if device is not None and torch.device(device).type != "cpu":
        dev = dev.to(device)
    parts, o = {}, 0
    for name, n in layout:
        parts[name] = dev[o:o + n]
        o += n
    return StepBatch(slots=list(slots), n_new=n_new, start=list(starts), n_tokens=T, tokens=parts["tokens"],
                     positions=parts["positions"], slot_of_token=parts["slot_of_token"],
                     cu_seqlens=parts["cu_seqlens"], slots_dev=parts["slots"], start_dev=parts["start"],
                     want_rows=parts["want_rows"], n_want=R)
