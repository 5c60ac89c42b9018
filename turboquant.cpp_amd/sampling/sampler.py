"""Choice of the next token of every sequence of a step, on the GPU.

The reference's order (/root/reference/src/engine/tq_generate.c:386-410, :587-603): repetition penalty over
the last ``rep_window`` tokens (prompt tail included), then ``tq_sample_topp``: greedy when temperature
or top_p is not positive (:84-86), else temperature and top-p with one uniform draw per token.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..csrc import ops
from .rng import XorShift64Star, stream_seed


@dataclass
class SamplingOptions:
    temperature: float = 0.7
    top_p: float = 0.9
    seed: int = 42
    rep_penalty: float = 1.1
    rep_window: int = 32

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0 or self.top_p <= 0.0


@dataclass
class SequenceSampling:
    """What sampling remembers of one sequence: its random stream and its recent tokens."""
    rng: XorShift64Star
    recent: list[int] = field(default_factory=list)

    def push(self, token: int, keep: int) -> None:
        self.recent.append(token)
        if len(self.recent) > max(keep, 128):
            del self.recent[:len(self.recent) - max(keep, 128)]


class Sampler:
    def __init__(self, options: SamplingOptions, act: str, device):
        self.options, self.act, self.device = options, act, device
        self.window = max(0, min(options.rep_window, 128))    # the reference caps the window at 128 (:367)
        self._staging = None

    def _staged(self, rows: int) -> dict:
        """Host arrays that the step's small inputs (recent tokens, their counts, the uniform draws) are written
        into before they go to the device: pinned where there is a GPU, so that the copies are issued without the
        host waiting for the stream (a copy from ordinary memory returns only when everything issued before it has
        run, the whole decode step included).  They are written again at the next ``launch``; by then the tokens of
        this one have been fetched, so its copies have run."""
        if self._staging is None or self._staging["rows"] < rows:
            pin = self.device is not None and torch.device(self.device).type == "cuda"
            n = max(rows, 8)
            self._staging = {"rows": n,
                             "recent": torch.empty((n, max(self.window, 1)), dtype=torch.int32, pin_memory=pin),
                             "counts": torch.empty((n,), dtype=torch.int32, pin_memory=pin),
                             "uniforms": torch.empty((n,), dtype=torch.float32, pin_memory=pin)}
        return self._staging

    def new_sequence(self, index: int, prompt: list[int]) -> SequenceSampling:
        st = SequenceSampling(XorShift64Star(stream_seed(self.options.seed, index)))
        st.recent = list(prompt[-self.window:]) if self.window else []
        return st

    def sample(self, logits: torch.Tensor, states: list[SequenceSampling]) -> list[int]:
        """One token per row of ``logits`` [R, V]; row i belongs to ``states[i]``.  Changes ``logits``
        when a repetition penalty applies."""
        out = self.launch(logits, states).tolist()
        self.finish(out, states)
        return out

    def launch(self, logits: torch.Tensor, states: list[SequenceSampling]) -> torch.Tensor:
        """Issues the choice and returns the tokens as int32 [R] on the device; ``finish`` must be told the
        tokens before the next ``launch`` for the same sequences."""
        o, R = self.options, logits.shape[0]
        staged = self._staged(R)
        if o.rep_penalty > 1.0 and self.window > 0:
            recent, counts = staged["recent"][:R], staged["counts"][:R]
            recent_np, counts_np = recent.numpy(), counts.numpy()
            recent_np.fill(-1)
            for i, st in enumerate(states):
                tail = st.recent[-self.window:][::-1]      # newest first, the reference's order
                recent_np[i, :len(tail)] = tail
                counts_np[i] = len(tail)
            ops.rep_penalty(logits, recent.to(self.device, non_blocking=True), counts.to(self.device, non_blocking=True),
                            o.rep_penalty, self.act)
        if o.greedy:
            return ops.argmax(logits, self.act)
        u = staged["uniforms"][:R]
        u.numpy()[:] = [st.rng.next_float() for st in states]
        return ops.sample_topp(logits, o.temperature, o.top_p, u.to(self.device, non_blocking=True), self.act)

    def finish(self, tokens: list[int], states: list[SequenceSampling]) -> None:
        for st, t in zip(states, tokens):
            st.push(t, self.window)


class TokenFetch:
    """Brings a step's chosen tokens to the host without waiting for what is issued after them: on a GPU the copy
    into pinned memory is issued right behind the choice, with an event behind it, and ``wait`` waits for that
    event only; a step issued between ``start`` and ``wait`` runs while the host looks at the tokens."""

    def __init__(self, device, capacity: int):
        self.on_gpu = device is not None and torch.device(device).type == "cuda"
        if self.on_gpu:
            self.host = torch.empty(capacity, dtype=torch.int32).pin_memory()
            self.done = torch.cuda.Event()
        self.pending = None

    def start(self, ids: torch.Tensor) -> None:
        if self.on_gpu:
            self.host[:ids.numel()].copy_(ids, non_blocking=True)
            self.done.record()
        self.pending = ids

    def wait(self) -> list[int]:
        ids, self.pending = self.pending, None
        if not self.on_gpu:
            return ids.tolist()
        self.done.synchronize()
        return self.host[:ids.numel()].tolist()
