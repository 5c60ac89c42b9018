"""Decode steps as HIP graphs.

A decode step is some hundreds of small kernels whose launch costs more than their work; once a step of a
given shape has run, its whole launch sequence is captured and replayed.  What changes from step to step
(tokens, positions, slots) lives in one device array that is refilled by a copy before each replay; what
the launches bake in (number of sequences, the number of 256-position runs attention is split into) is the
key of the graph.  No memset is recorded (only kernels), and results are the bits the eager step gives.
"""
from __future__ import annotations

import gc

import numpy as np
import torch

from .batch import StepBatch
from .context import StepContext

RUN_BUCKET = 2048        # graphs are keyed by the longest sequence rounded up to this many positions


class DecodeGraph:
    def __init__(self, engine, n_seqs: int, bucket_end: int, pool):
        self.engine, self.B, self.bucket_end = engine, n_seqs, bucket_end
        B = n_seqs
        self.layout = [("tokens", B), ("positions", B), ("slot_of_token", B), ("cu_seqlens", B + 1), ("slots", B),
                       ("start", B), ("want_rows", B)]
        total = sum(n for _, n in self.layout)
        self.host = torch.empty(total, dtype=torch.int32).pin_memory()
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(total, dtype=torch.int32, device=engine.device)
        self.views, o = {}, 0
        self.offsets = {}
        for name, n in self.layout:
            self.views[name] = self.dev[o:o + n]
            self.offsets[name] = (o, o + n)
            o += n
        a, b = self.offsets["cu_seqlens"]
        self.host_np[a:b] = np.arange(B + 1, dtype=np.int32)
        a, b = self.offsets["want_rows"]
        self.host_np[a:b] = np.arange(B, dtype=np.int32)
        self.copied = torch.cuda.Event()
        self.graph = torch.cuda.CUDAGraph()
        self.logits = None
        self.pool = pool

    def fill(self, slots, starts, tokens) -> None:
        """``tokens``: a list, or an int32 tensor on the device that is copied in behind the other arrays."""
        self.copied.synchronize()          # the last copy out of the pinned array has been done
        h, off = self.host_np, self.offsets
        on_device = isinstance(tokens, torch.Tensor)
        if not on_device:
            h[off["tokens"][0]:off["tokens"][1]] = tokens
        h[off["positions"][0]:off["positions"][1]] = starts
        h[off["slot_of_token"][0]:off["slot_of_token"][1]] = slots
        h[off["slots"][0]:off["slots"][1]] = slots
        h[off["start"][0]:off["start"][1]] = starts
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()
        if on_device:
            self.views["tokens"].copy_(tokens)

    def batch(self, slots, starts) -> StepBatch:
        v = self.views
        b = StepBatch(slots=list(slots), n_new=[1] * self.B, start=list(starts), n_tokens=self.B, tokens=v["tokens"],
                      positions=v["positions"], slot_of_token=v["slot_of_token"], cu_seqlens=v["cu_seqlens"],
                      slots_dev=v["slots"], start_dev=v["start"], want_rows=v["want_rows"], n_want=self.B)
        b.fixed_max_end = self.bucket_end
        return b

    def capture(self, slots, starts, tokens) -> torch.Tensor:
        self.fill(slots, starts, tokens)
        e = self.engine
        ctx = StepContext(batch=self.batch(slots, starts), cache=e.cache, act=e.model.act, device=e.device,
                          side_stream=e.side_stream, capturing=True, native=e.native)
        torch.cuda.synchronize()
        # Nothing may be destroyed on the device while the stream is capturing: an older graph that the garbage
        # collector happens to find in the middle of the capture would end the process.  So the collector rests
        # until the capture is over (a collection beforehand is not needed for that, and costs 20 ms).
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(self.graph, pool=self.pool):
                self.logits = e.model.forward(ctx)
        finally:
            if collecting:
                gc.enable()
        self.graph.replay()
        return self.logits

    def replay(self, slots, starts, tokens) -> torch.Tensor:
        self.fill(slots, starts, tokens)
        self.graph.replay()
        return self.logits


class DecodeGraphs:
    """The graphs of one engine, by (number of sequences, length bucket); the first step of a shape runs eagerly
    (kernels are loaded at their first launch, which must not happen under capture), the second is captured."""

    def __init__(self, engine, max_graphs: int = 24):
        self.engine, self.max_graphs = engine, max_graphs
        self.graphs: dict[tuple[int, int], DecodeGraph] = {}
        self.seen: set[tuple[int, int]] = set()
        self.pool = None
        self._replayable: dict[int, bool] = {}

    def replayable(self, n_seqs: int) -> bool:
        """Whether every part of the model lets a decode step of ``n_seqs`` sequences be captured."""
        if n_seqs not in self._replayable:
            self._replayable[n_seqs] = all(p.replayable(n_seqs) for p in self.engine.model.parts())
        return self._replayable[n_seqs]

    def key(self, n_seqs: int, max_end: int) -> tuple[int, int]:
        cap = self.engine.cache.max_positions
        return n_seqs, min(cap, -(-max_end // RUN_BUCKET) * RUN_BUCKET)

    def run(self, slots, starts, tokens):
        """Logits [B, vocab] of one decode step, or None if this shape has not been seen before or a part of the
        model does not let it be replayed."""
        if not self.replayable(len(slots)):
            return None
        key = self.key(len(slots), max(starts) + 1)
        g = self.graphs.get(key)
        if g is not None:
            return g.replay(slots, starts, tokens)
        if key not in self.seen:
            self.seen.add(key)
            return None
        if len(self.graphs) >= self.max_graphs:
            self.graphs.pop(next(iter(self.graphs)))
        if self.pool is None:
            self.pool = torch.cuda.graph_pool_handle()
        g = DecodeGraph(self.engine, key[0], key[1], self.pool)
        self.graphs[key] = g
        return g.capture(slots, starts, tokens)
