"""The step function: runs the next tokens of a batch of sequences, from the cache, and returns the logits
at the wanted places.

The reference steps one token of one sequence (``tq_forward``, /root/reference/src/engine/tq_transformer.c:2281)
and its multi-token path serves one sequence and no experts (``tq_forward_batch``, :3049-3083).  Here a
step takes any set of live sequences, each with its own next tokens (a whole prompt, or one decoded
token) and its own length; the tokens run as one packed batch without padding, every token at position
``length of its sequence + its place``, and afterwards the lengths have grown by what was run.
"""
from __future__ import annotations

import torch

from ..cache.paged import CacheError
from ..csrc import ops
from .batch import pack_step
from .context import StepContext
from .graph import DecodeGraphs
from .model import CausalLM
from .native import NativeModel


class StepError(ValueError):
    pass


class Engine:
    """A model with its cache.  ``max_tokens`` is the most positions that live sequences hold at once,
    each sequence rounded up to whole pages of ``page_size``."""

    def __init__(self, model: CausalLM, max_tokens: int, page_size: int = 64, max_slots: int | None = None,
                 use_graphs: bool = True, max_positions: int | None = None, window_step: int = 2048):
        """``max_positions``: the most positions one sequence may reach (default and upper bound: the model's).
        ``window_step``: layers that keep a window have pages for their windows and for this many new positions per
        sequence; a step that brings a sequence more is run in cuts of that length."""
        self.model = model
        self.cache = model.new_cache(max_tokens, page_size=page_size, max_slots=max_slots, max_positions=max_positions,
                                     window_step=window_step)
        self.device = model.device
        self.vocab_size = model.plan.vocab_size
        # decode steps are replayed as HIP graphs where a GPU runs them
        on_gpu = self.device is not None and self.device.type == "cuda"
        self.side_stream = torch.cuda.Stream(device=self.device) if on_gpu else None     # default priority
        # (which shapes of step are replayed is the parts' word, asked shape by shape: Part.replayable)
        self.graphs = DecodeGraphs(self) if use_graphs and on_gpu else None
        self.layer_hook = None      # see StepContext.layer_hook; while it is set, steps run eagerly
        # the model and this cache as the library's step executor takes them (None: steps run part by part from here)
        self.native = NativeModel.build(model, self.cache) if on_gpu else None

    # ------------------------------------------------------------ sequences
    def open(self, n: int = 1) -> list[int]:
        """Slots for ``n`` new sequences."""
        slots = []
        try:
            for _ in range(n):
                slots.append(self.cache.open())
        except CacheError:
            for s in slots:
                self.cache.close(s)
            raise
        return slots

    def close(self, slots) -> None:
        for s in slots:
            self.cache.close(s)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    # ------------------------------------------------------------ the step
    def step(self, slots: list[int], token_lists: list[list[int]], wants: list[list[int]] | None = None) -> torch.Tensor:
        """Runs ``token_lists[i]`` as the next tokens of the sequence in ``slots[i]``.

        ``wants[i]`` lists the places among those tokens whose logits are returned (default: the last).
        Returns float32 logits [number of wanted places, vocab] in the order of the sequences and of
        their wanted places."""
        if len(slots) != len(token_lists) or not slots:
            raise StepError("a step needs as many token lists as slots, and at least one")
        if len(set(slots)) != len(slots):
            raise StepError("a slot appears twice in one step")
        if wants is None:
            wants = [[len(t) - 1] for t in token_lists]
        if len(wants) != len(slots):
            raise StepError("a step needs as many lists of wanted places as slots")
        V = self.vocab_size
        for i, (toks, want) in enumerate(zip(token_lists, wants)):
            if len(toks) == 0:
                raise StepError(f"sequence {i} of the step brings no token")
            bad = [t for t in toks if not 0 <= t < V]
            if bad:
                raise StepError(f"sequence {i} brings token {bad[0]}, outside the vocabulary of {V}")
            bad = [w for w in want if not 0 <= w < len(toks)]
            if bad:
                raise StepError(f"wanted place {bad[0]} is outside the {len(toks)} tokens that sequence {i} brings")
        limit = self.cache.step_limit
        if limit is not None and max(len(t) for t in token_lists) > limit:
            return self._step_in_cuts(slots, token_lists, wants, limit)
        starts = self._reserve(slots, [len(t) for t in token_lists])
        try:
            logits = None
            if self.graphs is not None and self.layer_hook is None and all(len(t) == 1 for t in token_lists):
                all_rows = self.graphs.run(slots, starts, [t[0] for t in token_lists])
                if all_rows is not None:       # the graph gives every row; hand out a copy of the wanted ones
                    rows = [i for i, w in enumerate(wants) for _ in w]
                    logits = all_rows.clone() if rows == list(range(len(slots))) else \
                        all_rows[torch.tensor(rows, dtype=torch.int64, device=self.device)] if rows else \
                        torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
            if logits is None:
                logits = self._eager(pack_step(slots, starts, token_lists, wants, self.device))
        except BaseException:
            self._unreserve(slots)
            raise
        for slot in slots:
            self.cache.commit(slot)
        return logits

    def _step_in_cuts(self, slots, token_lists, wants, limit: int) -> torch.Tensor:
        """A step whose sequences bring more tokens than a group with a window has room for at once: cuts of
        ``limit`` tokens per sequence, one after the other (the logits at a position do not depend on how its
        sequence was cut).  Whether the whole step has room is looked at before the first cut runs."""
        self.cache.room_for(slots, [len(t) for t in token_lists])
        pieces, where = [], {}          # (sequence, place in its wants) -> (cut, row of that cut's logits)
        for cut in range(-(-max(len(t) for t in token_lists) // limit)):
            lo = cut * limit
            live = [i for i, t in enumerate(token_lists) if len(t) > lo]
            cut_wants, row = [], 0
            for i in live:
                mine = [(j, w - lo) for j, w in enumerate(wants[i]) if lo <= w < lo + limit]
                for j, _ in mine:
                    where[(i, j)] = (cut, row)
                    row += 1
                cut_wants.append([w for _, w in mine])
            pieces.append(self.step([slots[i] for i in live], [token_lists[i][lo:lo + limit] for i in live], cut_wants))
        order = [where[(i, j)] for i in range(len(slots)) for j in range(len(wants[i]))]
        if not order:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        offsets, total = [], 0
        for p in pieces:
            offsets.append(total)
            total += p.shape[0]
        rows = torch.tensor([offsets[c] + r for c, r in order], dtype=torch.int64, device=self.device)
        return torch.cat(pieces)[rows]

    def step_from_device(self, slots: list[int], tokens: torch.Tensor) -> torch.Tensor:
        """A decode step whose tokens are already on the device: ``tokens`` int32 [len(slots)], one for each
        sequence, each inside the vocabulary (as a sampler's output is; nothing checks it here).  The host
        need not have seen the tokens, so the step can be issued while the choice of these tokens is still
        running.  Returns the logits of every sequence, [len(slots), vocab]; they may live in memory that the
        next step of the same shape overwrites, so use them (or copy them) before that step is issued."""
        if not slots or len(set(slots)) != len(slots):
            raise StepError("a step needs at least one slot, and each only once")
        if tokens.dtype != torch.int32 or tuple(tokens.shape) != (len(slots),) or \
                (self.device is not None and tokens.device != torch.device(self.device)):
            raise StepError(f"tokens must be int32 [{len(slots)}] on the model's device")
        starts = self._reserve(slots, [1] * len(slots))
        try:
            logits = self.graphs.run(slots, starts, tokens) if self.graphs is not None and self.layer_hook is None else None
            if logits is None:
                batch = pack_step(slots, starts, [[0]] * len(slots), [[0]] * len(slots), self.device)
                batch.tokens.copy_(tokens)
                logits = self._eager(batch)
        except BaseException:
            self._unreserve(slots)
            raise
        for slot in slots:
            self.cache.commit(slot)
        return logits

    def _reserve(self, slots, counts) -> list[int]:
        """Room for ``counts[i]`` more positions in each slot, or none at all; returns where each sequence goes on."""
        starts, reserved = [], []
        try:
            for slot, n in zip(slots, counts):
                starts.append(self.cache.reserve(slot, n))
                reserved.append(slot)
        except CacheError:
            self._unreserve(reserved)
            raise
        self.cache.sync()
        return starts

    def _unreserve(self, slots) -> None:
        """A step that did not run: its positions do not count and the pages taken for them go back."""
        for slot in slots:
            self.cache.cancel(slot)
        self.cache.sync()

    def _eager(self, batch) -> torch.Tensor:
        # a second stream for what does not depend on the main line (the parts decide what they put there)
        ctx = StepContext(batch=batch, cache=self.cache, act=self.model.act, device=self.device,
                          side_stream=self.side_stream, layer_hook=self.layer_hook, native=self.native)
        with ops.own_products(max(batch.n_new) == 1):      # a decode step runs the kernels that its replay runs
            return self.model.forward(ctx)
