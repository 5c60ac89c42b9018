"""The generation loop: batches of prompts of unequal length, stop tokens, sequences that end early.

The reference's loop serves one prompt (/root/reference/src/engine/tq_generate.c:167-643): prefill, sample;
then, while fewer than ``max_tokens`` tokens are out: stop on an end token (:426-446) without emitting it,
emit, run the token, apply the repetition penalty, sample, and stop when the same 4-gram has come three
times (:611-629).  Here the same decisions are taken per sequence of a batch: all prompts of a batch run
in one step, then every live sequence decodes one token per step; a sequence that ends gives its slot
and pages back at once and the others go on; when more requests wait than a batch holds, batch follows
batch.  Where the reference shifts a full context (:456-514), a sequence here ends with reason ``"context"``:
when it reaches the positions a sequence may hold, and also when the cache's pages run out while several
sequences grow (the longest of those that need a page ends, its pages let the others go on); a prompt that
finds no room beside the others of its batch waits for the next batch.  The decisions are kept apart from
the device work (``SequenceTrack``) so that they are tested without one.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Sequence

import torch

from ..cache.paged import CacheFull
from ..sampling.sampler import Sampler, SamplingOptions, TokenFetch


@dataclass
class GenerationOptions:
    max_tokens: int = 256                     # reference default (tq_ops.c:1883-1897)
    temperature: float = 0.7
    top_p: float = 0.9
    seed: int = 42
    rep_penalty: float = 1.1
    rep_window: int = 32
    stop_tokens: tuple[int, ...] = ()
    loop_detection: bool = True               # stop when a 4-gram has repeated three times
    max_batch: int = 8
    on_token: Callable[[int, int], None] | None = None   # (request index, token)

    def sampling(self) -> SamplingOptions:
        return SamplingOptions(self.temperature, self.top_p, self.seed, self.rep_penalty, self.rep_window)


@dataclass
class GenerationResult:
    tokens: list[int]
    finish_reason: str            # "stop" (end token), "length" (max_tokens), "context" (cache or model limit), "loop"
    cached_positions: int = 0     # positions the cache held for the sequence when it ended (a token that ended it was not run)
    pages_held: tuple = ()        # pages it held then, per cache group (a group with a window has given the older ones back)


class LoopDetector:
    """Hash of the last four tokens kept in a ring of 64; three earlier occurrences end the sequence
    (/root/reference/src/engine/tq_generate.c:611-629)."""

    def __init__(self):
        self.hashes: list[int] = []
        self.count = 0

    def push(self, recent: Sequence[int]) -> bool:
        if len(recent) < 4:
            return False
        h = 0
        for t in recent[-4:]:
            h = (h * 31 + t) & 0xFFFFFFFF
        ring = self.hashes[:64]
        matches = sum(1 for x in ring if x == h)
        if len(self.hashes) < 64:
            self.hashes.append(h)
        else:
            self.hashes[self.count % 64] = h
        self.count += 1
        return matches >= 3


@dataclass
class SequenceTrack:
    """The decisions for one sequence: what to do with each sampled token."""
    request: int
    prompt_len: int
    options: GenerationOptions
    max_positions: int
    out: list[int] = field(default_factory=list)
    # the last tokens of the prompt (as many as the repetition window, tq_generate.c:381-384) and every sampled
    # token: what the loop detector hashes its 4-grams from
    history: list[int] = field(default_factory=list)
    detector: LoopDetector = field(default_factory=LoopDetector)
    finish_reason: str | None = None
    n_sampled: int = 0

    @classmethod
    def start(cls, request: int, prompt: Sequence[int], options: GenerationOptions, max_positions: int) -> "SequenceTrack":
        window = max(0, min(options.rep_window, 128))
        return cls(request, len(prompt), options, max_positions, history=list(prompt[-window:]) if window else [])

    def room_after_next(self) -> bool:
        """Whether the sequence can go on after its next token, as far as that does not depend on the token:
        neither the number of tokens asked for nor the positions are used up by it."""
        return len(self.out) + 1 < self.options.max_tokens and self.prompt_len + len(self.out) + 1 < self.max_positions

    def accept(self, token: int) -> bool:
        """Takes the sampled token.  Returns True if the token is to be run through the model next,
        False if the sequence has ended (``finish_reason`` says why)."""
        o = self.options
        self.history.append(token)
        del self.history[:-128]
        self.n_sampled += 1
        # the reference looks for a loop right after it has sampled a token in its loop, not after the first
        # token, which it samples before the loop (tq_generate.c:403-410, :603-629); the token that closes a loop
        # is not emitted
        if o.loop_detection and self.n_sampled > 1 and self.detector.push(self.history):
            self.finish_reason = "loop"
            return False
        if token in o.stop_tokens:
            self.finish_reason = "stop"          # the end token is not emitted
            return False
        self.out.append(token)
        if o.on_token is not None:
            o.on_token(self.request, token)
        if len(self.out) >= o.max_tokens:
            self.finish_reason = "length"
            return False
        if self.prompt_len + len(self.out) >= self.max_positions:
            self.finish_reason = "context"       # no room for another position; the reference would shift (:456-514)
            return False
        return True


def plan_batches(n_requests: int, max_batch: int) -> list[list[int]]:
    """Requests in order, ``max_batch`` at a time."""
    if max_batch < 1:
        raise ValueError("max_batch must be at least 1")
    return [list(range(i, min(i + max_batch, n_requests))) for i in range(0, n_requests, max_batch)]


def generate(engine, prompts: Sequence[Sequence[int]], options: GenerationOptions | None = None) -> list[GenerationResult]:
    """Generates a continuation for every prompt (lists of token ids)."""
    o = options or GenerationOptions()
    if any(len(p) == 0 for p in prompts):
        raise ValueError("every prompt needs at least one token")
    if o.max_batch < 1:
        raise ValueError("max_batch must be at least 1")
    if o.max_tokens < 1:
        return [GenerationResult([], "length") for _ in prompts]
    sampler = Sampler(o.sampling(), engine.model.act, engine.device)
    results: list[GenerationResult | None] = [None] * len(prompts)
    max_pos = engine.cache.max_positions
    waiting = deque(range(len(prompts)))

    def end(r, tracks, slot_of, reason=None):
        if reason is not None:
            tracks[r].finish_reason = reason
        slot = slot_of.pop(r)
        held = tuple(int((g.host_table[slot] >= 0).sum()) for g in engine.cache.groups)
        results[r] = GenerationResult(tracks[r].out, tracks[r].finish_reason, engine.length(slot), held)
        engine.close([slot])

    while waiting:
        batch = []
        room = min(o.max_batch, engine.cache.n_free_slots)
        if room < 1:
            raise CacheFull("no slot is free to start a batch with")
        while waiting and len(batch) < room:
            r = waiting.popleft()
            if len(prompts[r]) > max_pos:
                results[r] = GenerationResult([], "context")
            else:
                batch.append(r)
        if not batch:
            continue
        slots = engine.open(len(batch))
        tracks = {r: SequenceTrack.start(r, prompts[r], o, max_pos) for r in batch}
        samp = {r: sampler.new_sequence(r, list(prompts[r])) for r in batch}
        slot_of = dict(zip(batch, slots))
        live = list(batch)
        fetch = TokenFetch(engine.device, len(batch))
        try:
            logits = None
            while live:
                try:
                    logits = engine.step([slot_of[r] for r in live], [list(prompts[r]) for r in live])
                    break
                except CacheFull:
                    # the prompts of this batch do not fit into the cache together: the last one waits for the
                    # next batch; a prompt that does not even fit alone has no room at all
                    r = live.pop()
                    if live:
                        engine.close([slot_of.pop(r)])
                        waiting.appendleft(r)
                    else:
                        end(r, tracks, slot_of, "context")
            while live:
                states = [samp[r] for r in live]
                ids = sampler.launch(logits, states)
                fetch.start(ids)
                # The next step is issued before the host has seen these tokens, for every sequence that can
                # go on whatever its token is; the host then reads the tokens while that step runs.  A sequence
                # that ends on this token (an end token, a loop) has run one step in vain.
                ahead = [i for i, r in enumerate(live) if tracks[r].room_after_next()]
                next_logits = None
                if ahead:
                    feed = ids if len(ahead) == len(live) else ids[torch.tensor(ahead, dtype=torch.int64, device=ids.device)]
                    try:
                        next_logits = engine.step_from_device([slot_of[live[i]] for i in ahead], feed)
                    except CacheFull:
                        # no page to run ahead with: a sequence that ends on this token may give one back, so the
                        # step waits for the tokens this once
                        ahead = []
                tokens = fetch.wait()
                sampler.finish(tokens, states)
                going = []
                for i, (r, t) in enumerate(zip(live, tokens)):
                    if tracks[r].accept(t):
                        going.append(i)
                    else:
                        end(r, tracks, slot_of)
                if going and not ahead:
                    while going:
                        try:
                            logits = engine.step([slot_of[live[i]] for i in going], [[tokens[i]] for i in going])
                            break
                        except CacheFull:
                            # the pages have run out: of the sequences that need one, the longest ends here, and
                            # what it held lets the others go on
                            needy = [i for i in going if engine.cache.needs_page(slot_of[live[i]], 1)]
                            i = max(needy or going, key=lambda i: engine.length(slot_of[live[i]]))
                            going.remove(i)
                            end(live[i], tracks, slot_of, "context")
                elif going:
                    rows = [ahead.index(i) for i in going]       # a sequence that goes on was run ahead
                    logits = next_logits if rows == list(range(len(ahead))) else \
                        next_logits[torch.tensor(rows, dtype=torch.int64, device=next_logits.device)]
                live = [live[i] for i in going]
        finally:
            engine.close(list(slot_of.values()))
    return results


def continue_in_slot(engine, slot: int, history: Sequence[int], options: GenerationOptions | None = None) -> GenerationResult:
    """One sequence that outlives the call, as the reference's chat keeps its state between turns
    (/root/reference/quant.h:17634-17700): ``history`` is everything the sequence has seen and is to see, the slot's
    cache holds its first ``engine.length(slot)`` tokens (fewer than all of them), the rest is run as one prompt step
    and a continuation is generated.  The slot stays open; afterwards its cache holds the history and the generated
    tokens but the last, if that one ended the turn by its number (``engine.length(slot)`` says how many)."""
    o = options or GenerationOptions()
    cached = engine.length(slot)
    if not 0 <= cached < len(history):
        raise ValueError(f"the cache holds {cached} tokens, the history {len(history)}: at least one must be new")
    max_pos = engine.cache.max_positions
    if len(history) > max_pos:
        return GenerationResult([], "context")
    if o.max_tokens < 1:
        return GenerationResult([], "length")
    sampler = Sampler(o.sampling(), engine.model.act, engine.device)
    track = SequenceTrack.start(0, history, o, max_pos)
    state = sampler.new_sequence(0, list(history))
    fetch = TokenFetch(engine.device, 1)
    try:
        logits = engine.step([slot], [list(history[cached:])])
    except CacheFull:
        return GenerationResult([], "context")
    while True:
        ids = sampler.launch(logits, [state])
        fetch.start(ids)
        tokens = fetch.wait()
        sampler.finish(tokens, [state])
        if not track.accept(tokens[0]):
            break
        try:
            logits = engine.step([slot], [[tokens[0]]])
        except CacheFull:
            track.finish_reason = "context"
            break
    return GenerationResult(track.out, track.finish_reason)
