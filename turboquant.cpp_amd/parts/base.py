"""What every part of a layer has in common, and the registries parts are chosen from.

A part is built from a :class:`~..config.plan.PartSpec`: a kind (the registry key), arguments (its sizes
and constants) and the checkpoint tensors behind its parameters.  It declares its parameters with
:class:`ParamSpec`, receives them as device tensors, and does its work through the kernels in
``csrc.ops``.  A part never looks at the model or the architecture it is used in.

Interfaces (``ctx`` is the :class:`~..engine.context.StepContext` of the running step):

* norm      ``forward(x, delta, ctx, rows=None, want_f32=False) -> (normed, normed32)``: adds the pending
            ``delta`` [S, T, H] float32 into the residual stream ``x`` [T, H] float32 and returns the normalised
            rows in the activation type (and in float32 if asked).
* mixer     ``forward(normed, ctx, entry) -> delta``: mixes tokens of each sequence; ``entry`` is the index of
            the schedule entry that runs, by which it finds its cache (``ctx.kv(entry)``) or its fixed-size
            state (``ctx.state(entry)``; ``ctx.state_rows(entry)`` / ``ctx.store_state_rows(entry, rows)`` read and
            write the rows of the step's sequences through the slots on the device, which a decode step that is to
            be replayed must use).  ``cache_need()`` / ``state_need()`` say what storage each run wants.
* ffn       ``forward(normed, normed32, ctx) -> delta``; ``wants_f32`` says whether it reads the float32 copy.
* position  ``table(device)``, ``pairing``, ``rotary_dim``: the rotation a mixer applies to queries and keys.
* block     ``forward(x, pending, ctx, entry) -> pending``: the arrangement of norms, mixer and ffn around
            the residual stream.

``delta`` is float32 [S, T, H], S partial results that the next norm adds to the stream in order, or a
``csrc.ops.GatheredSum``: a weighted sum over rows of a matrix (the experts' outputs) that is left to the next
norm, whose ``materialize`` gives the tensor to an arrangement that needs it earlier.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable

import torch

from ..config.plan import PartSpec


@dataclass(frozen=True)
class ParamSpec:
    """One parameter: its shape, its role (``matrix``, ``bias``, ``scale`` for norm weights, ``table`` for
    embeddings, ``router`` for rows whose products are float32 arithmetic whatever the activation type) and, if it is several checkpoint tensors joined along dimension 0, their sizes there."""
    shape: tuple[int, ...]
    role: str = "matrix"
    splits: tuple[int, ...] | None = None


@dataclass(frozen=True)
class CacheNeed:
    """Keys and values per position: ``window`` None keeps all positions, else the last ``window``.
    ``head_dim`` is the width of a key row; ``value_dim`` that of a value row (None: the same; 0: no values are
    kept, one row per position and kv head only)."""
    num_kv_heads: int
    head_dim: int
    window: int | None = None
    value_dim: int | None = None

    @property
    def value_width(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class StateNeed:
    """State of fixed size per sequence, zero when a sequence starts."""
    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Part:
    category: str = ""
    kind: str = ""
    # True if forward(), in a decode step (one token per sequence), reads what changes from step to step (tokens,
    # positions, slots, lengths) from the batch's device arrays only and launches nothing that a stream capture
    # cannot record, so that a captured launch sequence can be replayed for other sequences.
    graph_safe: bool = False

    def replayable(self, n_seqs: int) -> bool:
        """Whether a decode step of ``n_seqs`` sequences may be captured and replayed as far as this part goes.  The
        engine asks every part before it captures a step of a shape; one that says no makes steps of that shape run
        eagerly, others are still replayed."""
        return self.graph_safe

    def param_specs(self) -> dict[str, ParamSpec]:
        return {}

    def children(self) -> dict[str, "Part"]:
        return {}

    def set_params(self, tensors: dict[str, torch.Tensor]) -> None:
        for name, t in tensors.items():
            setattr(self, name, t)

    def prepare(self, device, act: str) -> None:
        """Called once after the parameters are on the device."""

    def native(self):
        """The part's description for the step executor (a structure of ``csrc.host_api``: its sizes, constants and the
        addresses of its parameters), or None if the executor has no form of this part.  A model whose layers all have
        one is stepped by one call into the executor; any other is stepped part by part through ``forward``."""
        return None


_REGISTRIES: dict[str, dict[str, Callable[..., Part]]] = {
    "norm": {}, "mixer": {}, "ffn": {}, "position": {}, "block": {},
}


def register_part(category: str, kind: str):
    """Class decorator: makes a part available to model plans under ``kind``."""
    if category not in _REGISTRIES:
        raise ValueError(f"unknown part category {category!r}; known: {sorted(_REGISTRIES)}")

    def deco(cls):
        if kind in _REGISTRIES[category]:
            raise ValueError(f"{category} {kind!r} is already registered")
        cls.category, cls.kind = category, kind
        _REGISTRIES[category][kind] = cls
        return cls
    return deco


def unregister_part(category: str, kind: str) -> None:
    _REGISTRIES[category].pop(kind, None)


def known_parts(category: str) -> list[str]:
    return sorted(_REGISTRIES[category])


def build_part(category: str, spec: PartSpec) -> Part:
    try:
        cls = _REGISTRIES[category][spec.kind]
    except KeyError:
        raise ValueError(f"unknown {category} {spec.kind!r}; known: {', '.join(known_parts(category))}") from None
    args: dict[str, Any] = dict(spec.args)
    return cls(**args)
