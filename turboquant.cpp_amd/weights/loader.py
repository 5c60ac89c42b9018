"""From checkpoint tensors, by name, to the parameters of a model's parts.

In the manner of the reference's loader (/root/reference/src/engine/tq_model.c:847-1666): tensors are looked up
by name (:324-360) and converted as they are placed (:367-412, :440-451): on the bfloat16 path bfloat16 stays
bfloat16, and of the tensors that the checkpoint stores in 32 bits the matrices of the products and the embedding
table are rounded to bfloat16 once, here (with a warning that counts them), while norm weights, biases and the
router's rows, which feed float32 arithmetic, stay in 32 bits; ``f32_matrices="keep"`` leaves every 32-bit tensor
as it is stored, and the products of those matrices then run the plain multiply-add kernel.  Unlike it, a
tensor that is not there is never a silent NULL (tq_model.c:418-423): everything is checked before
anything is copied, and one error lists all missing tensors, all wrong shapes and, beside them, the tensors
that the model does not read.  A checkpoint whose only difference is such extra tensors (a stray buffer) loads,
with a warning that names them.
Experts stored one tensor each are stacked, and q, k, v are joined, as the plan's sources say.
"""
from __future__ import annotations

import warnings
from dataclasses import dataclass

import torch

from ..config.plan import Source
from ..parts.base import ParamSpec


class WeightError(ValueError):
    """Checkpoint and model do not fit; the message lists every difference."""

    def __init__(self, missing, unexpected, wrong_shape, other=()):
        self.missing, self.unexpected, self.wrong_shape, self.other = list(missing), list(unexpected), list(wrong_shape), list(other)
        lines = ["checkpoint does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing[:20]) + (" ..." if len(self.missing) > 20 else ""))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected[:20]) + (" ..." if len(self.unexpected) > 20 else ""))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n} is {tuple(got)}, model wants {tuple(want)}" for n, got, want in self.wrong_shape[:20]) + (" ..." if len(self.wrong_shape) > 20 else ""))
        for o in self.other:
            lines.append("  " + o)
        super().__init__("\n".join(lines))


class UnexpectedTensors(UserWarning):
    """The checkpoint holds tensors that the model does not read."""


class RoundedWeights(UserWarning):
    """Matrices that the checkpoint stores in 32 bits were rounded to bfloat16 as they were placed."""


class SlowWeights(UserWarning):
    """Matrices were kept in 32 bits on the bfloat16 path: their products do not run on the matrix cores."""


F32_MATRICES = ("bfloat16", "keep")
ROUNDED_ROLES = ("matrix", "table")      # what feeds bfloat16 products; scale, bias and router feed float32 arithmetic


@dataclass
class Binding:
    """One parameter of one part and the checkpoint tensors behind it."""
    owner: object
    attr: str
    spec: ParamSpec
    source: Source
    path: str           # where the parameter sits in the model, for messages

    def pieces(self) -> list[tuple[str, tuple[int, ...]]]:
        """(checkpoint name, shape) of every tensor this parameter is made of."""
        shape = tuple(self.spec.shape)
        if self.source.how == "single":
            return [(self.source.names[0], shape)]
        if self.source.how == "stack":
            if len(self.source.names) != shape[0]:
                raise ValueError(f"{self.path}: {len(self.source.names)} tensors are stacked into a leading size of {shape[0]}")
            return [(n, shape[1:]) for n in self.source.names]
        if self.source.how == "concat":
            splits = self.spec.splits
            if splits is None or len(splits) != len(self.source.names) or sum(splits) != shape[0]:
                raise ValueError(f"{self.path}: joined sources need sizes that add up to {shape[0]}")
            return [(n, (s, *shape[1:])) for n, s in zip(self.source.names, splits)]
        raise ValueError(f"{self.path}: unknown source kind {self.source.how!r}")


def expected_tensors(bindings: list[Binding]) -> dict[str, tuple[tuple[int, ...], str]]:
    """name -> (shape, role) of every checkpoint tensor the model reads."""
    out: dict[str, tuple[tuple[int, ...], str]] = {}
    for b in bindings:
        for name, shape in b.pieces():
            if name in out and out[name][0] != tuple(shape):
                raise ValueError(f"tensor {name!r} is wanted with two shapes: {out[name][0]} and {tuple(shape)}")
            out[name] = (tuple(shape), b.spec.role)
    return out


def check(bindings: list[Binding], available: dict[str, tuple[tuple[int, ...], torch.dtype]]) -> None:
    want = expected_tensors(bindings)
    missing = [n for n in want if n not in available]
    unexpected = [n for n in available if n not in want]
    wrong = [(n, available[n][0], want[n][0]) for n in want if n in available and tuple(available[n][0]) != want[n][0]]
    other = [f"tensor {n} has type {available[n][1]}, which no kernel takes" for n in want
             if n in available and available[n][1] not in (torch.float32, torch.bfloat16, torch.float16, torch.int32, torch.int64)]
    if missing or wrong or other:
        raise WeightError(missing, unexpected, wrong, other)
    if unexpected:
        warnings.warn(f"checkpoint holds {len(unexpected)} tensors that the model does not read: "
                      + ", ".join(unexpected[:20]) + (" ..." if len(unexpected) > 20 else ""), UnexpectedTensors,
                      stacklevel=3)


def stored_dtype(dtypes: list[torch.dtype], act: str, role: str = "scale", f32_matrices: str = "keep") -> torch.dtype:
    """The type a parameter is kept in: float32 on the 32-bit path; else bfloat16, but a tensor that the
    checkpoint stores in 32 bits stays so unless it is a matrix of a product or the embedding table and
    ``f32_matrices`` is "bfloat16"; integer tables are int32."""
    if any(d in (torch.int32, torch.int64) for d in dtypes):
        return torch.int32
    if act == "float32":
        return torch.float32
    if any(d == torch.float32 for d in dtypes) and not (f32_matrices == "bfloat16" and role in ROUNDED_ROLES):
        return torch.float32
    return torch.bfloat16


def load_bindings(bindings: list[Binding], reader, act: str, device, f32_matrices: str = "bfloat16") -> int:
    """Checks all names and shapes, then fills every parameter on the device.  ``reader`` has
    ``entries`` (name -> object with .shape and .dtype name) and ``read(name)``.  Returns bytes placed."""
    from .safetensors_io import DTYPES
    if f32_matrices not in F32_MATRICES:
        raise ValueError(f"f32_matrices must be one of {F32_MATRICES}, got {f32_matrices!r}")
    available = {n: (tuple(e.shape), DTYPES[e.dtype][0]) for n, e in reader.entries.items()}
    check(bindings, available)
    placed = 0
    rounded = kept = 0
    for b in bindings:
        pieces = b.pieces()
        stored = [available[n][1] for n, _ in pieces]
        dtype = stored_dtype(stored, act, b.spec.role, f32_matrices)
        if act != "float32" and b.spec.role in ROUNDED_ROLES and torch.float32 in stored:
            rounded += dtype == torch.bfloat16
            kept += dtype == torch.float32
        dst = torch.empty(tuple(b.spec.shape), dtype=dtype, device=device)
        if b.source.how == "single":
            dst.copy_(reader.read(pieces[0][0]).to(dtype))
        elif b.source.how == "stack":
            for i, (n, _) in enumerate(pieces):
                dst[i].copy_(reader.read(n).to(dtype))
        else:
            o = 0
            for n, shape in pieces:
                dst[o:o + shape[0]].copy_(reader.read(n).to(dtype))
                o += shape[0]
        setattr(b.owner, b.attr, dst)
        placed += dst.numel() * dst.element_size()
    if rounded:
        warnings.warn(f"{rounded} matrices that the checkpoint stores in 32 bits were rounded to bfloat16 as they were "
                      "placed (f32_matrices=\"keep\" leaves them as they are stored)", RoundedWeights, stacklevel=3)
    if kept:
        warnings.warn(f"{kept} matrices stay in 32 bits on the bfloat16 path: their products run the plain multiply-add "
                      "kernel, not the matrix cores", SlowWeights, stacklevel=3)
    return placed


class TensorDict:
    """Tensors in memory with the reading interface of a safetensors folder."""

    @dataclass
    class _Entry:
        shape: tuple[int, ...]
        dtype: str

    def __init__(self, tensors: dict[str, torch.Tensor]):
        from .safetensors_io import NAMES
        self.tensors = tensors
        self.entries = {n: TensorDict._Entry(tuple(t.shape), NAMES[t.dtype]) for n, t in tensors.items()}

    def read(self, name: str) -> torch.Tensor:
        return self.tensors[name]
