"""A model's plan as a text file that a host without Python reads.

The reference's C host gets everything it needs to know about a model from the model file's own metadata
(/root/reference/src/engine/tq_model.c:2867-2921).  A host in C that drives the step executor (``csrc/host/quant_main.cpp``)
is told the same by this file: for every layer the kinds of its parts with their sizes and constants, which checkpoint
tensors make up each parameter and how they are joined, the table of rotation angles, and the order in which layers run.
It is written from the model's plan by the same code that builds the model here, so an architecture is still described
in one place (its module under ``models/``); the file holds no weights.

Format: lines of words separated by blanks, ``key=value`` for sizes and constants.

    tqplan 1
    model <architecture> act=<float32|bfloat16> vocab=.. hidden=.. n_layers=.. n_entries=.. embedding_scale=.. logit_softcap=.. max_positions=..
    stop <n> <ids...>
    param -1 model <attribute> <role> <single|stack|concat> <ndim> <dims...> <n names> <names...>
    layer <i> <block kind>
    part <i> <slot> <kind> key=value ...            (slot: mixer_norm, mixer, ffn_norm, ffn, final_norm with layer -1)
    table <i> <slot> inv_freq <n> <float32 bits as hex...>
    param <i> <slot> <attribute> <role> <how> <ndim> <dims...> <n names> <names...>
    entry <e> layer=<l> cache_of=<e' or -1>
"""
from __future__ import annotations

import struct

from ..parts.base import Part
from ..weights.loader import Binding


def _value(v) -> str:
    if isinstance(v, bool):
        return "1" if v else "0"
    if isinstance(v, float):
        return repr(v)
    return str(v)


def _part_line(layer: int, slot: str, part: Part) -> str:
    """A part's constructor arguments that are numbers, flags or names (a nested part is written on a line of its own)."""
    words = [f"part {layer} {slot} {part.kind}"]
    for key, val in sorted(vars(part).items()):
        if key.startswith("_") or val is None or isinstance(val, Part) or hasattr(val, "shape"):
            continue        # (a constant that is None is left out: no window, no norm of the heads)
        if isinstance(val, (bool, int, float, str)):
            words.append(f"{key}={_value(val)}")
    return " ".join(words)


def _param_line(layer: int, slot: str, b: Binding) -> str:
    shape = tuple(b.spec.shape)
    if b.source.how == "concat":
        extra = " splits " + " ".join(str(n) for n in b.spec.splits)
    else:
        extra = ""
    return (f"param {layer} {slot} {b.attr} {b.spec.role} {b.source.how} {len(shape)} " + " ".join(str(d) for d in shape)
            + f" {len(b.source.names)} " + " ".join(b.source.names) + extra)


def plan_text(model) -> str:
    """The plan file of a ``CausalLM`` (its weights need not be loaded)."""
    plan = model.plan
    lines = ["tqplan 1",
             f"model {plan.architecture} act={model.act} vocab={plan.vocab_size} hidden={plan.hidden_size} "
             f"n_layers={len(model.blocks)} n_entries={len(model.schedule)} embedding_scale={plan.embedding_scale!r} "
             f"logit_softcap={plan.logit_softcap or 0.0!r} max_positions={plan.max_positions}",
             "stop " + " ".join(str(t) for t in (len(plan.stop_tokens),) + tuple(plan.stop_tokens))]
    by_owner: dict[int, list[Binding]] = {}
    for b in model.bindings:
        by_owner.setdefault(id(b.owner), []).append(b)
    for b in by_owner.get(id(model), []):
        lines.append(_param_line(-1, "model", b))
    if plan.lm_head is None:
        lines.append("tied -1 model lm_head embedding")

    def write_part(layer: int, slot: str, part: Part) -> None:
        lines.append(_part_line(layer, slot, part))
        for b in by_owner.get(id(part), []):
            lines.append(_param_line(layer, slot, b))
        for name, child in part.children().items():
            if hasattr(child, "frequencies") and hasattr(child, "pairing_code"):
                lines.append(f"part {layer} {slot}.{name} {child.kind} pairing_code={child.pairing_code} rotary_dim={child.rotary_dim}")
                bits = struct.unpack(f"<{child.rotary_dim // 2}I", child.frequencies().astype("<f4").tobytes())
                lines.append(f"table {layer} {slot} inv_freq {len(bits)} " + " ".join(f"{x:08x}" for x in bits))

    for i, block in enumerate(model.blocks):
        lines.append(f"layer {i} {block.kind}")
        for slot in block.slots:
            write_part(i, slot, getattr(block, slot))
    write_part(-1, "final_norm", model.final_norm)
    for e, entry in enumerate(model.schedule):
        lines.append(f"entry {e} layer={entry.layer} cache_of={-1 if entry.cache_of is None else entry.cache_of}")
    return "\n".join(lines) + "\n"


def write_plan_file(model, path: str) -> str:
    with open(path, "w", encoding="utf-8") as f:
        f.write(plan_text(model))
    return path
