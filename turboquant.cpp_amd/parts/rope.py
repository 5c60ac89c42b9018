"""Rotary position encoding: the table of angles per pair and how pairs are formed.

``freq_i = 1 / theta^(2i / rotary_dim)`` evaluated in float32 as the reference does
(``1.0f / powf(base, 2.0f * i / head_dim)``, /root/reference/src/engine/tq_ops.c:1418-1448); the angle of
pair i at position p is ``p * freq_i`` in float32.  ``pairing`` says which two dimensions form pair i:
``"half"`` pairs (i, i + rotary_dim/2) (/root/reference/src/engine/tq_transformer.c:1263-1289), the layout of
un-permuted checkpoints (/root/reference/docs/supported_models.md:99-108); ``"interleaved"`` pairs
(2i, 2i+1) as ``tq_rope`` does.  Dimensions from ``rotary_dim`` on are not rotated.

A mixer asks a position part for three things only: ``table(device)`` (float32 [rotary_dim/2] angles
per position step), ``pairing_code`` and ``rotary_dim``.  Another encoding that rotates pairs (scaled,
partial, with per-pair factors) is another table.
"""
from __future__ import annotations

import numpy as np
import torch

from .base import Part, register_part

PAIRINGS = {"half": 0, "interleaved": 1}


@register_part("position", "rope")
class RotaryEncoding(Part):
    graph_safe = True
    def __init__(self, head_dim: int, rotary_dim: int, theta: float, pairing: str = "half"):
        if pairing not in PAIRINGS:
            raise ValueError(f"unknown pairing {pairing!r}; known: {sorted(PAIRINGS)}")
        if rotary_dim % 2 or not 0 <= rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {rotary_dim} must be even and at most head_dim {head_dim}")
        self.head_dim, self.rotary_dim, self.theta, self.pairing = head_dim, rotary_dim, theta, pairing
        self._table = None

    @property
    def pairing_code(self) -> int:
        return PAIRINGS[self.pairing]

    def frequencies(self) -> np.ndarray:
        i = np.arange(self.rotary_dim // 2, dtype=np.float32)
        expo = (np.float32(2.0) * i) / np.float32(self.rotary_dim)
        return (np.float32(1.0) / np.power(np.float32(self.theta), expo, dtype=np.float32)).astype(np.float32)

    def table(self, device) -> torch.Tensor:
        if self._table is None or self._table.device != torch.device(device):
            self._table = torch.from_numpy(self.frequencies()).to(device)
        return self._table

    def prepare(self, device, act):
        self.table(device)
