"""The reference's random numbers: xorshift64* to a float in [0, 1)
(/root/reference/src/engine/tq_generate.c:53-58); seed 0 stands for 42 (:407)."""
from __future__ import annotations

_MASK = (1 << 64) - 1


class XorShift64Star:
    def __init__(self, seed: int):
        self.state = (seed & _MASK) or 42

    def next_float(self) -> float:
        s = self.state
        s ^= s >> 12
        s ^= (s << 25) & _MASK
        s ^= s >> 27
        self.state = s
        return float(((s * 0x2545F4914F6CDD1D) & _MASK) >> 33) / float(1 << 31)


def stream_seed(seed: int, index: int) -> int:
    """Seed of the ``index``-th sequence of a call: sequence 0 draws exactly what a single request would."""
    base = (seed & _MASK) or 42
    if index == 0:
        return base
    return (base ^ (index * 0x9E3779B97F4A7C15)) & _MASK or 42
