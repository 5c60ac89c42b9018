"""RMS norm fused with the sum into the residual stream.

``out = (v * (1 / sqrt(mean(v^2) + eps))) * weight`` with ``v = x + pending``, everything in float32
(/root/reference/src/engine/tq_ops.c:1373-1410; a plain weight, no ``+1``).
"""
from __future__ import annotations

from ..csrc import ops
from .base import ParamSpec, Part, register_part


@register_part("norm", "rmsnorm")
class RMSNorm(Part):
    graph_safe = True
    def __init__(self, size: int, eps: float):
        self.size, self.eps = size, eps
        self.weight = None

    def param_specs(self):
        return {"weight": ParamSpec((self.size,), role="scale")}

    def native(self):
        from ..csrc import host_api
        return host_api.NormDesc(host_api.weight(self.weight), self.eps)

    def forward(self, x, delta, ctx, rows=None, want_act=True, want_f32=False):
        return ops.add_rmsnorm(x, delta, self.weight, self.eps, ctx.act, rows=rows, want_act=want_act,
                               want_f32=want_f32)
