"""Arrangement of a layer's parts around the residual stream.

Pre-norm with two residual sums, ``x += mixer(norm(x)); x += ffn(norm(x))``
(/root/reference/src/engine/tq_transformer.c:2494,2531,2685-2701).  The sums are not done here: a part's
output travels as ``pending`` to the next norm, which adds it into the stream in float32 in the same
pass that normalises.
"""
from __future__ import annotations

from .base import Part, register_part


@register_part("block", "prenorm")
class PreNormBlock(Part):
    graph_safe = True
    # the parts a layer of this arrangement is made of, and the registry each comes from
    slots = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "ffn": "ffn"}

    def __init__(self, mixer_norm, mixer, ffn_norm, ffn):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def children(self):
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "ffn_norm": self.ffn_norm, "ffn": self.ffn}

    def cache_need(self):
        return self.mixer.cache_need()

    def state_need(self):
        return self.mixer.state_need()

    def native(self):
        from ..csrc import host_api
        norm1, mixer, norm2, ffn = (p.native() for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn))
        if not (isinstance(norm1, host_api.NormDesc) and isinstance(mixer, host_api.AttentionDesc)
                and isinstance(norm2, host_api.NormDesc) and isinstance(ffn, (host_api.DenseFfnDesc, host_api.MoeFfnDesc))):
            return None
        layer = host_api.LayerDesc()
        layer.mixer_norm, layer.attention, layer.ffn_norm = norm1, mixer, norm2
        if isinstance(ffn, host_api.DenseFfnDesc):
            layer.ffn_kind, layer.dense = host_api.FFN_DENSE, ffn
        else:
            layer.ffn_kind, layer.moe = host_api.FFN_MOE, ffn
        return layer

    def forward(self, x, pending, ctx, entry):
        normed, _ = self.mixer_norm.forward(x, pending, ctx)
        pending = self.mixer.forward(normed, ctx, entry)
        want32 = getattr(self.ffn, "wants_f32", False)
        normed, normed32 = self.ffn_norm.forward(x, pending, ctx, want_f32=want32)
        return self.ffn.forward(normed, normed32, ctx)
