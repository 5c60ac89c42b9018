"""Grouped-query attention over the paged cache.

In the reference's order (/root/reference/src/engine/tq_transformer.c:934-2269, Qwen2 path):
q, k, v = W x (+ bias) (:1031-1093); rotation of q and k (:1342-1344); k and v written at the token's
position (:1363-1371, :1451-1455); per head, scores of the positions in reach scaled by 1/sqrt(head_dim),
softmax, weighted sum of values (:1908-1976); output projection (:2239-2240).  Query head h reads
kv head h / (heads / kv_heads) (:1675-1679).  With a window a token reaches the last ``window``
positions, itself included (:1646-1654).  With ``qk_norm_eps`` set, every head of q and of k is RMS-normed with
weights of its own between the product and the rotation (:1111-1124), which this architecture does not use.
"""
from __future__ import annotations

import math

import torch

from ..config.plan import PartSpec
from ..csrc import ops
from .base import CacheNeed, ParamSpec, Part, build_part, register_part


@register_part("mixer", "gqa_attention")
class GroupedQueryAttention(Part):
    graph_safe = True
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, position,
                 qkv_bias: bool = False, out_bias: bool = False, window: int | None = None,
                 scale: float | None = None, qk_norm_eps: float | None = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        if window is not None and window < 1:
            raise ValueError(f"window must be positive, got {window}")
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.has_qkv_bias, self.has_out_bias, self.window = qkv_bias, out_bias, window
        self.qk_norm_eps = qk_norm_eps
        self.q_norm = self.k_norm = None
        self.scale = scale if scale is not None else 1.0 / math.sqrt(head_dim)
        self.position = build_part("position", position) if isinstance(position, PartSpec) else position
        self.qkv_weight = self.qkv_bias = self.out_weight = self.out_bias = None

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def param_specs(self):
        rows = self.q_size + 2 * self.kv_size
        splits = (self.q_size, self.kv_size, self.kv_size)
        specs = {
            "qkv_weight": ParamSpec((rows, self.hidden_size), splits=splits),
            "out_weight": ParamSpec((self.hidden_size, self.q_size)),
        }
        if self.has_qkv_bias:
            specs["qkv_bias"] = ParamSpec((rows,), role="bias", splits=splits)
        if self.has_out_bias:
            specs["out_bias"] = ParamSpec((self.hidden_size,), role="bias")
        if self.qk_norm_eps is not None:
            specs["q_norm"] = ParamSpec((self.head_dim,), role="scale")
            specs["k_norm"] = ParamSpec((self.head_dim,), role="scale")
        return specs

    def children(self):
        return {"position": self.position}

    def cache_need(self) -> CacheNeed:
        return CacheNeed(self.num_kv_heads, self.head_dim, self.window)

    def state_need(self):
        return None

    def native(self):
        from ..csrc import host_api
        if self.qk_norm_eps is not None:        # the executor has no form with a norm of the heads
            return None
        table = self.position.table(self.qkv_weight.device)
        if table.dtype != torch.float32 or not table.is_contiguous() or table.numel() * 2 != self.position.rotary_dim:
            return None
        return host_api.AttentionDesc(self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim, self.window or 0,
                                      self.position.pairing_code, self.position.rotary_dim, self.scale,
                                      host_api.weight(self.qkv_weight), host_api.weight(self.qkv_bias),
                                      host_api.weight(self.out_weight), host_api.weight(self.out_bias), table.data_ptr())

    def forward(self, normed, ctx, entry):
        b, kv = ctx.batch, ctx.kv(entry)
        rope = (b.positions, b.slot_of_token, kv.table, self.position.table(ctx.device), self.position.pairing_code,
                self.position.rotary_dim, kv.k_pages if kv.owns else None, kv.v_pages if kv.owns else None,
                kv.layer_offset, kv.page_size, kv.page_stride, self.num_heads, self.num_kv_heads, self.head_dim, ctx.act)
        if self.qk_norm_eps is None:
            q = ops.qkv_rope_write(normed, self.qkv_weight, self.qkv_bias, *rope, runs=b.runs())
        else:
            qkv = ops.gemm(normed, self.qkv_weight, ctx.act, bias=self.qkv_bias)
            ops.head_rmsnorm(qkv, self.q_norm, self.k_norm, self.qk_norm_eps, self.num_heads, self.num_kv_heads,
                             self.head_dim, ctx.act)
            q = ops.rope_kv_write(qkv, *rope, runs=b.runs())
        o = ops.attention(q, kv.k_pages, kv.v_pages, kv.layer_offset, b.positions, b.slot_of_token, kv.table,
                          kv.page_size, kv.page_stride, self.num_heads, self.num_kv_heads, self.head_dim,
                          self.window, self.scale, ctx.act, runs=b.runs())
        return ops.gemm(o, self.out_weight, ctx.act, bias=self.out_bias, partial_sums=True)
