"""Feed-forward parts: a dense gated one and a sparse one with routed experts and a shared expert.

Dense (/root/reference/src/engine/tq_transformer.c:2707-2824): ``down(silu(gate x) * (up x))``, no biases; the
gate's activation is an argument (``silu``, ``gelu_tanh`` as /root/reference/src/engine/tq_ops.c:1482-1484, ``relu2``)
that the products' epilogues take.
Sparse (/root/reference/src/engine/tq_moe.c:600-1059): router logits in float32, top-k with the highest index
winning ties, weights from a softmax; every chosen expert is the dense formula with its own matrices, summed
with its weight in the order chosen; the shared expert, scaled by ``sigmoid(x . shared_scale)``, is added
last.  ``renormalize`` false keeps the softmax over all experts un-normalised for the chosen ones; true is
the reference's softmax over the chosen logits.
"""
from __future__ import annotations

import torch

from ..csrc import ops
from .base import ParamSpec, Part, register_part


SIDE_STREAM_FROM = 320      # tokens of an eager step from which the shared expert goes to a second stream
# The same border where the step executor issues the launches: forking and joining cost it two events a layer, not the
# 2.6 ms a step that they cost a step issued from Python, so the second stream pays from far fewer tokens on (measured
# on 24 layers, one prompt, with and without it: 48 tokens 4.32 against 4.36 ms, 96 tokens 5.27 against 5.73, 192 tokens
# 5.39 against 6.44, 320 tokens 6.31 against 7.71, 512 tokens 8.06 against 9.06; 24 tokens 3.59 against 3.46).
SIDE_STREAM_FROM_IN_EXECUTOR = 64


@register_part("ffn", "dense_swiglu")
class DenseSwiGLU(Part):
    graph_safe = True
    wants_f32 = False

    def __init__(self, hidden_size: int, inner_size: int, activation: str = "silu"):
        if activation not in ops.GATES:
            raise ValueError(f"unknown activation {activation!r}; known: {', '.join(sorted(ops.GATES))}")
        self.hidden_size, self.inner_size, self.activation = hidden_size, inner_size, activation
        self.gate = self.up = self.down = None

    def param_specs(self):
        return {"gate": ParamSpec((self.inner_size, self.hidden_size)),
                "up": ParamSpec((self.inner_size, self.hidden_size)),
                "down": ParamSpec((self.hidden_size, self.inner_size))}

    def prepare(self, device, act):
        # gate and up side by side: a long prompt's pair may then go out as one product over both
        self.gate, self.up = ops.side_by_side(self.gate, self.up)

    def native(self):
        from ..csrc import host_api
        return host_api.DenseFfnDesc(self.hidden_size, self.inner_size, ops.GATES[self.activation], host_api.weight(self.gate),
                                     host_api.weight(self.up), host_api.weight(self.down))

    def forward(self, normed, normed32, ctx):
        h = ops.gemm(normed, self.gate, ctx.act, w2=self.up, out_act=True, activation=self.activation)
        return ops.gemm(h, self.down, ctx.act, partial_sums=True)


@register_part("ffn", "moe_swiglu")
class SparseMoE(Part):
    graph_safe = True
    wants_f32 = True    # the router reads the normalised activations in float32

    def __init__(self, hidden_size: int, num_experts: int, top_k: int, expert_size: int, shared_size: int = 0,
                 shared_gated: bool = True, renormalize: bool = False, activation: str = "silu"):
        if not 1 <= top_k <= num_experts:
            raise ValueError(f"top_k {top_k} must be within 1..num_experts {num_experts}")
        if activation not in ops.GATES:
            raise ValueError(f"unknown activation {activation!r}; known: {', '.join(sorted(ops.GATES))}")
        self.activation = activation
        self.hidden_size, self.num_experts, self.top_k = hidden_size, num_experts, top_k
        self.expert_size, self.shared_size = expert_size, shared_size
        self.shared_gated, self.renormalize = shared_gated and shared_size > 0, renormalize
        self.router = self.expert_gate = self.expert_up = self.expert_down = None
        self.shared_gate = self.shared_up = self.shared_down = self.shared_scale = None

    def param_specs(self):
        E, H, I, S = self.num_experts, self.hidden_size, self.expert_size, self.shared_size
        specs = {"router": ParamSpec((E, H), role="router"),
                 "expert_gate": ParamSpec((E, I, H)), "expert_up": ParamSpec((E, I, H)),
                 "expert_down": ParamSpec((E, H, I))}
        if S > 0:
            specs.update({"shared_gate": ParamSpec((S, H)), "shared_up": ParamSpec((S, H)),
                          "shared_down": ParamSpec((H, S))})
            if self.shared_gated:
                specs["shared_scale"] = ParamSpec((1, H), role="router")
        return specs

    def prepare(self, device, act):
        if self.shared_size > 0:     # as in the dense part; the experts' products never leave this library's kernels
            self.shared_gate, self.shared_up = ops.side_by_side(self.shared_gate, self.shared_up)

    def native(self):
        from ..csrc import host_api
        w = host_api.weight
        return host_api.MoeFfnDesc(self.hidden_size, self.num_experts, self.top_k, self.expert_size, self.shared_size,
                                   int(self.renormalize), ops.GATES[self.activation], w(self.router),
                                   w(self.shared_scale if self.shared_gated else None), w(self.expert_gate), w(self.expert_up),
                                   w(self.expert_down), w(self.shared_gate), w(self.shared_up), w(self.shared_down))

    def forward(self, normed, normed32, ctx):
        T = normed.shape[0]
        unit = ops.expert_tile_rows(T * self.top_k, self.num_experts, ctx.act, normed, self.expert_gate)
        route = lambda: ops.route(normed32, self.router, self.shared_scale if self.shared_gated else None,
                                  self.top_k, self.renormalize, unit, ctx.act)
        if self.shared_size > 0 and T <= 16 and unit == 16:
            # a handful of tokens: the shared expert's two products ride in the launches of the routed experts'
            _, weights, gate, sorted_token, pair_slot, tile_expert, n_tiles = route()
            experts = dict(a_rows=sorted_token, tile_group=tile_expert, n_tiles=n_tiles, tile_rows=unit)
            h, hs = ops.gemm_pair(dict(a=normed, w=self.expert_gate, w2=self.expert_up, out_act=True,
                                       activation=self.activation, **experts),
                                  dict(a=normed, w=self.shared_gate, w2=self.shared_up, out_act=True,
                                       activation=self.activation), ctx.act)
            y, shared = ops.gemm_pair(dict(a=h, w=self.expert_down, gather=False, **experts),
                                      dict(a=hs, w=self.shared_down, partial_sums=True), ctx.act)
            return ops.GatheredSum(y, pair_slot, weights, shared, gate)
        # The shared expert needs nothing from the router: it may run on a second stream beside the routed experts.
        # That pays while its products are a few passes of tiles over the chip, whose ends the other stream's work
        # fills (2,048 tokens of width 5,632: 5 % of the step; 512 tokens: 10 %); with eight passes and more the two
        # only disturb each other (2,048 tokens of width 20,480: 2 % slower).
        shared, side = None, None
        if self.shared_size > 0:
            tiles = -(-T // 128) * -(-self.shared_size // 128)
            # Below some 300 tokens the host's part of forking and joining (2.6 ms of a step of 24 layers, which is
            # then as long on the host as on the chip) is more than the second stream gains: a prompt step of 65 tokens
            # took 6.8 ms with it and 5.4 without, one of 200 tokens 6.8 and 6.3, of 320 tokens 7.15 and 7.2, of 512
            # tokens 7.9 and 8.8.  A step that is being captured pays the host once and is replayed with the two
            # streams (64 sequences: 10.8 ms a step with them, 11.15 without).
            worth = T >= SIDE_STREAM_FROM or getattr(ctx, "capturing", False)
            side = ctx.fork() if hasattr(ctx, "fork") and worth and tiles < 8 * 256 else None
            if side is not None:
                with torch.cuda.stream(side):
                    shared = self._shared(normed, ctx)
            else:
                shared = self._shared(normed, ctx)
        _, weights, gate, sorted_token, pair_slot, tile_expert, n_tiles = route()
        rows = ops.expert_product_rows(unit, T * self.top_k, self.num_experts)
        h = ops.gemm(normed, self.expert_gate, ctx.act, w2=self.expert_up, out_act=True, a_rows=sorted_token,
                     tile_group=tile_expert, n_tiles=n_tiles, tile_rows=rows, activation=self.activation)
        y = ops.gemm(h, self.expert_down, ctx.act, a_rows=sorted_token, tile_group=tile_expert, n_tiles=n_tiles,
                     tile_rows=rows, gather=False)
        if side is not None:
            ctx.join()
        # the weighted sum over the chosen experts and the shared expert is left to the next norm
        return ops.GatheredSum(y, pair_slot, weights, shared, gate)

    def _shared(self, normed, ctx):
        hs = ops.gemm(normed, self.shared_gate, ctx.act, w2=self.shared_up, out_act=True, activation=self.activation)
        return ops.gemm(hs, self.shared_down, ctx.act, partial_sums=True)
