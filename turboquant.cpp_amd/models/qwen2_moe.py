"""Qwen2-MoE (``Qwen2MoeForCausalLM``): typed configuration, model plan, checkpoint names.

The reference runs this architecture only from GGUF (``model_type = 2``,
/root/reference/src/engine/tq_model.c:3031-3056); the formulas of its layers are in
/root/reference/src/engine/tq_transformer.c:2281-3029 (step), :934-2269 (attention)
and /root/reference/src/engine/tq_moe.c:600-1059 (routing, experts, shared expert).
Tensor names are the safetensors names the reference's loader uses for the dense
tensors (tq_model.c:954,1243-1298,1474-1499) plus the Hugging Face names of the
bias, router, expert and shared-expert tensors, for which the reference has only
GGUF names (tq_model.c:3310-3319,3440-3553).

This module holds what is specific to the architecture and nothing else: which
keys of config.json mean what, which layer is sparse, which tensor feeds which
parameter.  The parts it names live in ``parts/`` and know nothing of it.
"""
from __future__ import annotations

from dataclasses import asdict, dataclass, field

from ..config.base import ConfigError, KeyReader, require
from ..config.plan import LayerSpec, ModelPlan, PartSpec, ScheduleEntry, Source
from ..config.registry import Architecture, register_architecture

ARCHITECTURE = "Qwen2MoeForCausalLM"
FULL, SLIDING = "full_attention", "sliding_attention"


@dataclass
class Qwen2MoeConfig:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int                  # feed-forward width of dense layers
    moe_intermediate_size: int              # width of one routed expert
    shared_expert_intermediate_size: int    # 0: no shared expert
    num_experts: int
    num_experts_per_tok: int
    norm_topk_prob: bool
    decoder_sparse_step: int
    mlp_only_layers: list[int]
    rope_theta: float
    rms_norm_eps: float
    use_sliding_window: bool
    sliding_window: int | None
    max_window_layers: int
    max_position_embeddings: int
    tie_word_embeddings: bool
    torch_dtype: str
    stop_token_ids: list[int] = field(default_factory=list)
    qkv_bias: bool = True                   # q, k and v have a bias unless the folder says otherwise
    layer_types: list[str] | None = None    # per layer "full_attention" or "sliding_attention", if the folder lists them

    # ---- derived ----
    def layer_is_sparse(self, layer: int) -> bool:
        """A layer has experts unless it is listed in ``mlp_only_layers`` or the sparse step skips it.
        (The reference decides by the presence of a router tensor, tq_model.c:3440-3444.)"""
        return (layer not in self.mlp_only_layers and self.num_experts > 0
                and (layer + 1) % self.decoder_sparse_step == 0)

    def layer_window(self, layer: int) -> int | None:
        """A sliding layer attends to the last ``sliding_window`` positions, the current one included (window
        semantics of tq_transformer.c:1646-1654).  Which layers slide: those that ``layer_types`` names, if the
        folder has that list (the reference likewise takes a per-layer list where its metadata holds one,
        tq_model.c:2867-2905); else the layers from ``max_window_layers`` on while ``use_sliding_window`` is true."""
        if self.layer_types is not None:
            return self.sliding_window if self.layer_types[layer] == SLIDING else None
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return None


def config_from_json(data: dict) -> Qwen2MoeConfig:
    r = KeyReader(data)
    hidden = r.integer("hidden_size", minimum=1)
    heads = r.integer("num_attention_heads", minimum=1)
    head_dim = r.optional_integer("head_dim")
    if head_dim is None:
        require(hidden % heads == 0, f"hidden_size {hidden} is not a multiple of num_attention_heads {heads} and no head_dim is given")
        head_dim = hidden // heads
    use_window = r.boolean("use_sliding_window", False)
    window = r.optional_integer("sliding_window")
    # options that would change the formulas and that this architecture's plan does not carry out
    require(data.get("rope_scaling") is None, f"rope_scaling {data.get('rope_scaling')!r} is not implemented")
    require(data.get("hidden_act", "silu") == "silu", f"hidden_act {data.get('hidden_act')!r} is not implemented (silu is)")
    layers = r.integer("num_hidden_layers", minimum=1)
    # newer folders keep the rotation's constants in an object of their own
    rope = data.get("rope_parameters")
    require(rope is None or isinstance(rope, dict), f"rope_parameters must be an object, got {rope!r}")
    if rope is not None:
        kind = rope.get("rope_type", rope.get("type", "default"))
        require(kind in (None, "default"), f"rope_parameters.rope_type {kind!r} is not implemented (default is)")
    if data.get("rope_theta") is not None or rope is None:
        rope_theta = r.number("rope_theta")
        require(rope is None or rope.get("rope_theta") in (None, rope_theta),
                f"rope_theta {rope_theta} and rope_parameters.rope_theta {rope and rope.get('rope_theta')} differ")
    else:
        rope_theta = KeyReader(rope, "config.json: rope_parameters").number("rope_theta")
    layer_types = data.get("layer_types")
    if layer_types is not None:
        require(isinstance(layer_types, list) and len(layer_types) == layers,
                f"layer_types must list one kind for each of the {layers} layers, got {layer_types!r}")
        unknown = sorted({str(t) for t in layer_types if t not in (FULL, SLIDING)})
        require(not unknown, f"layer_types names {unknown}; this architecture has {FULL!r} and {SLIDING!r}")
        require(SLIDING not in layer_types or (window is not None and window > 0),
                "layer_types names sliding layers but sliding_window is not a positive integer")
    stop: list[int] = []
    for key in ("eos_token_id",):
        if data.get(key) is not None:
            stop += r.integer_list(key)
    cfg = Qwen2MoeConfig(
        vocab_size=r.integer("vocab_size", minimum=1),
        hidden_size=hidden,
        num_hidden_layers=layers,
        num_attention_heads=heads,
        num_key_value_heads=r.integer("num_key_value_heads", heads, minimum=1),
        head_dim=head_dim,
        intermediate_size=r.integer("intermediate_size", minimum=1),
        moe_intermediate_size=r.integer("moe_intermediate_size", minimum=1),
        shared_expert_intermediate_size=r.integer("shared_expert_intermediate_size", minimum=0),
        num_experts=r.integer("num_experts", minimum=0),
        num_experts_per_tok=r.integer("num_experts_per_tok", minimum=1),
        norm_topk_prob=r.boolean("norm_topk_prob", False),
        decoder_sparse_step=r.integer("decoder_sparse_step", 1, minimum=1),
        mlp_only_layers=r.integer_list("mlp_only_layers", []),
        rope_theta=rope_theta,
        rms_norm_eps=r.number("rms_norm_eps"),
        use_sliding_window=use_window,
        sliding_window=window,
        max_window_layers=r.integer("max_window_layers", layers, minimum=0),
        max_position_embeddings=r.integer("max_position_embeddings", minimum=1),
        tie_word_embeddings=r.boolean("tie_word_embeddings", False),
        torch_dtype=r.string("torch_dtype", data.get("dtype") or "bfloat16"),
        stop_token_ids=stop,
        qkv_bias=r.boolean("qkv_bias", True),
        layer_types=layer_types,
    )
    validate(cfg)
    return cfg


def validate(c: Qwen2MoeConfig) -> None:
    require(c.num_attention_heads % c.num_key_value_heads == 0,
            f"num_attention_heads {c.num_attention_heads} is not a multiple of num_key_value_heads {c.num_key_value_heads}")
    require(c.head_dim % 2 == 0, f"head_dim {c.head_dim} must be even for rotary position encoding")
    if c.num_experts > 0:
        require(c.num_experts_per_tok <= c.num_experts,
                f"num_experts_per_tok {c.num_experts_per_tok} exceeds num_experts {c.num_experts}")
    for l in c.mlp_only_layers:
        require(0 <= l < c.num_hidden_layers, f"mlp_only_layers names layer {l}, model has {c.num_hidden_layers}")
    if c.use_sliding_window:
        require(c.sliding_window is not None and c.sliding_window > 0,
                "use_sliding_window is true but sliding_window is not a positive integer")
    require(c.rope_theta > 0, "rope_theta must be positive")
    require(c.rms_norm_eps > 0, "rms_norm_eps must be positive")
    require(c.torch_dtype in ("bfloat16", "float32", "float16"), f"torch_dtype {c.torch_dtype!r} is not supported")


def config_to_json(c: Qwen2MoeConfig) -> dict:
    d = asdict(c)
    stop = d.pop("stop_token_ids")
    if d["layer_types"] is None:
        del d["layer_types"]
    d["architectures"] = [ARCHITECTURE]
    d["model_type"] = "qwen2_moe"
    if stop:
        d["eos_token_id"] = stop if len(stop) > 1 else stop[0]
    return d


def plan(c: Qwen2MoeConfig) -> ModelPlan:
    layers = []
    for l in range(c.num_hidden_layers):
        p = f"model.layers.{l}"
        attn = PartSpec(
            kind="gqa_attention",
            args=dict(hidden_size=c.hidden_size, num_heads=c.num_attention_heads,
                      num_kv_heads=c.num_key_value_heads, head_dim=c.head_dim,
                      qkv_bias=c.qkv_bias, out_bias=False, window=c.layer_window(l),
                      position=PartSpec(kind="rope", args=dict(head_dim=c.head_dim, rotary_dim=c.head_dim,
                                                             theta=c.rope_theta, pairing="half"))),
            tensors={
                # q, k and v are stacked into one matrix so one product makes all three
                "qkv_weight": Source.concat([f"{p}.self_attn.{n}_proj.weight" for n in "qkv"]),
                "out_weight": Source.single(f"{p}.self_attn.o_proj.weight"),
            })
        if c.qkv_bias:
            attn.tensors["qkv_bias"] = Source.concat([f"{p}.self_attn.{n}_proj.bias" for n in "qkv"])
        if c.layer_is_sparse(l):
            tensors = {
                "router": Source.single(f"{p}.mlp.gate.weight"),
                "expert_gate": Source.stack([f"{p}.mlp.experts.{e}.gate_proj.weight" for e in range(c.num_experts)]),
                "expert_up": Source.stack([f"{p}.mlp.experts.{e}.up_proj.weight" for e in range(c.num_experts)]),
                "expert_down": Source.stack([f"{p}.mlp.experts.{e}.down_proj.weight" for e in range(c.num_experts)]),
            }
            if c.shared_expert_intermediate_size > 0:
                tensors.update({
                    "shared_gate": Source.single(f"{p}.mlp.shared_expert.gate_proj.weight"),
                    "shared_up": Source.single(f"{p}.mlp.shared_expert.up_proj.weight"),
                    "shared_down": Source.single(f"{p}.mlp.shared_expert.down_proj.weight"),
                    "shared_scale": Source.single(f"{p}.mlp.shared_expert_gate.weight"),
                })
            ffn = PartSpec(
                kind="moe_swiglu",
                args=dict(hidden_size=c.hidden_size, num_experts=c.num_experts, top_k=c.num_experts_per_tok,
                          expert_size=c.moe_intermediate_size, shared_size=c.shared_expert_intermediate_size,
                          shared_gated=True, renormalize=c.norm_topk_prob),
                tensors=tensors)
        else:
            ffn = PartSpec(
                kind="dense_swiglu",
                args=dict(hidden_size=c.hidden_size, inner_size=c.intermediate_size),
                tensors={
                    "gate": Source.single(f"{p}.mlp.gate_proj.weight"),
                    "up": Source.single(f"{p}.mlp.up_proj.weight"),
                    "down": Source.single(f"{p}.mlp.down_proj.weight"),
                })

        def norm(name: str) -> PartSpec:
            return PartSpec(kind="rmsnorm", args=dict(size=c.hidden_size, eps=c.rms_norm_eps),
                            tensors={"weight": Source.single(name)})

        layers.append(LayerSpec(block="prenorm", parts={
            "mixer_norm": norm(f"{p}.input_layernorm.weight"),
            "mixer": attn,
            "ffn_norm": norm(f"{p}.post_attention_layernorm.weight"),
            "ffn": ffn,
        }))
    return ModelPlan(
        architecture=ARCHITECTURE,
        vocab_size=c.vocab_size,
        hidden_size=c.hidden_size,
        layers=layers,
        schedule=[ScheduleEntry(layer=l) for l in range(c.num_hidden_layers)],
        final_norm=PartSpec(kind="rmsnorm", args=dict(size=c.hidden_size, eps=c.rms_norm_eps),
                            tensors={"weight": Source.single("model.norm.weight")}),
        embedding=Source.single("model.embed_tokens.weight"),
        lm_head=None if c.tie_word_embeddings else Source.single("lm_head.weight"),
        max_positions=c.max_position_embeddings,
        stop_tokens=tuple(c.stop_token_ids),
    )


register_architecture(Architecture(
    name=ARCHITECTURE,
    config_from_json=config_from_json,
    plan=plan,
    config_to_json=config_to_json,
))
