"""A causal language model put together from a plan: embedding, layers in schedule order, final norm,
vocabulary projection.

Order of the reference's step (/root/reference/src/engine/tq_transformer.c:2281-3029): embedding row without
scaling (:2297-2329); for each layer norm, mixer, residual, norm, feed-forward, residual (:2410-2824); final
norm (:2922); ``logits = W_out x`` with the embedding standing in for a missing output matrix
(:2931-2942; /root/reference/src/engine/tq_model.c:1499-1516).  The projection runs only on the rows whose
logits are wanted.
"""
from __future__ import annotations

import os

import torch

from ..cache.paged import PagedCache
from ..config.plan import LayerSpec, ModelPlan, PartSpec, Source
from ..config.registry import config_from_dict, config_from_dir
from ..csrc import ops
from ..parts.base import ParamSpec, Part, build_part, _REGISTRIES
from ..weights.loader import Binding, TensorDict, expected_tensors, load_bindings
from ..weights.random_init import random_tensors, write_random_model
from ..weights.safetensors_io import SafetensorsFolder
from .context import StepContext

ACT_NAMES = {"float32": "float32", "f32": "float32", "fp32": "float32", "bfloat16": "bfloat16", "bf16": "bfloat16"}


def build_block(spec: LayerSpec) -> Part:
    """Builds a layer: the block kind says which parts it is made of and from which registry each comes."""
    try:
        cls = _REGISTRIES["block"][spec.block]
    except KeyError:
        raise ValueError(f"unknown block {spec.block!r}; known: {', '.join(sorted(_REGISTRIES['block']))}") from None
    missing = [n for n in cls.slots if n not in spec.parts]
    if missing:
        raise ValueError(f"block {spec.block!r} needs parts {missing}")
    return cls(**{name: build_part(category, spec.parts[name]) for name, category in cls.slots.items()})


def _bind(part: Part, spec: PartSpec, path: str, out: list[Binding]) -> None:
    for name, pspec in part.param_specs().items():
        if name not in spec.tensors:
            raise ValueError(f"{path}: the plan names no checkpoint tensor for parameter {name!r}")
        out.append(Binding(part, name, pspec, spec.tensors[name], f"{path}.{name}"))
    for name in spec.tensors:
        if name not in part.param_specs():
            raise ValueError(f"{path}: the plan gives a tensor for {name!r}, which {spec.kind} does not have")


class CausalLM:
    def __init__(self, plan: ModelPlan, act: str, config=None):
        plan.validate()
        self.plan, self.config = plan, config
        self.act = ACT_NAMES[act]
        self.act_dtype = ops.ACT_DTYPES[self.act]
        self.blocks = [build_block(ls) for ls in plan.layers]
        self.final_norm = build_part("norm", plan.final_norm)
        self.schedule = list(plan.schedule)
        self.embedding = None      # [V, H]
        self.lm_head = None        # [V, H]; the embedding when tied
        self.device = None
        self.bindings: list[Binding] = []
        for i, (ls, block) in enumerate(zip(plan.layers, self.blocks)):
            for name in block.slots:
                _bind(getattr(block, name), ls.parts[name], f"layers.{i}.{name}", self.bindings)
        _bind(self.final_norm, plan.final_norm, "final_norm", self.bindings)
        V, H = plan.vocab_size, plan.hidden_size
        self.bindings.append(Binding(self, "embedding", ParamSpec((V, H), role="table"), plan.embedding, "embedding"))
        if plan.lm_head is not None:
            self.bindings.append(Binding(self, "lm_head", ParamSpec((V, H)), plan.lm_head, "lm_head"))

    # ------------------------------------------------------------ weights
    def tensor_table(self) -> dict:
        """name -> (shape, role) of every checkpoint tensor this model reads."""
        return expected_tensors(self.bindings)

    def load(self, reader, device, f32_matrices: str = "bfloat16") -> "CausalLM":
        """``f32_matrices``: what becomes, on the bfloat16 path, of matrices that the checkpoint stores in 32 bits:
        "bfloat16" rounds them once as they are placed, "keep" leaves them as stored."""
        self.device = torch.device(device)
        self.weight_bytes = load_bindings(self.bindings, reader, self.act, self.device, f32_matrices)
        if self.plan.lm_head is None:
            self.lm_head = self.embedding
        for part in self.parts():
            part.prepare(self.device, self.act)
        return self

    def parts(self):
        def walk(p):
            yield p
            for c in p.children().values():
                yield from walk(c)
        for b in self.blocks:
            yield from walk(b)
        yield self.final_norm

    # ------------------------------------------------------------ cache
    def cache_needs(self):
        needs = []
        for e in self.schedule:
            block = self.blocks[e.layer]
            needs.append((block.cache_need(), block.state_need(), e.cache_of))
        return needs

    def new_cache(self, max_tokens: int, page_size: int = 64, max_slots: int | None = None,
                  max_positions: int | None = None, window_step: int = 2048) -> PagedCache:
        """``max_positions``: the most positions a sequence may reach, if that is to be fewer than the model allows."""
        limit = self.plan.max_positions if max_positions is None else min(max_positions, self.plan.max_positions)
        return PagedCache(self.cache_needs(), max_tokens, self.act_dtype, self.device, page_size=page_size,
                          max_slots=max_slots, max_positions=limit, window_step=window_step)

    # ------------------------------------------------------------ forward
    def forward(self, ctx: StepContext) -> torch.Tensor:
        """Runs the step's tokens through the schedule; returns float32 logits [wanted rows, vocab]."""
        b = ctx.batch
        if ctx.native is not None and ctx.layer_hook is None and ops._PROFILE is None:
            # one call into the library's step executor issues every launch of the step; what follows here is the
            # same step part by part, for models with parts that the executor does not know, for whoever looks at
            # the layers (layer_hook) and for the profile, which puts an event behind every launch
            return ctx.native.forward(ctx)
        x = ops.embed(b.tokens, self.embedding, self.act, scale=self.plan.embedding_scale)
        pending = None
        for entry, e in enumerate(self.schedule):
            pending = self.blocks[e.layer].forward(x, pending, ctx, entry)
            if ctx.layer_hook is not None:      # the stream with what the entry has left for the next norm to add
                held = pending.materialize(self.act) if isinstance(pending, ops.GatheredSum) else pending
                ctx.layer_hook(entry, x.clone() if held is None else x + held.sum(0), b)
        if b.n_want == 0:
            return torch.empty((0, self.plan.vocab_size), dtype=torch.float32, device=x.device)
        normed, _ = self.final_norm.forward(x, pending, ctx, rows=b.want_rows)
        logits = ops.gemm(normed, self.lm_head, self.act)
        if self.plan.logit_softcap is not None:
            ops.softcap(logits, self.plan.logit_softcap, self.act)
        return logits


# ---------------------------------------------------------------- construction
def model_from_config(config_json: dict, act: str) -> CausalLM:
    arch, cfg = config_from_dict(config_json)
    return CausalLM(arch.plan(cfg), act, config=cfg)


def load_model(model_dir: str, act: str = "bfloat16", device="cuda:0", f32_matrices: str = "bfloat16") -> CausalLM:
    """Reads config.json, picks the architecture from it, and loads model.safetensors by tensor name."""
    arch, cfg = config_from_dir(model_dir)
    model = CausalLM(arch.plan(cfg), act, config=cfg)
    with SafetensorsFolder(model_dir) as folder:
        model.load(folder, device, f32_matrices)
    return model


def random_model(config_json: dict, seed: int, act: str = "bfloat16", device="cuda:0", std: float = 0.02,
                 norm_std: float = 0.0, on_device: bool = True, dtype: str | None = None,
                 f32_matrices: str = "bfloat16") -> CausalLM:
    """A model with random weights drawn in memory, tensor by tensor, where the model lives: the values of the
    folder that ``write_random_model_dir`` writes for the same configuration, seed and ``dtype`` (the type the
    folder's tensors would have; default: the activation type)."""
    model = model_from_config(config_json, act)
    table = model.tensor_table()
    dtype = {"float32": torch.float32, "bfloat16": torch.bfloat16}[ACT_NAMES[dtype] if dtype else model.act]
    gen_device = device if on_device else "cpu"

    class _Lazy:
        """Draws each tensor when it is read, so no second copy of the model is ever held."""
        def __init__(self):
            from ..weights.safetensors_io import NAMES
            self.index = {n: i for i, n in enumerate(table)}
            self.entries = {n: TensorDict._Entry(tuple(s), NAMES[dtype]) for n, (s, _r) in table.items()}

        def read(self, name):
            from ..weights.random_init import random_tensor
            shape, role = table[name]
            return random_tensor(self.index[name], shape, role, seed, std, norm_std, dtype, gen_device)

    return model.load(_Lazy(), device, f32_matrices)


def write_random_model_dir(model_dir: str, config_json: dict, seed: int, std: float = 0.02, norm_std: float = 0.0,
                           dtype: str = "bfloat16") -> str:
    """Random-weights mode: writes config.json and model.safetensors for a configuration and a seed."""
    model = model_from_config(config_json, "float32")
    arch, cfg = config_from_dict(config_json)
    return write_random_model(model_dir, arch.config_to_json(cfg), model.tensor_table(), seed, std, norm_std, dtype)
