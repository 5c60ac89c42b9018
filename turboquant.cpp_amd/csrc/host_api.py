"""Python face of the step executor (``csrc/host/engine.h``): the descriptors as ``ctypes`` structures.

Every field of the C structures is 8 bytes wide, so the mirrors below use ``c_int64``, ``c_double`` and ``c_void_p``
only; ``check_layout`` compares their sizes with what the library reports and raises if they ever part.
"""
from __future__ import annotations

import ctypes

import torch

from . import ops

i64, f64, ptr = ctypes.c_int64, ctypes.c_double, ctypes.c_void_p

FFN_DENSE, FFN_MOE = 1, 2


class Weight(ctypes.Structure):
    _fields_ = [("ptr", ptr), ("wtype", i64)]


class NormDesc(ctypes.Structure):
    _fields_ = [("weight", Weight), ("eps", f64)]


class AttentionDesc(ctypes.Structure):
    _fields_ = [("hidden", i64), ("num_heads", i64), ("num_kv_heads", i64), ("head_dim", i64), ("window", i64),
                ("pairing", i64), ("rotary_dim", i64), ("scale", f64), ("qkv_weight", Weight), ("qkv_bias", Weight),
                ("out_weight", Weight), ("out_bias", Weight), ("inv_freq", ptr)]


class DenseFfnDesc(ctypes.Structure):
    _fields_ = [("hidden", i64), ("inner", i64), ("gate", i64), ("gate_w", Weight), ("up_w", Weight), ("down_w", Weight)]


class MoeFfnDesc(ctypes.Structure):
    _fields_ = [("hidden", i64), ("num_experts", i64), ("top_k", i64), ("inner", i64), ("shared_inner", i64),
                ("renormalize", i64), ("gate", i64), ("router", Weight), ("shared_scale", Weight),
                ("expert_gate", Weight), ("expert_up", Weight), ("expert_down", Weight), ("shared_gate", Weight),
                ("shared_up", Weight), ("shared_down", Weight)]


class LayerDesc(ctypes.Structure):
    _fields_ = [("mixer_norm", NormDesc), ("attention", AttentionDesc), ("ffn_norm", NormDesc), ("ffn_kind", i64),
                ("dense", DenseFfnDesc), ("moe", MoeFfnDesc)]


class EntryDesc(ctypes.Structure):
    _fields_ = [("layer", i64), ("k_pages", ptr), ("v_pages", ptr), ("table", ptr), ("table_width", i64),
                ("layer_offset", i64), ("page_size", i64), ("page_stride", i64), ("owns", i64)]


class ModelDesc(ctypes.Structure):
    _fields_ = [("vocab", i64), ("hidden", i64), ("n_layers", i64), ("n_entries", i64), ("layers", ptr), ("entries", ptr),
                ("embedding", Weight), ("lm_head", Weight), ("final_norm", NormDesc), ("embedding_scale", f64),
                ("logit_softcap", f64)]


class StepDesc(ctypes.Structure):
    _fields_ = [("T", i64), ("B", i64), ("n_want", i64), ("max_new", i64), ("max_end", i64), ("decode", i64),
                ("capturing", i64), ("vendor_min_rows", i64), ("vendor_gated_rows", i64), ("expert_128_from", i64),
                ("expert_256_from", i64), ("expert_pairs_from", i64), ("side_from", i64), ("tokens", ptr), ("positions", ptr), ("slot_of_token", ptr), ("cu_seqlens", ptr),
                ("slots", ptr), ("start", ptr), ("want_rows", ptr), ("workspace", ptr), ("workspace_bytes", i64),
                ("logits", ptr), ("stream", ptr), ("side_stream", ptr)]


STRUCTS = (Weight, NormDesc, AttentionDesc, DenseFfnDesc, MoeFfnDesc, LayerDesc, EntryDesc, ModelDesc, StepDesc)


def weight(t: torch.Tensor | None) -> Weight:
    """A parameter on the device as the executor takes it (None: absent)."""
    if t is None:
        return Weight(None, 0)
    if not (t.is_cuda and t.is_contiguous() and t.dtype in ops._WTYPE):
        raise ops.KernelError("a parameter of the step executor must be a contiguous float32 or bfloat16 tensor on the GPU")
    return Weight(t.data_ptr(), ops._WTYPE[t.dtype])


def library(act):
    """The kernel library of an activation type with the executor's entry points declared."""
    lib = ops.library(act)
    if not getattr(lib, "_host_declared", False):
        if not hasattr(lib, "tq_step_forward"):
            raise ops.KernelError("the kernel library holds no step executor")
        lib.tq_step_workspace.argtypes, lib.tq_step_workspace.restype = [ptr, ptr], i64
        lib.tq_step_forward.argtypes, lib.tq_step_forward.restype = [ptr, ptr], ctypes.c_int
        lib.tq_engine_last_error.argtypes, lib.tq_engine_last_error.restype = [], ctypes.c_char_p
        lib.tq_engine_last_launches.argtypes, lib.tq_engine_last_launches.restype = [], i64
        lib.tq_engine_last_vendor_products.argtypes, lib.tq_engine_last_vendor_products.restype = [], i64
        lib.tq_engine_struct_sizes.argtypes, lib.tq_engine_struct_sizes.restype = [ptr], None
        lib.tq_vendor_available.argtypes, lib.tq_vendor_available.restype = [], ctypes.c_int
        check_layout(lib)
        lib._host_declared = True
    return lib


def check_layout(lib) -> None:
    sizes = (i64 * len(STRUCTS))()
    lib.tq_engine_struct_sizes(sizes)
    mine = [ctypes.sizeof(s) for s in STRUCTS]
    if list(sizes) != mine:
        raise ops.KernelError(f"the step executor's structures are laid out as {list(sizes)} in the library and as {mine} here")
