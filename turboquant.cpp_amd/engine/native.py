"""A step through the step executor of the kernel library: one call from here issues every launch of the step.

The layers' parts describe themselves to the executor (``Part.native``); a model whose schedule entries all run layers
that can be described is stepped by ``NativeModel.forward``, which packs nothing and computes nothing itself: it hands
the executor the model's descriptors, the step's packed arrays, a workspace and the place for the logits.  A model
with a part that the executor does not know (a part registered from outside, a norm of the heads) has no
``NativeModel``, and its steps are run part by part through the parts' ``forward`` (``CausalLM.forward``); both ways
launch the same kernels with the same arguments and give the same bits.
"""
from __future__ import annotations

import ctypes
import os

import torch

from ..csrc import host_api, ops
from ..parts import ffn as ffn_parts


class NativeModel:
    """The descriptors of one model with one cache, kept alive for the executor."""

    def __init__(self, model, cache):
        self.model, self.cache = model, cache
        self.lib = host_api.library(model.act)
        layers = [b.native() for b in model.blocks]
        if any(l is None for l in layers):
            raise ValueError("a layer of the model has no form in the step executor")
        self.layers = (host_api.LayerDesc * len(layers))(*layers)
        entries = []
        for e, sched in enumerate(model.schedule):
            block = model.blocks[sched.layer]
            if block.state_need() is not None or block.cache_need() is None:
                raise ValueError("the step executor runs layers that keep keys and values and no state of their own")
            kv = cache.kv(e)
            if kv.v_pages is None or kv.v_layer_offset != kv.layer_offset or kv.v_page_stride != kv.page_stride:
                raise ValueError("the step executor's attention keeps values as wide as its keys")
            entries.append(host_api.EntryDesc(sched.layer, kv.k_pages.data_ptr(), kv.v_pages.data_ptr(), kv.table.data_ptr(),
                                              kv.table.shape[1], kv.layer_offset, kv.page_size, kv.page_stride, int(kv.owns)))
        self.entries = (host_api.EntryDesc * len(entries))(*entries)
        plan = model.plan
        self.desc = host_api.ModelDesc(plan.vocab_size, plan.hidden_size, len(layers), len(entries),
                                       ctypes.cast(self.layers, ctypes.c_void_p), ctypes.cast(self.entries, ctypes.c_void_p),
                                       host_api.weight(model.embedding), host_api.weight(model.lm_head),
                                       model.final_norm.native(), float(plan.embedding_scale), float(plan.logit_softcap or 0.0))
        self.last_launches = 0          # launcher calls of the last step
        self.vendor_products = 0        # products that steps so far handed to the vendor's matrix library

    @staticmethod
    def build(model, cache):
        """The model's ``NativeModel``, or None where the executor cannot run it (no GPU, a part it does not know)."""
        if model.device is None or model.device.type != "cuda" or os.environ.get("TQ_HOST", "native") == "python":
            return None
        try:
            if not isinstance(model.final_norm.native(), host_api.NormDesc):
                return None
            return NativeModel(model, cache)
        except (ValueError, ops.KernelError):
            return None

    def forward(self, ctx) -> torch.Tensor:
        """The logits [wanted rows, vocab] of the step that ``ctx`` describes."""
        b = ctx.batch
        dev = self.model.device
        V = self.model.plan.vocab_size
        logits = torch.empty((b.n_want, V), dtype=torch.float32, device=dev)
        side = ctx.side_stream
        step = host_api.StepDesc(
            b.n_tokens, b.n_seqs, b.n_want, b.max_new, b.max_end, int(b.is_decode), int(bool(ctx.capturing)),
            ops.VENDOR_MIN_ROWS if ops._VENDOR else 0, ops.VENDOR_GATED_ROWS, ops.EXPERT_128_FROM, ops.EXPERT_256_FROM, ops.EXPERT_PAIRS_FROM,
            ffn_parts.SIDE_STREAM_FROM_IN_EXECUTOR,
            b.tokens.data_ptr(), b.positions.data_ptr(), b.slot_of_token.data_ptr(), b.cu_seqlens.data_ptr(),
            b.slots_dev.data_ptr(), b.start_dev.data_ptr(), b.want_rows.data_ptr() if b.n_want else None, None, 0,
            logits.data_ptr() if b.n_want else None, ops._stream(), side.cuda_stream if side is not None else None)
        need = self.lib.tq_step_workspace(ctypes.byref(self.desc), ctypes.byref(step))
        if need < 0:
            raise ops.KernelError(f"step executor: {self.lib.tq_engine_last_error().decode()}")
        workspace = torch.empty((need + 256,), dtype=torch.uint8, device=dev)
        at = workspace.data_ptr()
        step.workspace = (at + 255) // 256 * 256
        step.workspace_bytes = need
        rc = self.lib.tq_step_forward(ctypes.byref(self.desc), ctypes.byref(step))
        if rc != 0:
            raise ops.KernelError(f"step executor: {self.lib.tq_engine_last_error().decode()}")
        self.last_launches = int(self.lib.tq_engine_last_launches())
        self.vendor_products += int(self.lib.tq_engine_last_vendor_products())
        # (the workspace goes back to the allocator here, which hands it out again for work on the main stream only;
        # the main stream has waited for whatever the side stream did in it)
        return logits
