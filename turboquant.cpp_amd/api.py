"""The Python entry point, in the manner of the reference's ``quantcpp.Model``
(/root/reference/bindings/python/quantcpp/__init__.py:220-683): a model is opened from a path with keyword
options ``temperature``, ``top_p``, ``max_tokens``, ``context_length``, generates, and is closed or used as a
context manager.  The reference's model takes text; this one takes and returns token ids (no tokenizer is
part of the library).
"""
from __future__ import annotations

import math
import os
from typing import Iterator, Sequence

import numpy as np
import torch

from .csrc import ops
from .engine.generate import GenerationOptions, GenerationResult, generate
from .engine.model import load_model, random_model
from .engine.step import Engine


class Model:
    """A loaded model ready to generate.

    ``path``: a folder with ``config.json`` and ``model.safetensors``.  ``dtype``: ``"bfloat16"`` (serving
    kernels) or ``"float32"`` (everything in true 32-bit).  ``context_length``: the most positions (prompt and
    generated tokens) of a sequence, which the cache is sized for; a sequence that reaches it ends with reason
    ``"context"`` (0: the model's ``max_position_embeddings``, at most 4096 as in the reference,
    /root/reference/src/engine/tq_model.c:2951).  ``max_batch``: sequences that generate together.
    """

    def __init__(self, path: str, *, temperature: float = 0.7, top_p: float = 0.9, max_tokens: int = 256,
                 context_length: int = 0, dtype: str = "bfloat16", seed: int = 42, rep_penalty: float = 1.1,
                 max_batch: int = 8, device: str = "cuda:0", stop_tokens: Sequence[int] | None = None):
        if not os.path.isdir(path):
            raise FileNotFoundError(f"model folder not found: {path}")
        self._path = path
        self._model = load_model(path, act=dtype, device=device)
        self._setup(temperature, top_p, max_tokens, context_length, seed, rep_penalty, max_batch, stop_tokens)

    @classmethod
    def from_random(cls, config_json: dict, seed: int, **kw) -> "Model":
        """A model with random weights drawn in memory from a config.json dictionary and a seed."""
        self = cls.__new__(cls)
        self._path = "<random>"
        opts = dict(temperature=0.7, top_p=0.9, max_tokens=256, context_length=0, dtype="bfloat16",
                    gen_seed=42, rep_penalty=1.1, max_batch=8, device="cuda:0", stop_tokens=None, std=0.02, norm_std=0.0)
        opts.update(kw)
        self._model = random_model(config_json, seed, act=opts["dtype"], device=opts["device"], std=opts["std"],
                                   norm_std=opts["norm_std"])
        self._setup(opts["temperature"], opts["top_p"], opts["max_tokens"], opts["context_length"], opts["gen_seed"],
                    opts["rep_penalty"], opts["max_batch"], opts["stop_tokens"])
        return self

    def _setup(self, temperature, top_p, max_tokens, context_length, seed, rep_penalty, max_batch, stop_tokens):
        plan = self._model.plan
        ctx = context_length if context_length > 0 else min(plan.max_positions, 4096)
        ctx = min(ctx, plan.max_positions)
        self.context_length = ctx
        self.options = GenerationOptions(
            max_tokens=max_tokens, temperature=temperature, top_p=top_p, seed=seed, rep_penalty=rep_penalty,
            stop_tokens=tuple(stop_tokens) if stop_tokens is not None else tuple(plan.stop_tokens), max_batch=max_batch)
        page = 64
        per_seq = -(-ctx // page) * page
        # the cache holds ``max_batch`` sequences of ``context_length`` positions, and no sequence may grow beyond that
        self._engine = Engine(self._model, max_tokens=per_seq * max_batch, page_size=page, max_slots=max_batch,
                              max_positions=ctx)

    # ------------------------------------------------------------ generation
    def generate(self, prompts, **overrides) -> list[list[int]]:
        """Token ids in, token ids out.  ``prompts`` is one list of ids or a list of such lists."""
        return [r.tokens for r in self.generate_detailed(prompts, **overrides)] if _is_batch(prompts) \
            else self.generate_detailed([prompts], **overrides)[0].tokens

    def generate_detailed(self, prompts, **overrides) -> list[GenerationResult]:
        self._ensure_open()
        opts = GenerationOptions(**{**self.options.__dict__, **overrides})
        return generate(self._engine, [list(p) for p in prompts], opts)

    def stream(self, prompt: Sequence[int], **overrides) -> Iterator[int]:
        """Yields the tokens of one continuation (the reference's ``generate`` yields text pieces)."""
        yield from self.generate(list(prompt), **overrides)

    def perplexity(self, tokens: Sequence[int], chunk: int = 512, save_logits: str | None = None,
                   kl_baseline: str | None = None) -> dict:
        """Teacher-forced evaluation of a token sequence as the reference's ``--ppl`` does it
        (/root/reference/tools/quant.c:430-720): the sequence, cut to the context length, goes through the model once
        (here ``chunk`` tokens a step), and every token but the first is scored by the logits of the position
        before it.  Returns ``tokens``, ``tokens_evaluated`` (targets outside the vocabulary are left out, :575),
        ``avg_nll`` and ``perplexity`` = exp(avg_nll).

        ``save_logits``: a file that receives, as the reference's ``--save-logits`` writes it (:542-547, :594-611), two
        int32 (tokens - 1, vocabulary) and then every scored position's probabilities as 16-bit floats.
        ``kl_baseline``: such a file of another run (another activation type, say); the result then also holds
        ``mean_kl``, the mean over the scored positions of KL(baseline || this run), and ``kl_tokens`` (:612-636)."""
        self._ensure_open()
        tokens = [int(t) for t in tokens][:self.context_length]
        if len(tokens) < 2:
            raise ValueError("need at least 2 tokens for perplexity")
        eng, act = self._engine, self._model.act
        V = eng.vocab_size
        feed = [t if 0 <= t < V else 0 for t in tokens]      # a token outside the vocabulary is fed as token 0, never scored
        save_f = base_f = None
        total, n_eval, total_kl, n_kl = 0.0, 0, 0.0, 0
        slot = eng.open(1)
        try:
            if save_logits:
                save_f = open(save_logits, "wb")
                save_f.write(np.array([len(tokens) - 1, V], dtype="<i4").tobytes())
            if kl_baseline:
                base_f = open(kl_baseline, "rb")
                header = np.frombuffer(base_f.read(8), dtype="<i4")
                if header.size != 2 or int(header[1]) != V:
                    raise ValueError(f"KL baseline header mismatch (expected vocab={V})")
            for lo in range(0, len(tokens) - 1, chunk):
                hi = min(lo + chunk, len(tokens) - 1)           # positions lo .. hi - 1 predict tokens lo + 1 .. hi
                logits = eng.step(slot, [feed[lo:hi]], [list(range(hi - lo))])
                targets = torch.tensor(tokens[lo + 1:hi + 1], dtype=torch.int32).to(logits.device)
                nll = ops.nll(logits, targets, act).double().cpu()
                scored = ~torch.isnan(nll)
                total += float(nll[scored].sum())
                n_eval += int(scored.sum())
                if save_f is None and base_f is None:
                    continue
                rows = torch.nonzero(scored).flatten()
                if rows.numel() == 0:
                    continue
                if rows.numel() < hi - lo:                    # only scored positions have a row in either file
                    logits = logits[rows.to(logits.device)].contiguous()
                base = None
                if base_f is not None:
                    raw = np.frombuffer(base_f.read(rows.numel() * V * 2), dtype="<i2")
                    have = raw.size // V                        # a baseline that ends early is compared as far as it goes
                    if have:
                        base = torch.from_numpy(raw[:have * V].reshape(have, V).copy()).to(logits.device)
                probs = ops.probs_half(logits, act)[0] if save_f is not None else None
                kl = None
                if base is not None:
                    cur = logits if base.shape[0] == logits.shape[0] else logits[:base.shape[0]].contiguous()
                    kl = ops.probs_half(cur, act, want_probs=False, base=base)[1]
                if save_f is not None:
                    save_f.write(probs.cpu().numpy().astype("<i2").tobytes())
                if kl is not None:
                    total_kl += float(kl.sum())
                    n_kl += kl.numel()
        finally:
            eng.close(slot)
            for f in (save_f, base_f):
                if f is not None:
                    f.close()
        if n_eval == 0:
            raise ValueError("no token of the sequence is a token of the vocabulary")
        avg = total / n_eval
        res = {"tokens": len(tokens), "tokens_evaluated": n_eval, "avg_nll": avg, "perplexity": math.exp(avg)}
        if kl_baseline:
            res.update({"mean_kl": total_kl / n_kl if n_kl else float("nan"), "kl_tokens": n_kl})
        return res

    # ------------------------------------------------------------ lower level, for tests and tools
    @property
    def engine(self) -> Engine:
        self._ensure_open()
        return self._engine

    @property
    def path(self) -> str:
        return self._path

    @property
    def config(self):
        return self._model.config

    def close(self) -> None:
        self._engine = None
        self._model = None

    def _ensure_open(self) -> None:
        if self._model is None:
            raise ValueError("model has been closed")

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __repr__(self):
        return f"Model(path={self._path!r}, open={self._model is not None})"


def _is_batch(prompts) -> bool:
    return len(prompts) > 0 and isinstance(prompts[0], (list, tuple))


def load(path: str, **kw) -> Model:
    """Same as ``Model(path, **kw)`` (/root/reference/bindings/python/quantcpp/__init__.py:679-683)."""
    return Model(path, **kw)
