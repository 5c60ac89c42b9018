"""The Python entry point, in the manner of the reference's ``quantcpp.Model``
(/root/reference/bindings/python/quantcpp/__init__.py:220-683): a model is opened from a path with keyword
options ``temperature``, ``top_p``, ``max_tokens``, ``context_length``, generates, and is closed or used as a
context manager.  The reference's model takes text; this one takes and returns token ids (no tokenizer is
part of the library).
"""
from __future__ import annotations

import json
import math
import os
from typing import Iterator, Sequence

import numpy as np
import torch

from .csrc import ops
from .cache.paged import CacheError
from .engine.generate import GenerationOptions, GenerationResult, continue_in_slot, generate
from .engine.model import load_model, random_model
from .engine.step import Engine


class ChatContextOverflow(RuntimeError):
    """The conversation no longer fits the context; the session has been reset
    (/root/reference/bindings/python/quantcpp/__init__.py:44-60)."""


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
                 max_batch: int = 8, device: str = "cuda:0", stop_tokens: Sequence[int] | None = None,
                 f32_matrices: str = "bfloat16"):
        """``f32_matrices``: with ``dtype="bfloat16"``, matrices that the folder stores in 32 bits are rounded to
        bfloat16 as they are loaded ("bfloat16"), or stay as they are stored ("keep": their products are slow)."""
        if not os.path.isdir(path):
            raise FileNotFoundError(f"model folder not found: {path}")
        self._path = path
        self._model = load_model(path, act=dtype, device=device, f32_matrices=f32_matrices)
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
        self._chat_slot, self._chat_tokens, self.last_finish_reason = None, [], None
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
        if self._chat_slot is not None and self._engine.cache.n_free_slots == 0:
            raise RuntimeError("the conversation holds the model's only slot: reset_chat() first, or open the model "
                               "with max_batch > 1")
        opts = GenerationOptions(**{**self.options.__dict__, **overrides})
        return generate(self._engine, [list(p) for p in prompts], opts)

    def stream(self, prompt: Sequence[int], **overrides) -> Iterator[int]:
        """Yields the tokens of one continuation (the reference's ``generate`` yields text pieces)."""
        yield from self.generate(list(prompt), **overrides)

    # ------------------------------------------------------------ a conversation that keeps its cache
    def chat(self, history: Sequence[int] | None, **overrides) -> list[int]:
        """A turn of a conversation whose cache stays between calls, as the reference's ``chat``
        (/root/reference/bindings/python/quantcpp/__init__.py:514-601, /root/reference/quant.h:17634-17700): send the
        whole history every turn (token ids here); what it has in common with the tokens already in the cache is not
        run again, only the rest is, and the continuation comes back.  ``None`` ends the conversation, as
        ``reset_chat``.  Where the history parts from what the cache holds, the cache goes back to that point if it
        can (no window has dropped pages there), else the conversation starts over.  Raises
        :class:`ChatContextOverflow` (and resets) when the history does not fit the context."""
        self._ensure_open()
        if history is None:
            self.reset_chat()
            return []
        history = self._align_chat(history)
        opts = GenerationOptions(**{**self.options.__dict__, **overrides})
        try:
            res = continue_in_slot(self._engine, self._chat_slot, history, opts)
        except BaseException:
            self.reset_chat()
            raise
        self._chat_tokens = history + res.tokens
        self.last_finish_reason = res.finish_reason
        return res.tokens

    def feed(self, history: Sequence[int]) -> int:
        """Runs a history into the conversation's cache without generating (a long text read once, to be saved or
        asked about later); returns the number of tokens the cache then holds."""
        self._ensure_open()
        history = self._align_chat(history, keep_last=False)
        eng = self._engine
        rest = history[eng.length(self._chat_slot):]
        if rest:
            try:
                eng.step([self._chat_slot], [rest], [[]])
            except BaseException:
                self.reset_chat()
                raise
        self._chat_tokens = list(history)
        return eng.length(self._chat_slot)

    @property
    def chat_tokens(self) -> list[int]:
        """The tokens that the conversation's cache holds."""
        if self._chat_slot is None:
            return []
        return self._chat_tokens[:self._engine.length(self._chat_slot)]

    def _align_chat(self, history, keep_last: bool = True) -> list[int]:
        """Brings the conversation's cache to the longest beginning that it shares with ``history`` (all but the
        history's last token at most, if ``keep_last``: that one is run for its logits)."""
        history = [int(t) for t in history]
        if not history:
            raise ValueError("the history needs at least one token")
        eng = self._engine
        if len(history) >= self.context_length:
            self.reset_chat()
            raise ChatContextOverflow("conversation history exceeds the model's context window; the session has "
                                      "been reset, retry with a shorter history")
        if self._chat_slot is None:
            self._chat_slot, self._chat_tokens = eng.open(1)[0], []
        held = self._chat_tokens[:eng.length(self._chat_slot)]
        limit = min(len(held), len(history) - (1 if keep_last else 0))
        common = 0
        while common < limit and held[common] == history[common]:
            common += 1
        if common < len(held):
            try:
                eng.cache.truncate(self._chat_slot, common)
            except CacheError:
                eng.close([self._chat_slot])
                self._chat_slot = eng.open(1)[0]
        return history

    def reset_chat(self) -> None:
        """Forgets the conversation; the next ``chat`` starts afresh."""
        if self._chat_slot is not None and self._engine is not None:
            self._engine.close([self._chat_slot])
        self._chat_slot, self._chat_tokens = None, []

    def save_context(self, path: str) -> None:
        """Writes the conversation's cache and tokens to a file, as the reference's ``save_context`` does
        (/root/reference/quant.h:17518-17563; here a safetensors file: per cache group the pages the sequence holds,
        the rows of fixed-size state, and the tokens): read a long text once, ask about it in later processes."""
        self._ensure_open()
        if self._chat_slot is None:
            raise RuntimeError("there is no conversation to save")
        from .weights.safetensors_io import write_safetensors
        data = self._engine.cache.export_slot(self._chat_slot)
        tensors = {"tokens": torch.tensor(self._chat_tokens[:data["length"]], dtype=torch.int32)}
        groups = []
        for i, g in enumerate(data["groups"]):
            tensors[f"group.{i}.keys"] = g["keys"]
            if g["values"] is not None:
                tensors[f"group.{i}.values"] = g["values"]
            groups.append({"first_page": g["first_page"], "entries": g["entries"], "key": list(g["key"])})
        for e, st in data["states"].items():
            tensors[f"state.{e}"] = st
        meta = {"format": "turboquant_cpp_amd.context.1", "length": str(data["length"]), "page_size": str(data["page_size"]),
                "groups": json.dumps(groups), "dtype": self._model.act}
        write_safetensors(path, tensors, metadata=meta)

    def load_context(self, path: str) -> None:
        """Restores a conversation that ``save_context`` wrote (by a model of the same configuration and activation
        type); the next ``chat`` runs only what its history holds beyond the saved tokens
        (/root/reference/quant.h:17565-17622)."""
        self._ensure_open()
        from .weights.safetensors_io import SafetensorsFolder
        with SafetensorsFolder(os.path.dirname(path) or ".", files=[path]) as f:
            meta = f.metadata
            if meta.get("format") != "turboquant_cpp_amd.context.1":
                raise RuntimeError(f"{path} is no saved context")
            if meta.get("dtype") != self._model.act:
                raise RuntimeError(f"{path} was saved by a {meta.get('dtype')} model, this one is {self._model.act}")
            groups = []
            for i, g in enumerate(json.loads(meta["groups"])):
                values = f.read(f"group.{i}.values").clone() if f"group.{i}.values" in f.entries else None
                groups.append({"first_page": g["first_page"], "entries": g["entries"], "key": tuple(g["key"]),
                               "keys": f.read(f"group.{i}.keys").clone(), "values": values})
            states = {int(n.split(".")[1]): f.read(n).clone() for n in f.entries if n.startswith("state.")}
            tokens = f.read("tokens").tolist()
            data = {"length": int(meta["length"]), "page_size": int(meta["page_size"]), "groups": groups, "states": states}
        if len(tokens) != data["length"]:
            raise RuntimeError(f"{path} holds {len(tokens)} tokens for {data['length']} cached positions")
        V = self._engine.vocab_size
        bad = [t for t in tokens if not 0 <= t < V]
        if bad:
            raise RuntimeError(f"{path} holds token {bad[0]}, outside the vocabulary of {V}")
        if data["length"] >= self.context_length:
            raise ChatContextOverflow(f"{path} holds {data['length']} tokens, the context is {self.context_length}")
        self.reset_chat()
        try:
            self._chat_slot = self._engine.cache.import_slot(data)
        except CacheError as e:
            raise RuntimeError(f"cannot load {path}: {e}") from e
        self._chat_tokens = tokens

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
        self.reset_chat()
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
