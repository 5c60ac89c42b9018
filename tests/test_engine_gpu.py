"""The engine on the GPU against the plain implementation, in 32-bit and in bfloat16: each request alone and
whole, with the last 32 tokens one by one, in batches of unequal lengths one after another (through
``bin/trace_run``, as a user runs it); long decoding; the first tokens; generation through the entry point;
each part alone; and a toy mixer with state of its own that is registered from here.

How results are compared.  A routing decision is a comparison of two router logits, and where the plain model
(float64) finds the last expert chosen and the best one left out close together, an arithmetic with other
rounding may order them the other way; then another expert runs, and the logits of that position and of every
later position of the sequence (which attend to it) move by far more than rounding.  So wherever all positions of
a sequence are observed, results are compared with the plain model *after it has taken the engine's side at such
near-ties*, found like this (``check_sequence``): at the first position that differs, the plain model's near-ties at
that position (a chosen expert and one left out whose router logits differ by less than F32_TIE = 1e-5 of the
logits' spread in 32-bit, BF16_TIE = 0.08 in bfloat16) are decided the other way, one at a time or one in each of
two layers, and the one way that brings the position within the
bound is kept; a difference that no near-tie of that very position explains is a failure, and so is any position
that stays beyond the bound.  No position is left out.  The bounds: 1e-4 in 32-bit; in bfloat16, where every
rounding is about 2^-9 of a value, 4 % of the largest logit at every position and 1.5 % at nine in ten.
Where only some positions are observed (decoded tokens after a long prompt), near-ties of the unobserved part
cannot be found that way: 32-bit is still held to 1e-4 (the fixed seeds have no near-tie there), bfloat16 to the
looser ``check_logits``: positions with a margin under 0.02 are left out, there may not be many of them, and the
rest must lie within 10 % of the largest logit, nine in ten within 2 %.
"""
import itertools
import json
import math
import os
import shutil
import subprocess
import sys

import pytest
import torch

from plain_qwen2moe import PlainQwen2Moe, generate as plain_generate
from tiny_configs import TINY

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
SHARP = 0.1        # weights this wide make attention and routing matter; 0.02 leaves softmaxes nearly flat
ACTS = ["float32", "bfloat16"]
MARGIN = 0.02
F32_TIE = 1e-5     # routing margin under which float32 and float64 may order two experts differently
BF16_TIE = 0.08    # the same for bfloat16 activations


@pytest.fixture(scope="module")
def sharp_dirs(tmp_path_factory):
    """Model folders with wide weights, stored in the activation type they are run in."""
    from turboquant_cpp_amd.engine.model import write_random_model_dir
    made = {}

    def get(name, act):
        if (name, act) not in made:
            cfg, init = TINY[name]
            d = str(tmp_path_factory.mktemp(f"sharp_{name}_{act}"))
            write_random_model_dir(d, cfg, init["seed"], SHARP, init["norm_std"], act)
            made[(name, act)] = (d, PlainQwen2Moe(d))
        return made[(name, act)]
    return get


@pytest.fixture(scope="module")
def engines(sharp_dirs):
    from turboquant_cpp_amd.engine.model import load_model
    from turboquant_cpp_amd.engine.step import Engine
    made = {}

    def get(name, act, max_tokens=4096):
        key = (name, act, max_tokens)
        if key not in made:
            d, plain = sharp_dirs(name, act)
            made[key] = (Engine(load_model(d, act=act, device=DEV), max_tokens=max_tokens), plain)
        return made[key]
    return get


def prompts_for(name, lens, seed):
    V = TINY[name][0]["vocab_size"]
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, V, (n,), generator=g).tolist() for n in lens]


def check_logits(got, ref, margins, act, what):
    """``got`` and ``ref``: [positions, vocab]; ``margins``: routing margin of each position."""
    got, ref = got.double().cpu(), ref.double()
    assert got.shape == ref.shape, what
    err = (got - ref).abs().max(dim=-1).values
    if act == "float32":
        assert err.max() < 1e-4, f"{what}: float32 logits differ by {err.max():.2e} at position {int(err.argmax())}"
        return
    scale = ref.abs().max()
    robust = margins >= MARGIN
    assert robust.float().mean() > 0.6, f"{what}: only {robust.float().mean():.0%} of the positions have a clear routing margin"
    rel = err[robust] / scale
    assert rel.max() < 0.10, f"{what}: bfloat16 logits differ by {rel.max():.1%} of the largest logit at a position with a clear margin"
    assert rel.quantile(0.9) < 0.02, f"{what}: a tenth of the bfloat16 logits differ by more than {rel.quantile(0.9):.1%}"


def check_sequence(got, plain, prompt, act, what):
    """``got``: the engine's logits at every position of one sequence.  They must agree with the plain model once
    it has decided its near-ties as the engine did (see the top of this file).  Returns how many decisions were
    turned."""
    got = got.double().cpu()
    assert got.shape[0] == len(prompt), what
    tie = F32_TIE if act == "float32" else BF16_TIE
    plain.other_side = {}
    try:
        # the plain model's logits with no decision turned are kept per sequence: several cuts of a sequence share them
        kept = plain.__dict__.setdefault("_undecided", {})
        key = tuple(prompt)
        at_hand = key not in kept          # whether the plain model's record of margins is that of `ref`
        if at_hand:
            kept[key] = plain.logits(prompt)
        ref = kept[key]
        scale = ref.abs().max().item()
        tol = 1e-4 if act == "float32" else 0.04 * scale
        for _ in range(len(prompt)):
            err = (got - ref).abs().max(dim=-1).values
            bad = (err > tol).nonzero()
            if bad.numel() == 0:
                break
            p = int(bad[0])
            if not at_hand:
                plain.logits(prompt)
                at_hand = True
            swaps = [(l, i, j) for _gap, l, _p, i, j in plain.near_ties(tie, p) if (l, p) not in plain.other_side]
            tries = [(s,) for s in swaps] + [c for c in itertools.combinations(swaps[:6], 2) if c[0][0] != c[1][0]]
            settled = False
            for combo in tries:
                for l, i, j in combo:
                    plain.other_side[(l, p)] = (i, j)
                ref2 = plain.logits(prompt)
                if (got[p] - ref2[p]).abs().max().item() <= tol:
                    ref, settled = ref2, True
                    break
                for l, i, j in combo:
                    del plain.other_side[(l, p)]
            if not settled:
                plain.logits(prompt)
                raise AssertionError(f"{what}: {act} logits at position {p} differ by {err[p]:.2e} (bound {tol:.2e}) and no "
                                     f"near-tie of that position explains it (nearest exchanges {plain.near_ties(1.0, p)[:4]})")
        err = (got - ref).abs().max(dim=-1).values
        assert err.max() <= tol, f"{what}: position {int(err.argmax())} differs by {err.max():.2e}"
        if act != "float32":
            q90 = err.quantile(0.9).item() / scale
            assert q90 < 0.015, f"{what}: a tenth of the bfloat16 logits differ by more than {q90:.1%} of the largest logit"
        return len(plain.other_side)
    finally:
        plain.other_side = {}


def plain_rows(plain, prompt):
    ref = plain.logits(prompt)
    return ref, plain.min_margins() if plain.margins else torch.full((len(prompt),), math.inf)


# ------------------------------------------------------------------------------------------------ replay through bin/trace_run
def build_trace(prompts):
    """One trace with three ways of cutting the same requests.  Returns (lines, expectations, max_tokens):
    expectations map a step to [(request, position), ...] in the order of its output rows."""
    lines, expect, step = [], {}, 0
    live, peak = {}, 0

    def emit(entries, end):
        nonlocal step, peak
        for rid, toks, want, first in entries:
            live[rid] = live.get(rid, 0) + len(toks)
        peak = max(peak, sum(-(-n // 64) * 64 for n in live.values()))
        rows = [(rid.split(":")[1], first + w) for rid, toks, want, first in entries for w in want]
        if rows:
            expect[step] = rows
        lines.append(json.dumps({"step": step, "entries": [{"id": rid, "tokens": toks, "want": want}
                                                            for rid, toks, want, _ in entries], "end": end}))
        for rid in end:
            del live[rid]
        step += 1

    # 1. each request alone and whole
    for i, p in enumerate(prompts):
        emit([(f"w:{i}", p, list(range(len(p))), 0)], [f"w:{i}"])
    # 2. each request with its last 32 tokens one by one
    for i, p in enumerate(prompts):
        cut = max(1, len(p) - 32)
        emit([(f"d:{i}", p[:cut], list(range(cut)), 0)], [f"d:{i}"] if cut == len(p) else [])
        for t in range(cut, len(p)):
            emit([(f"d:{i}", [p[t]], [0], t)], [f"d:{i}"] if t == len(p) - 1 else [])
    # 3. batches of unequal lengths that start together, go on token by token, and whose shorter members end
    #    earlier; batch after batch, so that slots and pages are used again
    order = sorted(range(len(prompts)), key=lambda i: -len(prompts[i]))
    batches = [order[0::2], order[1::2], order[::-1][:3]]
    for b, members in enumerate(batches):
        ids = {i: f"b{b}:{i}" for i in members}
        cut = {i: max(1, len(prompts[i]) - 5 - 3 * j) for j, i in enumerate(members)}
        done = [i for i in members if cut[i] == len(prompts[i])]
        emit([(ids[i], prompts[i][:cut[i]], list(range(cut[i])), 0) for i in members], [ids[i] for i in done])
        pos = dict(cut)
        going = [i for i in members if i not in done]
        while going:
            done = [i for i in going if pos[i] == len(prompts[i]) - 1]
            emit([(ids[i], [prompts[i][pos[i]]], [0], pos[i]) for i in going], [ids[i] for i in done])
            for i in going:
                pos[i] += 1
            going = [i for i in going if i not in done]
    # 4. cuts that the step function takes beyond what the replay format promises: a prompt fed as chunks of several
    #    tokens (a run of tokens that does not start at position 0), and steps in which one request brings a whole
    #    prompt or a chunk while others go on by one token
    big = max(range(len(prompts)), key=lambda i: len(prompts[i]))
    p = prompts[big]
    a, b = max(1, len(p) // 3), max(2, 2 * len(p) // 3)
    if len(p) >= 3:
        emit([(f"m:{big}", p[:a], list(range(a)), 0)], [])
        emit([(f"m:{big}", p[a:b], list(range(b - a)), a)], [])
        emit([(f"m:{big}", p[b:], list(range(len(p) - b)), b)], [f"m:{big}"])
    others = [i for i in range(len(prompts)) if i != big and len(prompts[i]) >= 6][:2]
    if others:
        ids = {i: f"m2:{i}" for i in others}
        cut = {i: len(prompts[i]) - 4 for i in others}
        emit([(ids[i], prompts[i][:cut[i]], list(range(cut[i])), 0) for i in others], [])
        # the big request's first chunk arrives while the others decode; then its next chunk; then all go on by one
        emit([(ids[i], [prompts[i][cut[i]]], [0], cut[i]) for i in others] + [(f"m2:{big}", p[:a], list(range(a)), 0)], [])
        emit([(f"m2:{big}", p[a:b], list(range(b - a)), a)] + [(ids[i], [prompts[i][cut[i] + 1]], [0], cut[i] + 1) for i in others], [])
        emit([(ids[i], [prompts[i][cut[i] + 2]], [0], cut[i] + 2) for i in others] + [(f"m2:{big}", [p[b]], [0], b)], [])
        emit([(ids[i], [prompts[i][cut[i] + 3]], [0], cut[i] + 3) for i in others] + [(f"m2:{big}", p[b + 1:], list(range(len(p) - b - 1)), b + 1)],
             list(ids.values()) + [f"m2:{big}"])
    return lines, expect, peak


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_replay(name, act, sharp_dirs, tmp_path):
    d, plain = sharp_dirs(name, act)
    prompts = prompts_for(name, [1, 7, 33, 70, 150], seed=11)
    lines, expect, peak = build_trace(prompts)
    out = tmp_path / "out"
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", act, "--out", str(out),
           "--max-tokens", str(peak)]
    run = subprocess.run(cmd, input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done ")] == [f"done {s}" for s in range(len(lines))]
    V = TINY[name][0]["vocab_size"]
    steps_with_output = sorted(int(f[:-4]) for f in os.listdir(out) if f.endswith(".f32"))
    assert steps_with_output == sorted(expect)
    seen = {}                      # request id -> {position: logits}
    for s_, rows in expect.items():
        data = torch.frombuffer(bytearray((out / f"{s_}.f32").read_bytes()), dtype=torch.float32).view(-1, V)
        assert data.shape[0] == len(rows)
        ids = [e["id"] for e in json.loads(lines[s_])["entries"] for _ in e["want"]]
        for r, ((req, posn), rid) in enumerate(zip(rows, ids)):
            seen.setdefault(rid, {})[posn] = data[r]
    names = {"w": "whole", "d": "last 32 one by one", "b": "unequal batches", "m": "chunks", "m2": "mixed steps"}
    assert {rid.split(":")[0].rstrip("0123456789") for rid in seen} == {"w", "d", "b", "m"}
    for rid, rows in seen.items():
        tag, req = rid.split(":")
        prompt = prompts[int(req)]
        assert sorted(rows) == list(range(len(prompt))), f"{rid}: the trace does not ask for every position"
        check_sequence(torch.stack([rows[i] for i in range(len(prompt))]), plain, prompt, act,
                       f"{name} {act} {names[tag if tag == 'm2' else tag[0]]} request {req}")


# ------------------------------------------------------------------------------------------------ in process
@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_first_tokens_and_long_decoding(name, act, engines):
    eng, plain = engines(name, act)
    (seq,) = prompts_for(name, [330], seed=12)
    slot = eng.open(1)
    rows = [eng.step(slot, [seq[:3]], [[0, 1, 2]])]                 # the first tokens of a sequence, in one step
    for t in range(3, len(seq)):
        rows.append(eng.step(slot, [[seq[t]]]))
    eng.close(slot)
    check_sequence(torch.cat(rows), plain, seq, act, f"{name} {act} long decoding")
    for n in (1, 2):                                                # and as the whole of a very short sequence
        slot = eng.open(1)
        lg = eng.step(slot, [seq[:n]], [list(range(n))])
        eng.close(slot)
        check_sequence(lg, plain, seq[:n], act, f"{name} {act} first {n} tokens")


def test_the_layer_sizes_of_a_real_checkpoint(tmp_path):
    """Two layers with the sizes of Qwen1.5-MoE-A2.7B (width 2,048, 16 heads of 128, 60 experts of 1,408, top 4, a
    shared expert of 5,632; a small vocabulary) with random weights, against the plain implementation, cut three
    ways: the prompts whole in one step (one long enough for the tiled products) and then steps of one token; the
    first tokens as prompts and the last 32 of each sequence token by token, shorter sequences ending earlier; and
    the sequences in another order over two batches in slots used before, their prompts cut elsewhere and continued
    by a second chunk.  The tiny configurations of the other tests never reach the kernel variants of these sizes
    (rows of whole cache lines, waves that split k, two products in one launch, head size 128, the product that
    rotates and stores)."""
    from turboquant_cpp_amd.engine.model import load_model, write_random_model_dir
    from turboquant_cpp_amd.engine.step import Engine
    cfg = {"architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "vocab_size": 8000, "hidden_size": 2048,
           "num_hidden_layers": 2, "num_attention_heads": 16, "num_key_value_heads": 16, "intermediate_size": 5632,
           "moe_intermediate_size": 1408, "shared_expert_intermediate_size": 5632, "num_experts": 60,
           "num_experts_per_tok": 4, "norm_topk_prob": False, "decoder_sparse_step": 1, "mlp_only_layers": [],
           "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "use_sliding_window": False, "sliding_window": 32768,
           "max_window_layers": 2, "max_position_embeddings": 4096, "tie_word_embeddings": False, "torch_dtype": "float32"}
    g = torch.Generator().manual_seed(41)
    n_fed = 4
    seqs = [torch.randint(0, 8000, (n + n_fed,), generator=g).tolist() for n in (200, 70, 9)]

    def run(eng, order, cuts):
        """The sequences `order` as one batch: tokens up to cuts[i][0] as prompts, then chunks up to each further
        cut, then token by token; returns every sequence's logits at all of its positions."""
        slots = eng.open(len(order))
        rows = {i: [] for i in order}
        pos = {i: 0 for i in order}
        depth = max(len(cuts[i]) for i in order)
        for c in range(depth):
            live = [i for i in order if c < len(cuts[i])]
            lg = eng.step([slots[order.index(i)] for i in live], [seqs[i][pos[i]:cuts[i][c]] for i in live],
                          [list(range(cuts[i][c] - pos[i])) for i in live]).cpu()
            o = 0
            for i in live:
                n = cuts[i][c] - pos[i]
                rows[i].append(lg[o:o + n])
                o += n
                pos[i] = cuts[i][c]
        live = [i for i in order if pos[i] < len(seqs[i])]
        for i in order:
            if i not in live:
                eng.close([slots[order.index(i)]])
        while live:
            lg = eng.step([slots[order.index(i)] for i in live], [[seqs[i][pos[i]]] for i in live]).cpu()
            for j, i in enumerate(live):
                rows[i].append(lg[j:j + 1])
                pos[i] += 1
            for i in [i for i in live if pos[i] == len(seqs[i])]:
                eng.close([slots[order.index(i)]])
                live.remove(i)
        return {i: torch.cat(rows[i]) for i in order}

    for act in ACTS:
        d = write_random_model_dir(str(tmp_path / f"a27b_two_layers_{act}"), cfg, 3, 0.02, 0.02, act)
        plain = PlainQwen2Moe(d)
        eng = Engine(load_model(d, act=act, device=DEV), max_tokens=64 * 8)
        L = [len(s) for s in seqs]
        splits = {
            "whole prompts, then four steps": run(eng, [0, 1, 2], {i: [L[i] - n_fed] for i in range(3)}),
            "the last 32 token by token": run(eng, [0, 1, 2], {i: [max(1, L[i] - 32)] for i in range(3)}),
        }
        other = run(eng, [2, 0], {2: [5], 0: [37, 150]})
        other.update(run(eng, [1], {1: [64, 65]}))
        splits["another order, two batches, prompts in chunks"] = other
        del eng
        torch.cuda.empty_cache()
        shutil.rmtree(d)              # gigabytes of weights: not kept for the next test session to find
        for i, s in enumerate(seqs):
            first = None
            for how, got in splits.items():
                # a cut that agrees with one already checked to a tenth of the bound needs no second run of the plain model
                if first is not None and act == "float32" and (got[i] - first).abs().max() < 1e-5:
                    continue
                check_sequence(got[i], plain, s, act, f"real layer sizes, {act}, sequence of {len(s)}, {how}")
                first = got[i] if first is None else first
        del plain


def test_sixty_four_unequal_sequences_at_real_layer_sizes_in_32_bits(tmp_path):
    """The stated 32-bit workload at its stated batch: 64 sequences of 1 to 2,048 tokens drawn uniformly (seed 4), two
    layers of Qwen1.5-MoE-A2.7B's sizes, cut three ways: all prompts whole in one step; all but the last 32 tokens as
    prompts and the rest token by token, shorter sequences ending earlier; and the sequences in another order over two
    batches in slots used before, each prompt in two chunks.  The logits at each sequence's last 32 positions agree
    between the three to 2e-5; the four shortest sequences agree with the plain model at every position, and four
    longer ones (up to the longest) at their first 100, which the tokens behind them do not touch."""
    from turboquant_cpp_amd.engine.model import load_model, write_random_model_dir
    from turboquant_cpp_amd.engine.step import Engine
    V = 8000
    cfg = {"architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "vocab_size": V, "hidden_size": 2048,
           "num_hidden_layers": 2, "num_attention_heads": 16, "num_key_value_heads": 16, "intermediate_size": 5632,
           "moe_intermediate_size": 1408, "shared_expert_intermediate_size": 5632, "num_experts": 60,
           "num_experts_per_tok": 4, "norm_topk_prob": False, "decoder_sparse_step": 1, "mlp_only_layers": [],
           "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "use_sliding_window": False, "sliding_window": 32768,
           "max_window_layers": 2, "max_position_embeddings": 4096, "tie_word_embeddings": False, "torch_dtype": "float32"}
    act = "float32"
    g = torch.Generator().manual_seed(4)
    lens = torch.randint(1, 2049, (64,), generator=g).tolist()
    seqs = [torch.randint(0, V, (n,), generator=g).tolist() for n in lens]
    cut = [max(1, n - 32) for n in lens]                      # the positions from cut - 1 on are compared
    by_length = sorted(range(64), key=lambda i: lens[i])
    sample = {i: lens[i] for i in by_length[:4]}             # sequence -> its first positions that the plain model checks
    sample.update({i: 100 for i in (by_length[20], by_length[35], by_length[50], by_length[63])})
    d = write_random_model_dir(str(tmp_path / "a27b_two_layers_64"), cfg, 4, 0.02, 0.02, act)
    eng = Engine(load_model(d, act=act, device=DEV), max_tokens=sum(-(-n // 64) * 64 for n in lens), max_slots=64)

    # whole prompts in one step
    slots = eng.open(64)
    wants = [sorted(set(range(sample.get(i, 0))) | set(range(cut[i] - 1, n))) for i, n in enumerate(lens)]
    lg = eng.step(slots, seqs, wants)
    eng.close(slots)
    whole, everything, o = {}, {}, 0
    for i, w in enumerate(wants):
        rows = lg[o:o + len(w)]
        o += len(w)
        if i in sample:
            everything[i] = rows[:sample[i]].cpu()
        whole[i] = rows[len(w) - (lens[i] - cut[i] + 1):].clone()
    del lg
    # the last 32 token by token
    slots = eng.open(64)
    lg = eng.step(slots, [s[:c] for s, c in zip(seqs, cut)])
    rows = {i: [lg[i:i + 1].clone()] for i in range(64)}
    pos = list(cut)
    live = [i for i in range(64) if pos[i] < lens[i]]
    eng.close([slots[i] for i in range(64) if i not in live])
    while live:
        lg = eng.step([slots[i] for i in live], [[seqs[i][pos[i]]] for i in live])
        for j, i in enumerate(live):
            rows[i].append(lg[j:j + 1].clone())
            pos[i] += 1
        eng.close([slots[i] for i in live if pos[i] == lens[i]])
        live = [i for i in live if pos[i] < lens[i]]
    one_by_one = {i: torch.cat(r) for i, r in rows.items()}
    # another order, two batches, every prompt in two chunks
    order = torch.randperm(64, generator=g).tolist()
    chunked = {}
    for batch in (order[:32], order[32:]):
        slots = eng.open(32)
        mid = [max(1, (cut[i] - 1) // 2) if cut[i] > 1 else 0 for i in batch]      # a first chunk that ends before cut - 1
        first = [(s, i, m) for s, i, m in zip(slots, batch, mid) if m > 0]
        if first:
            eng.step([s for s, _, _ in first], [seqs[i][:m] for _, i, m in first], [[] for _ in first])
        lg = eng.step(slots, [seqs[i][m:] for i, m in zip(batch, mid)],
                      [list(range(cut[i] - 1 - m, lens[i] - m)) for i, m in zip(batch, mid)])
        o = 0
        for i in batch:
            n = lens[i] - cut[i] + 1
            chunked[i] = lg[o:o + n].clone()
            o += n
        eng.close(slots)
    assert eng.cache.n_live == 0
    worst = {"the last 32 token by token": 0.0, "another order, two batches, two chunks": 0.0}
    for i in range(64):
        for how, got in (("the last 32 token by token", one_by_one[i]), ("another order, two batches, two chunks", chunked[i])):
            assert got.shape == whole[i].shape, (how, i, got.shape, whole[i].shape)
            diff = (got - whole[i]).abs().max().item()
            worst[how] = max(worst[how], diff)
            # two cuts sum the same products in other orders (prompt and decode kernels): a fifth of what the comparison
            # with the plain model allows
            assert diff <= 2e-5, f"sequence {i} of {lens[i]} tokens, {how}: differs from the whole prompt's logits by {diff:.2e}"
    print("64 unequal sequences, float32, against the whole prompts:", worst)
    del eng
    torch.cuda.empty_cache()
    plain = PlainQwen2Moe(d)
    shutil.rmtree(d)
    for i, n in sample.items():
        check_sequence(everything[i], plain, seqs[i][:n], act,
                       f"64 unequal sequences, float32, the first {n} of sequence {i}'s {lens[i]} tokens")


@pytest.mark.parametrize("act", ACTS)
def test_a_step_fed_from_the_device_is_the_step_fed_from_the_host(act, sharp_dirs):
    """Decode steps whose tokens come from a tensor on the device (eager, captured, replayed) give the bits of the
    same steps fed from lists, and the tokens come back to the host through the fetch."""
    from turboquant_cpp_amd.engine.model import load_model
    from turboquant_cpp_amd.engine.step import Engine
    from turboquant_cpp_amd.sampling.sampler import TokenFetch
    d, _ = sharp_dirs("B", act)
    model = load_model(d, act=act, device=DEV)
    prompts = prompts_for("B", [9, 30, 17], seed=31)
    feed = prompts_for("B", [6, 6, 6], seed=32)
    out = {}
    for how in ("host", "device"):
        eng = Engine(model, max_tokens=64 * 6)
        slots = eng.open(3)
        eng.step(slots, prompts)
        fetch = TokenFetch(eng.device, 3)
        rows = []
        for t in range(6):
            toks = [f[t] for f in feed]
            if how == "host":
                rows.append(eng.step(slots, [[x] for x in toks]).clone())
            else:
                ids = torch.tensor(toks, dtype=torch.int32, device=DEV)
                fetch.start(ids)
                lg = eng.step_from_device(slots, ids)
                assert fetch.wait() == toks
                rows.append(lg.clone())
        eng.close(slots)
        out[how] = torch.stack(rows)
    assert torch.equal(out["host"], out["device"])


@pytest.mark.parametrize("act", ACTS)
def test_a_request_does_not_feel_its_batch_or_its_place_in_the_cache(act, engines):
    """Alone in a fresh cache, then among others after the cache has been used and its pages handed round:
    the same logits, far inside what bfloat16 rounding allows."""
    eng, plain = engines("B", act, max_tokens=64 * 14)
    prompts = prompts_for("B", [90, 5, 150, 40], seed=13)
    slot = eng.open(1)
    alone = torch.cat([eng.step(slot, [prompts[0][:70]], [list(range(70))])] +
                      [eng.step(slot, [[t]]) for t in prompts[0][70:]])
    eng.close(slot)
    for round_ in range(2):                                         # use the cache up and give it back
        s = eng.open(3)
        eng.step(s, [prompts[2], prompts[1], prompts[3]])
        eng.close(s)
    s = eng.open(4)
    order = [1, 0, 2, 3]
    lg = eng.step(s, [prompts[i][:70] if i == 0 else prompts[i] for i in order],
                  [list(range(70)) if i == 0 else [] for i in order])
    rows = [lg]
    eng.close([s[0], s[3]])
    for t in prompts[0][70:]:
        rows.append(eng.step([s[1], s[2]], [[t], [5]], [[0], []]))
    eng.close([s[1], s[2]])
    diff = (torch.cat(rows) - alone).abs().max().item()
    scale = alone.abs().max().item()
    if act == "float32":
        assert diff < 2e-5
    else:
        check_sequence(torch.cat(rows), plain, prompts[0], act, "in a batch")
        check_sequence(alone, plain, prompts[0], act, "alone")
    assert eng.cache.n_live == 0


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("name", ["A", "B"])
def test_generation_through_the_entry_point(name, act, sharp_dirs):
    from turboquant_cpp_amd import Model
    d, plain = sharp_dirs(name, act)
    prompts = prompts_for(name, [4, 1, 30, 9, 17], seed=14)
    with Model(d, dtype=act, temperature=0.0, rep_penalty=1.0, max_tokens=12, max_batch=3, stop_tokens=()) as m:
        got = m.generate(prompts, loop_detection=False)
        single = m.generate(prompts[2], loop_detection=False)
        assert single == got[2]
        with_penalty = m.generate(prompts[:2], rep_penalty=1.5, loop_detection=False)
    assert all(len(g) == 12 for g in got)
    if act == "float32":
        assert got == [plain_generate(plain, p, max_tokens=12) for p in prompts]
        assert with_penalty == [plain_generate(plain, p, max_tokens=12, rep_penalty=1.5) for p in prompts[:2]]
    else:
        # every token the engine chose is, by the plain model's logits for the same history, the best or
        # within rounding of the best
        for p, g in zip(prompts, got):
            ref = plain.logits(p + g)
            for j, tok in enumerate(g):
                row = ref[len(p) - 1 + j]
                assert row[tok] >= row.max() - 0.05 * ref.abs().max(), (name, j)


def test_sampling_through_the_entry_point_follows_the_plain_loop(sharp_dirs):
    from turboquant_cpp_amd import Model
    d, plain = sharp_dirs("A", "float32")
    prompts = prompts_for("A", [6, 2], seed=15)
    with Model(d, dtype="float32", temperature=0.8, top_p=0.9, max_tokens=10, seed=9, rep_penalty=1.1,
               stop_tokens=(), max_batch=1) as m:
        got = [m.generate(p, loop_detection=False) for p in prompts]
        again = [m.generate(p, loop_detection=False) for p in prompts]
        other = m.generate(prompts[0], seed=10, loop_detection=False)
    want = [plain_generate(plain, p, max_tokens=10, temperature=0.8, top_p=0.9, seed=9, rep_penalty=1.1) for p in prompts]
    assert got == want and again == got and other != got[0]


def test_stop_tokens_of_the_configuration_end_generation(sharp_dirs):
    from turboquant_cpp_amd import Model
    d, plain = sharp_dirs("B", "float32")
    (p,) = prompts_for("B", [8], seed=16)
    free = plain_generate(plain, p, max_tokens=20)
    with Model(d, dtype="float32", temperature=0.0, rep_penalty=1.0, max_tokens=20) as m:
        assert m.options.stop_tokens == (7, 11)                     # eos_token_id of config.json
        r = m.generate_detailed([p], stop_tokens=(free[6],), loop_detection=False)[0]
    assert r.tokens == free[:free.index(free[6])] and r.finish_reason == "stop"


# ------------------------------------------------------------------------------------------------ each part alone
def part_context(part_needs, lens, act, starts=None):
    """A cache and a packed step for one part: sequences of the given lengths, each in its own slot."""
    from turboquant_cpp_amd.cache import PagedCache
    from turboquant_cpp_amd.engine.batch import pack_step
    from turboquant_cpp_amd.engine.context import StepContext
    dtype = torch.float32 if act == "float32" else torch.bfloat16
    cache = PagedCache(part_needs, 64 * 16, dtype, torch.device(DEV), page_size=64)
    slots = [cache.open() for _ in lens]
    slots = slots[::-1]
    starts = [cache.reserve(s, n) for s, n in zip(slots, lens)]
    cache.sync()
    batch = pack_step(slots, starts, [[0] * n for n in lens], [[] for _ in lens], DEV)
    return StepContext(batch=batch, cache=cache, act=act, device=torch.device(DEV)), cache, slots


def wdt(act):
    return torch.float32 if act == "float32" else torch.bfloat16


def rnd(shape, act, seed, scale=1.0):
    return (scale * torch.randn(shape, generator=torch.Generator().manual_seed(seed))).to(wdt(act))


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("out_bias,qk_norm", [(False, False), (True, False), (True, True)])
def test_attention_part_alone(act, out_bias, qk_norm):
    import plain_qwen2moe as P
    from turboquant_cpp_amd.config import PartSpec
    from turboquant_cpp_amd.parts import build_part
    H, nh, nkv, hd, window = 80, 6, 3, 16, 20
    spec = PartSpec("gqa_attention", dict(hidden_size=H, num_heads=nh, num_kv_heads=nkv, head_dim=hd, qkv_bias=True,
                                          out_bias=out_bias, qk_norm_eps=1e-3 if qk_norm else None, window=window, position=PartSpec("rope", dict(head_dim=hd, rotary_dim=hd,
                                                                                        theta=5000.0, pairing="interleaved"))))
    part = build_part("mixer", spec)
    specs = part.param_specs()
    assert specs["qkv_weight"].shape == ((nh + 2 * nkv) * hd, H) and specs["qkv_weight"].splits == (96, 48, 48)
    assert ("out_bias" in specs) == out_bias and ("q_norm" in specs) == qk_norm == ("k_norm" in specs)
    w = {n: rnd(s.shape, act, 20 + i, 0.3) for i, (n, s) in enumerate(specs.items())}
    part.set_params({n: t.to(DEV) for n, t in w.items()})
    lens = [50, 1, 27]
    ctx, cache, slots = part_context([(part.cache_need(), None, None)], lens, act)
    x = rnd((sum(lens), H), act, 30)
    y = part.forward(x.to(DEV), ctx, 0)
    assert y.shape[1:] == (sum(lens), H) and y.dtype == torch.float32
    y = y.double().sum(dim=0, keepdim=True)         # the partial sums that the next norm would add up
    o = 0
    for n in lens:
        xs = x[o:o + n].double()
        qkv = xs @ w["qkv_weight"].double().T + w["qkv_bias"].double()
        q, k, v = qkv[:, :96].view(n, nh, hd), qkv[:, 96:144].view(n, nkv, hd), qkv[:, 144:].view(n, nkv, hd)
        if qk_norm:         # every head by itself, before the rotation
            q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + 1e-3) * w["q_norm"].double()
            k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + 1e-3) * w["k_norm"].double()
        pos = list(range(n))
        att = P.attention(P.rope(q, pos, 5000.0, "interleaved"), P.rope(k, pos, 5000.0, "interleaved"), v, window=window)
        ref = att.reshape(n, nh * hd) @ w["out_weight"].double().T
        if out_bias:
            ref = ref + w["out_bias"].double()
        err = (y[0, o:o + n].cpu().double() - ref).abs().max() / ref.abs().max()
        assert err < (1e-5 if act == "float32" else 3e-2)
        o += n


@pytest.mark.parametrize("act", ACTS)
def test_feed_forward_parts_alone(act):
    import plain_qwen2moe as P
    from turboquant_cpp_amd.config import PartSpec
    from turboquant_cpp_amd.parts import build_part
    H, T = 72, 23
    ctx, _, _ = part_context([(None, None, None)], [T], act)
    x = rnd((T, H), act, 40)
    dense = build_part("ffn", PartSpec("dense_swiglu", dict(hidden_size=H, inner_size=104)))
    w = {n: rnd(s.shape, act, 41 + i, 0.2) for i, (n, s) in enumerate(dense.param_specs().items())}
    dense.set_params({n: t.to(DEV) for n, t in w.items()})
    y = dense.forward(x.to(DEV), None, ctx)[0].cpu().double()
    ref = P.swiglu_mlp(x.double(), w["gate"].double(), w["up"].double(), w["down"].double())
    assert (y - ref).abs().max() / ref.abs().max() < (1e-5 if act == "float32" else 2e-2)
    for renorm, shared in ((False, 40), (True, 0)):
        moe = build_part("ffn", PartSpec("moe_swiglu", dict(hidden_size=H, num_experts=7, top_k=3, expert_size=24,
                                                            shared_size=shared, renormalize=renorm)))
        assert moe.wants_f32 and ("shared_scale" in moe.param_specs()) == (shared > 0)
        w = {n: rnd(s.shape, act, 50 + i, 0.3) for i, (n, s) in enumerate(moe.param_specs().items())}
        moe.set_params({n: t.to(DEV) for n, t in w.items()})
        unsummed = moe.forward(x.to(DEV), x.float().to(DEV), ctx)
        y = unsummed.materialize(act)[0].cpu().double()
        # the next norm sums it in its own pass: the same bits as summing first
        norm = build_part("norm", PartSpec("rmsnorm", dict(size=H, eps=1e-5)))
        norm.set_params({"weight": rnd((H,), act, 77, 0.5).to(DEV)})
        stream_a, stream_b = x.float().to(DEV).clone(), x.float().to(DEV).clone()
        fused = norm.forward(stream_a, unsummed, ctx, want_f32=True)[1]
        apart = norm.forward(stream_b, unsummed.materialize(act), ctx, want_f32=True)[1]
        assert torch.equal(fused, apart) and torch.equal(stream_a, stream_b)
        pw = {"router": w["router"].double(),
              "experts": [{"gate": w["expert_gate"][e].double(), "up": w["expert_up"][e].double(),
                           "down": w["expert_down"][e].double()} for e in range(7)]}
        if shared:
            pw["shared"] = {"gate": w["shared_gate"].double(), "up": w["shared_up"].double(), "down": w["shared_down"].double()}
            pw["shared_scale"] = w["shared_scale"].double()
        ref = P.moe(x.double(), pw, 3, renorm)
        assert (y - ref).abs().max() / ref.abs().max() < (1e-5 if act == "float32" else 2e-2)


@pytest.mark.parametrize("act", ACTS)
def test_norm_and_position_parts_alone(act):
    import plain_qwen2moe as P
    from turboquant_cpp_amd.config import PartSpec
    from turboquant_cpp_amd.parts import build_part
    norm = build_part("norm", PartSpec("rmsnorm", dict(size=100, eps=1e-3)))
    w = rnd((100,), act, 60) + 1
    norm.set_params({"weight": w.to(DEV)})
    ctx, _, _ = part_context([(None, None, None)], [9], act)
    x, delta = torch.randn(9, 100), torch.randn(2, 9, 100)
    xd = x.clone().to(DEV)
    out, out32 = norm.forward(xd, delta.to(DEV), ctx, want_f32=True)
    ref = P.rmsnorm(x.double() + delta.double().sum(0), w.double(), 1e-3)
    assert (out32.cpu().double() - ref).abs().max() < 1e-4 and out.dtype == wdt(act)
    assert (xd.cpu().double() - (x.double() + delta.double().sum(0))).abs().max() < 1e-5
    rope = build_part("position", PartSpec("rope", dict(head_dim=48, rotary_dim=32, theta=1e6, pairing="half")))
    assert rope.pairing_code == 0 and rope.rotary_dim == 32
    assert torch.equal(rope.table(DEV).cpu(), torch.from_numpy(P.rope_frequencies(32, 1e6)))
    with pytest.raises(ValueError, match="pairing"):
        build_part("position", PartSpec("rope", dict(head_dim=8, rotary_dim=8, theta=1.0, pairing="odd")))
    with pytest.raises(ValueError, match="unknown norm"):
        build_part("norm", PartSpec("layernorm", {}))


# ------------------------------------------------------------------------------------------------ a toy mixer with state
def test_a_mixer_with_state_of_its_own_is_registered_built_and_stepped():
    """A recurrent mixer defined here: per sequence a state s of the model's width, s <- decay * s + x W_in for
    every token in order, output s W_out.  It keeps no keys or values, only its state in the cache's fixed-size
    area.  Registered, put into a model by a plan, loaded and stepped through the engine without touching the
    library's files; whole prompts, token by token and unequal batches must agree with a plain loop."""
    from turboquant_cpp_amd.config import LayerSpec, ModelPlan, PartSpec, ScheduleEntry, Source
    from turboquant_cpp_amd.engine.model import CausalLM
    from turboquant_cpp_amd.engine.step import Engine
    from turboquant_cpp_amd.parts import ParamSpec, Part, StateNeed, register_part, unregister_part
    from turboquant_cpp_amd.weights import TensorDict

    H, V, INNER, L = 48, 90, 64, 2

    class ToyDecayMixer(Part):
        graph_safe = True          # its decode steps reach the state through the slots on the device

        def __init__(self, hidden_size, decay):
            self.hidden_size, self.decay = hidden_size, decay
            self.w_in = self.w_out = None

        def param_specs(self):
            return {"w_in": ParamSpec((self.hidden_size, self.hidden_size)), "w_out": ParamSpec((self.hidden_size, self.hidden_size))}

        def cache_need(self):
            return None

        def state_need(self):
            return StateNeed((self.hidden_size,), torch.float32)

        def forward(self, normed, ctx, entry):
            u = normed.float() @ self.w_in.float().T
            b = ctx.batch
            if b.is_decode:                                        # one token per sequence: advance every state by one
                s = self.decay * ctx.state_rows(entry) + u
                ctx.store_state_rows(entry, s)
                return (s @ self.w_out.float().T).unsqueeze(0)
            state = ctx.state(entry)                               # [slots, H]; zero for a new sequence
            out = torch.empty_like(u)
            o = 0
            for slot, n in zip(b.slots, b.n_new):                  # a scan over each sequence's new tokens
                s = state[slot]
                for t in range(o, o + n):
                    s = self.decay * s + u[t]
                    out[t] = s
                state[slot] = s
                o += n
            return (out @ self.w_out.float().T).unsqueeze(0)

    register_part("mixer", "toy_decay")(ToyDecayMixer)
    try:
        def norm(name):
            return PartSpec("rmsnorm", dict(size=H, eps=1e-5), {"weight": Source.single(name)})
        layers = [LayerSpec("prenorm", {
            "mixer_norm": norm(f"l{l}.n1"), "ffn_norm": norm(f"l{l}.n2"),
            "mixer": PartSpec("toy_decay", dict(hidden_size=H, decay=0.5 + 0.2 * l),
                              {"w_in": Source.single(f"l{l}.in"), "w_out": Source.single(f"l{l}.out")}),
            "ffn": PartSpec("dense_swiglu", dict(hidden_size=H, inner_size=INNER),
                            {n: Source.single(f"l{l}.{n}") for n in ("gate", "up", "down")})}) for l in range(L)]
        plan = ModelPlan("ToyRecurrentLM", V, H, layers, [ScheduleEntry(l) for l in range(L)], norm("final"),
                         Source.single("embed"), None, max_positions=512)
        model = CausalLM(plan, "float32")
        g = torch.Generator().manual_seed(70)
        tensors = {n: (torch.ones(s) if role == "scale" else 0.3 * torch.randn(s, generator=g))
                   for n, (s, role) in model.tensor_table().items()}
        model.load(TensorDict(tensors), DEV)
        eng = Engine(model, max_tokens=64 * 4, max_slots=3)
        assert eng.cache.groups == [] and sorted(eng.cache.states) == [0, 1]
        assert eng.graphs.replayable(2)

        def plain(tokens):
            import plain_qwen2moe as P
            t = {n: v.double() for n, v in tensors.items()}
            x = t["embed"][tokens]
            for l in range(L):
                u = P.rmsnorm(x, t[f"l{l}.n1"], 1e-5) @ t[f"l{l}.in"].T
                s, ys = torch.zeros(H, dtype=torch.float64), []
                for i in range(len(tokens)):
                    s = (0.5 + 0.2 * l) * s + u[i]
                    ys.append(s)
                x = x + torch.stack(ys) @ t[f"l{l}.out"].T
                x = x + P.swiglu_mlp(P.rmsnorm(x, t[f"l{l}.n2"], 1e-5), t[f"l{l}.gate"], t[f"l{l}.up"], t[f"l{l}.down"])
            return P.rmsnorm(x, t["final"], 1e-5) @ t["embed"].T

        prompts = [torch.randint(0, V, (n,), generator=g).tolist() for n in (9, 1, 20)]
        refs = [plain(p) for p in prompts]
        slots = eng.open(3)
        lg = eng.step(slots, prompts, [list(range(len(p))) for p in prompts]).cpu().double()
        assert (lg - torch.cat(refs)).abs().max() < 1e-4
        eng.close(slots)
        # token by token in an unequal batch, in slots that have been used: state must start from zero again
        slots = eng.open(3)
        cut = [4, 1, 11]
        eng.step(slots, [p[:c] for p, c in zip(prompts, cut)], [[] for _ in prompts])
        pos, live = list(cut), [0, 2]
        eng.close([slots[1]])
        while live:
            lg = eng.step([slots[i] for i in live], [[prompts[i][pos[i]]] for i in live]).cpu().double()
            for j, i in enumerate(live):
                assert (lg[j] - refs[i][pos[i]]).abs().max() < 1e-4
                pos[i] += 1
            for i in [i for i in live if pos[i] == len(prompts[i])]:
                eng.close([slots[i]])
                live.remove(i)
        assert eng.cache.n_live == 0
        assert len(eng.graphs.graphs) >= 1, "the decode steps of the stateful mixer were not replayed"
        # replayed steps give the bits of eager ones, with other slots behind the same graph
        slow = Engine(model, max_tokens=64 * 4, max_slots=3, use_graphs=False)
        for order in ([0, 2], [2, 0]):
            sf, ss = eng.open(3), slow.open(3)
            for e, sl in ((eng, sf), (slow, ss)):
                e.step([sl[i] for i in order], [prompts[i][:4] for i in order], [[], []])
            for t in range(4, 9):
                a = eng.step([sf[i] for i in order], [[prompts[i][t]] for i in order])
                b_ = slow.step([ss[i] for i in order], [[prompts[i][t]] for i in order])
                assert torch.equal(a, b_), f"replayed step {t} differs from the eager one"
            eng.close(sf), slow.close(ss)
        # a sequence that leaves the cache and comes back (its rows of state with it) goes on as if it had stayed;
        # it cannot go back to an earlier position, having no earlier state
        from turboquant_cpp_amd.cache.paged import CacheError
        (a,) = eng.open(1)
        eng.step([a], [prompts[2][:12]], [[]])
        saved = eng.cache.export_slot(a)
        assert saved["length"] == 12 and sorted(saved["states"]) == [0, 1] and saved["groups"] == []
        with pytest.raises(CacheError, match="state"):
            eng.cache.truncate(a, 5)
        eng.close([a])
        (other,) = eng.open(1)                                    # takes the slot and leaves its own state there
        eng.step([other], [prompts[0]], [[]])
        eng.close([other])
        b_ = eng.cache.import_slot(saved)
        assert eng.length(b_) == 12
        lg = eng.step([b_], [prompts[2][12:]], [list(range(8))]).cpu().double()
        assert (lg - refs[2][12:]).abs().max() < 1e-4
        eng.close([b_])
    finally:
        unregister_part("mixer", "toy_decay")


@pytest.mark.parametrize("act", ACTS)
def test_the_order_of_layers_is_a_list(act):
    """A plan of the library's own parts whose schedule names layers twice: layer 0, layer 1, layer 0 again with keys
    and values of its own for that run, and layer 1 again reading the keys and values that its first run wrote
    (it writes none).  Whole prompts in an unequal batch and token by token in slots used before, against a plain
    loop over the same list; the cache holds three runs' worth of keys and values, not four."""
    import plain_qwen2moe as P
    from turboquant_cpp_amd.config import LayerSpec, ModelPlan, PartSpec, ScheduleEntry, Source
    from turboquant_cpp_amd.engine.model import CausalLM
    from turboquant_cpp_amd.engine.step import Engine
    from turboquant_cpp_amd.weights import TensorDict
    H, V, INNER, nh, nkv, hd, theta = 64, 120, 96, 4, 2, 16, 10000.0
    windows = [None, 12]

    def norm(name):
        return PartSpec("rmsnorm", dict(size=H, eps=1e-5), {"weight": Source.single(name)})
    layers = [LayerSpec("prenorm", {
        "mixer_norm": norm(f"l{l}.n1"), "ffn_norm": norm(f"l{l}.n2"),
        "mixer": PartSpec("gqa_attention", dict(hidden_size=H, num_heads=nh, num_kv_heads=nkv, head_dim=hd, qkv_bias=True,
                                                window=windows[l],
                                                position=PartSpec("rope", dict(head_dim=hd, rotary_dim=hd, theta=theta, pairing="half"))),
                          {"qkv_weight": Source.concat([f"l{l}.q", f"l{l}.k", f"l{l}.v"]),
                           "qkv_bias": Source.concat([f"l{l}.qb", f"l{l}.kb", f"l{l}.vb"]), "out_weight": Source.single(f"l{l}.o")}),
        "ffn": PartSpec("dense_swiglu", dict(hidden_size=H, inner_size=INNER),
                        {n: Source.single(f"l{l}.{n}") for n in ("gate", "up", "down")})}) for l in range(2)]
    schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1, cache_of=1)]
    plan = ModelPlan("ToyLoopedLM", V, H, layers, schedule, norm("final"), Source.single("embed"), None, max_positions=512)
    model = CausalLM(plan, act)
    g = torch.Generator().manual_seed(81)
    dt = torch.float32 if act == "float32" else torch.bfloat16
    tensors = {n: ((1 + 0.1 * torch.randn(sh, generator=g)) if role == "scale" else 0.12 * torch.randn(sh, generator=g)).to(dt)
               for n, (sh, role) in model.tensor_table().items()}
    model.load(TensorDict(tensors), DEV)
    eng = Engine(model, max_tokens=64 * 6, max_slots=3)
    # runs 0, 1 and 2 keep keys and values (run 1 with a window), run 3 keeps none
    assert sum(len(grp.entries) for grp in eng.cache.groups) == 3

    def plain(tokens):
        t = {n: v.double() for n, v in tensors.items()}
        n, pos = len(tokens), list(range(len(tokens)))
        x = t["embed"][tokens]
        kept = {}
        for run, e in enumerate(schedule):
            l = e.layer
            h = P.rmsnorm(x, t[f"l{l}.n1"], 1e-5)
            q = (h @ t[f"l{l}.q"].T + t[f"l{l}.qb"]).view(n, nh, hd)
            if e.cache_of is None:
                k = (h @ t[f"l{l}.k"].T + t[f"l{l}.kb"]).view(n, nkv, hd)
                v = (h @ t[f"l{l}.v"].T + t[f"l{l}.vb"]).view(n, nkv, hd)
                kept[run] = (P.rope(k, pos, theta, "half"), v)
            k, v = kept[run if e.cache_of is None else e.cache_of]
            att = P.attention(P.rope(q, pos, theta, "half"), k, v, window=windows[l])
            x = x + att.reshape(n, nh * hd) @ t[f"l{l}.o"].T
            x = x + P.swiglu_mlp(P.rmsnorm(x, t[f"l{l}.n2"], 1e-5), t[f"l{l}.gate"], t[f"l{l}.up"], t[f"l{l}.down"])
        return P.rmsnorm(x, t["final"], 1e-5) @ t["embed"].T

    prompts = [torch.randint(0, V, (n,), generator=g).tolist() for n in (70, 3, 31)]
    refs = [plain(p) for p in prompts]
    bound = 1e-4 if act == "float32" else 0.04 * max(r.abs().max().item() for r in refs)
    slots = eng.open(3)
    lg = eng.step(slots, prompts, [list(range(len(p))) for p in prompts]).cpu().double()
    assert (lg - torch.cat(refs)).abs().max() < bound
    eng.close(slots)
    slots = eng.open(3)
    cut = [40, 1, 9]
    eng.step(slots, [p[:c] for p, c in zip(prompts, cut)], [[] for _ in prompts])
    pos, live = list(cut), [0, 1, 2]
    while live:
        lg = eng.step([slots[i] for i in live], [[prompts[i][pos[i]]] for i in live]).cpu().double()
        for j, i in enumerate(live):
            assert (lg[j] - refs[i][pos[i]]).abs().max() < bound, (i, pos[i])
            pos[i] += 1
        for i in [i for i in live if pos[i] == len(prompts[i])]:
            eng.close([slots[i]])
            live.remove(i)
    assert eng.cache.n_live == 0


def test_a_feed_forward_with_routing_and_another_position_encoding_defined_here():
    """Two more parts defined in the test and registered from here: a feed-forward that sends each token to one of
    four small experts (chosen by the largest of four router scores, relu inside), and a position encoding whose
    angles grow linearly with the pair index and turn only half of each head, in interleaved pairs.  The library's
    attention part takes the encoding by its table alone; layer 1 uses the library's own encoding and a window.
    Whole prompts, token by token and a batch must agree with a plain loop."""
    import plain_qwen2moe as P
    from turboquant_cpp_amd.config import LayerSpec, ModelPlan, PartSpec, ScheduleEntry, Source
    from turboquant_cpp_amd.engine.model import CausalLM
    from turboquant_cpp_amd.engine.step import Engine
    from turboquant_cpp_amd.parts import ParamSpec, Part, register_part, unregister_part
    from turboquant_cpp_amd.weights import TensorDict

    H, V, NH, NKV, HD, E, I, L = 40, 70, 4, 2, 16, 4, 24, 2
    ROT, F0, F1 = 8, 0.9, 0.05

    class ToyLinearAngles(Part):
        pairing = "interleaved"
        pairing_code = 1

        def __init__(self, rotary_dim, first, last):
            self.rotary_dim, self.first, self.last = rotary_dim, first, last

        def table(self, device):
            return torch.linspace(self.first, self.last, self.rotary_dim // 2, dtype=torch.float32).to(device)

    class ToyOneOfFour(Part):
        wants_f32 = False

        def __init__(self, hidden_size, experts, inner_size):
            self.hidden_size, self.experts, self.inner_size = hidden_size, experts, inner_size
            self.router = self.w1 = self.w2 = None

        def param_specs(self):
            return {"router": ParamSpec((self.experts, self.hidden_size)),
                    "w1": ParamSpec((self.experts, self.inner_size, self.hidden_size)),
                    "w2": ParamSpec((self.experts, self.hidden_size, self.inner_size))}

        def forward(self, normed, normed32, ctx):
            x = normed.float()
            pick = (x @ self.router.float().T).argmax(dim=-1)
            h = torch.relu(torch.einsum("th,tih->ti", x, self.w1.float()[pick]))
            return torch.einsum("ti,thi->th", h, self.w2.float()[pick]).unsqueeze(0)

    register_part("position", "toy_linear")(ToyLinearAngles)
    register_part("ffn", "toy_one_of_four")(ToyOneOfFour)
    try:
        def norm(name):
            return PartSpec("rmsnorm", dict(size=H, eps=1e-6), {"weight": Source.single(name)})
        positions = [PartSpec("toy_linear", dict(rotary_dim=ROT, first=F0, last=F1)),
                     PartSpec("rope", dict(head_dim=HD, rotary_dim=HD, theta=100.0, pairing="half"))]
        windows = [None, 5]
        layers = [LayerSpec("prenorm", {
            "mixer_norm": norm(f"l{l}.n1"), "ffn_norm": norm(f"l{l}.n2"),
            "mixer": PartSpec("gqa_attention", dict(hidden_size=H, num_heads=NH, num_kv_heads=NKV, head_dim=HD,
                                                    position=positions[l], window=windows[l]),
                              {"qkv_weight": Source.concat([f"l{l}.q", f"l{l}.k", f"l{l}.v"]), "out_weight": Source.single(f"l{l}.o")}),
            "ffn": PartSpec("toy_one_of_four", dict(hidden_size=H, experts=E, inner_size=I),
                            {n: Source.single(f"l{l}.{n}") for n in ("router", "w1", "w2")})}) for l in range(L)]
        plan = ModelPlan("ToyRoutedLM", V, H, layers, [ScheduleEntry(l) for l in range(L)], norm("final"),
                         Source.single("embed"), None, max_positions=256)
        model = CausalLM(plan, "float32")
        g = torch.Generator().manual_seed(80)
        tensors = {n: (torch.ones(s) if role == "scale" else 0.4 * torch.randn(s, generator=g))
                   for n, (s, role) in model.tensor_table().items()}
        model.load(TensorDict(tensors), DEV)
        eng = Engine(model, max_tokens=64 * 6, max_slots=3)
        assert not eng.graphs.replayable(2) and not eng.graphs.graphs   # parts that do not say they are safe for replay keep their model's steps eager
        assert len(eng.cache.groups) == 2  # the windowed layer has storage of its own

        def turn(x, angles_per_step, pairing, rot):      # x [T, heads, hd]
            T = x.shape[0]
            ang = (torch.arange(T, dtype=torch.float32)[:, None] * angles_per_step[None, :]).double()
            cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            out = x.clone()
            if pairing == "interleaved":
                a, b = x[..., 0:rot:2], x[..., 1:rot:2]
                out[..., 0:rot:2], out[..., 1:rot:2] = a * cos - b * sin, a * sin + b * cos
            else:
                a, b = x[..., :rot // 2], x[..., rot // 2:rot]
                out[..., :rot // 2], out[..., rot // 2:rot] = a * cos - b * sin, a * sin + b * cos
            return out

        def plain(tokens):
            t = {n: v.double() for n, v in tensors.items()}
            x = t["embed"][tokens]
            T = len(tokens)
            tables = [torch.linspace(F0, F1, ROT // 2, dtype=torch.float32), torch.from_numpy(P.rope_frequencies(HD, 100.0))]
            for l in range(L):
                xb = P.rmsnorm(x, t[f"l{l}.n1"], 1e-6)
                q = (xb @ t[f"l{l}.q"].T).view(T, NH, HD)
                k = (xb @ t[f"l{l}.k"].T).view(T, NKV, HD)
                v = (xb @ t[f"l{l}.v"].T).view(T, NKV, HD)
                pairing, rot = ("interleaved", ROT) if l == 0 else ("half", HD)
                q, k = turn(q, tables[l], pairing, rot), turn(k, tables[l], pairing, rot)
                x = x + P.attention(q, k, v, window=windows[l]).reshape(T, NH * HD) @ t[f"l{l}.o"].T
                xb = P.rmsnorm(x, t[f"l{l}.n2"], 1e-6)
                pick = (xb @ t[f"l{l}.router"].T).argmax(dim=-1)
                ys = [t[f"l{l}.w2"][e] @ torch.relu(t[f"l{l}.w1"][e] @ xb[i]) for i, e in enumerate(pick.tolist())]
                x = x + torch.stack(ys)
            return P.rmsnorm(x, t["final"], 1e-6) @ t["embed"].T

        prompts = [torch.randint(0, V, (n,), generator=g).tolist() for n in (12, 3, 17)]
        refs = [plain(p) for p in prompts]
        slots = eng.open(3)
        lg = eng.step(slots, prompts, [list(range(len(p))) for p in prompts]).cpu().double()
        assert (lg - torch.cat(refs)).abs().max() < 2e-4
        eng.close(slots)
        slots = eng.open(2)                    # prefix, then token by token, in slots that were used before
        eng.step(slots, [prompts[0][:5], prompts[2][:9]], [[], []])
        for i in range(7):
            lg = eng.step(slots, [[prompts[0][5 + i]], [prompts[2][9 + i]]]).cpu().double()
            assert (lg[0] - refs[0][5 + i]).abs().max() < 2e-4 and (lg[1] - refs[2][9 + i]).abs().max() < 2e-4
        eng.close(slots)
        assert eng.cache.n_live == 0
    finally:
        unregister_part("position", "toy_linear")
        unregister_part("ffn", "toy_one_of_four")


def test_a_mixer_that_keeps_one_row_per_position_and_a_scaled_embedding_with_capped_logits():
    """A toy mixer defined here that keeps a single latent row per position (keys only, no value pool: ``value_dim``
    0) and attends over those rows, in a model whose plan scales the embedding and soft-caps the logits; the dense
    feed-forward takes another activation than silu.  None of this touches the framework's files."""
    import plain_qwen2moe as P
    from turboquant_cpp_amd.config import LayerSpec, ModelPlan, PartSpec, ScheduleEntry, Source
    from turboquant_cpp_amd.engine.model import CausalLM
    from turboquant_cpp_amd.engine.step import Engine
    from turboquant_cpp_amd.parts import CacheNeed, ParamSpec, Part, register_part, unregister_part
    from turboquant_cpp_amd.weights import TensorDict

    H, V, LAT, INNER, L = 40, 60, 24, 56, 2
    SCALE, CAP = 3.0, 2.5

    class ToyLatentMixer(Part):
        def __init__(self, hidden_size, latent):
            self.hidden_size, self.latent = hidden_size, latent
            self.w_q = self.w_c = self.w_o = None

        def param_specs(self):
            return {"w_q": ParamSpec((self.latent, self.hidden_size)), "w_c": ParamSpec((self.latent, self.hidden_size)),
                    "w_o": ParamSpec((self.hidden_size, self.latent))}

        def cache_need(self):
            return CacheNeed(1, self.latent, None, value_dim=0)

        def state_need(self):
            return None

        def forward(self, normed, ctx, entry):
            kv, b = ctx.kv(entry), ctx.batch
            assert kv.v_pages is None and kv.value_dim == 0
            x = normed.float()
            q, c = x @ self.w_q.float().T, x @ self.w_c.float().T
            table = kv.table.cpu()
            pages = kv.k_pages.view(-1, kv.page_stride)
            out, o = torch.empty_like(q), 0
            for slot, start, n in zip(b.slots, b.start, b.n_new):
                for j in range(n):                     # the new rows go into the sequence's pages
                    pos = start + j
                    off = kv.layer_offset + (pos % kv.page_size) * self.latent
                    pages[int(table[slot, pos // kv.page_size]), off:off + self.latent] = c[o + j].to(pages.dtype)
                rows = torch.stack([pages[int(table[slot, p // kv.page_size]),
                                          kv.layer_offset + (p % kv.page_size) * self.latent:][:self.latent]
                                    for p in range(start + n)]).float()
                for j in range(n):
                    seen = rows[:start + j + 1]
                    out[o + j] = torch.softmax(seen @ q[o + j] / self.latent ** 0.5, dim=0) @ seen
                o += n
            return (out @ self.w_o.float().T).unsqueeze(0)

    register_part("mixer", "toy_latent")(ToyLatentMixer)
    try:
        def norm(name):
            return PartSpec("rmsnorm", dict(size=H, eps=1e-6), {"weight": Source.single(name)})
        layers = [LayerSpec("prenorm", {
            "mixer_norm": norm(f"l{l}.n1"), "ffn_norm": norm(f"l{l}.n2"),
            "mixer": PartSpec("toy_latent", dict(hidden_size=H, latent=LAT),
                              {n: Source.single(f"l{l}.{n}") for n in ("w_q", "w_c", "w_o")}),
            "ffn": PartSpec("dense_swiglu", dict(hidden_size=H, inner_size=INNER, activation="gelu_tanh"),
                            {n: Source.single(f"l{l}.{n}") for n in ("gate", "up", "down")})}) for l in range(L)]
        plan = ModelPlan("ToyLatentLM", V, H, layers, [ScheduleEntry(l) for l in range(L)], norm("final"),
                         Source.single("embed"), None, max_positions=256, embedding_scale=SCALE, logit_softcap=CAP)
        model = CausalLM(plan, "float32")
        g = torch.Generator().manual_seed(90)
        tensors = {n: (torch.ones(s) if role == "scale" else 0.3 * torch.randn(s, generator=g))
                   for n, (s, role) in model.tensor_table().items()}
        model.load(TensorDict(tensors), DEV)
        eng = Engine(model, max_tokens=64 * 6, max_slots=3)
        (group,) = eng.cache.groups
        assert group.v_pages is None and group.key.value_dim == 0 and group.page_stride == L * 64 * LAT
        assert eng.cache.bytes() == group.k_pages.numel() * 4

        def plain(tokens):
            t = {n: v.double() for n, v in tensors.items()}
            x = SCALE * t["embed"][tokens]
            T = len(tokens)
            for l in range(L):
                xb = P.rmsnorm(x, t[f"l{l}.n1"], 1e-6)
                q, c = xb @ t[f"l{l}.w_q"].T, xb @ t[f"l{l}.w_c"].T
                att = torch.stack([torch.softmax(c[:i + 1] @ q[i] / LAT ** 0.5, dim=0) @ c[:i + 1] for i in range(T)])
                x = x + att @ t[f"l{l}.w_o"].T
                xb = P.rmsnorm(x, t[f"l{l}.n2"], 1e-6)
                gate = torch.nn.functional.gelu(xb @ t[f"l{l}.gate"].T, approximate="tanh")
                x = x + (gate * (xb @ t[f"l{l}.up"].T)) @ t[f"l{l}.down"].T
            logits = P.rmsnorm(x, t["final"], 1e-6) @ t["embed"].T
            return CAP * torch.tanh(logits / CAP)

        prompts = [torch.randint(0, V, (n,), generator=g).tolist() for n in (70, 3, 21)]
        refs = [plain(p) for p in prompts]
        assert max(r.abs().max() for r in refs) > 0.8 * CAP          # the cap bites
        slots = eng.open(3)
        lg = eng.step(slots, prompts, [list(range(len(p))) for p in prompts]).cpu().double()
        assert (lg - torch.cat(refs)).abs().max() < 2e-4
        eng.close(slots)
        slots = eng.open(2)                    # a prefix, then token by token, in slots and pages that were used before
        eng.step(slots, [prompts[0][:60], prompts[2][:9]], [[], []])
        for i in range(8):
            lg = eng.step(slots, [[prompts[0][60 + i]], [prompts[2][9 + i]]]).cpu().double()
            assert (lg[0] - refs[0][60 + i]).abs().max() < 2e-4 and (lg[1] - refs[2][9 + i]).abs().max() < 2e-4
        eng.close(slots)
        assert eng.cache.n_live == 0 and group.pool.n_free == group.pool.n_pages
    finally:
        unregister_part("mixer", "toy_latent")


def test_a_capture_is_not_disturbed_by_garbage_of_earlier_engines(engines, sharp_dirs):
    """Engines that are dropped leave graphs behind for the garbage collector; if it found them in the middle of
    another engine's capture, destroying them there would end the process.  Here the collector is made eager and
    garbage is left lying about before a capture; the capture must go through and give the bits of an eager step."""
    import gc
    from turboquant_cpp_amd.engine.model import load_model
    from turboquant_cpp_amd.engine.step import Engine
    d, _ = sharp_dirs("A", "bfloat16")
    model = load_model(d, act="bfloat16", device=DEV)
    prompts = prompts_for("A", [5, 9], 200)

    def decode(engine, steps):
        slots = engine.open(2)
        engine.step(slots, prompts)
        out = [engine.step(slots, [[3 + i], [4 + i]]).clone() for i in range(steps)]
        engine.close(slots)
        return out

    want = decode(Engine(model, max_tokens=256, use_graphs=False), 4)
    gc.collect()
    gc.disable()
    for _ in range(3):                       # engines with captured graphs, dropped but not yet collected
        decode(Engine(model, max_tokens=256), 3)
    old = gc.get_threshold()
    gc.set_threshold(1, 1, 1)                # the collector runs at the next allocations
    gc.enable()
    try:
        got = decode(Engine(model, max_tokens=256), 4)      # eager, capture, replay, replay
    finally:
        gc.set_threshold(*old)
    for a, b in zip(got, want):
        assert torch.equal(a, b)


def test_the_kernels_refuse_to_run_without_their_library(monkeypatch):
    """No silent fallback: if the compiled library cannot be found or built, the first kernel call raises."""
    from turboquant_cpp_amd.csrc import build, ops
    monkeypatch.setattr(ops, "_LIBS", {})
    monkeypatch.setattr(build, "find_library", lambda dtype: None)

    def no_build(dtype, **kw):
        raise build.BuildError("hipcc not found")
    monkeypatch.setattr(build, "build", no_build)
    with pytest.raises(build.BuildError):
        ops.embed(torch.zeros(1, dtype=torch.int32, device=DEV), torch.zeros((2, 4), device=DEV), "float32")


# ------------------------------------------------------------------------------------------------ decode steps as graphs
@pytest.mark.parametrize("act", ACTS)
def test_replayed_decode_steps_give_the_bits_of_eager_steps(act, sharp_dirs):
    """Many replays, with eager prompt steps, closed and reopened slots and synchronisations between them; every
    replay is checked against the step run eagerly by a second engine on the same model."""
    from turboquant_cpp_amd.engine.model import load_model
    from turboquant_cpp_amd.engine.step import Engine
    d, _ = sharp_dirs("B", act)
    model = load_model(d, act=act, device=DEV)
    fast, slow = Engine(model, max_tokens=64 * 12), Engine(model, max_tokens=64 * 12, use_graphs=False)
    assert fast.graphs is not None and slow.graphs is None
    prompts = prompts_for("B", [40, 3, 70], seed=17)
    g = torch.Generator().manual_seed(18)
    sf, ss = fast.open(3), slow.open(3)
    assert torch.equal(fast.step(sf, prompts), slow.step(ss, prompts))
    live = [0, 1, 2]
    for step in range(40):
        toks = [[int(torch.randint(0, 384, (1,), generator=g))] for _ in live]
        a = fast.step([sf[i] for i in live], toks)
        b = slow.step([ss[i] for i in live], toks)
        torch.cuda.synchronize()
        assert torch.equal(a, b), f"replay {step} differs from the eager step"
        if step == 12:                       # a sequence ends; the others go on as a smaller batch
            fast.close([sf[1]]), slow.close([ss[1]])
            live = [0, 2]
        if step == 20:                       # a new one starts in the freed slot: an eager prompt step in between
            sf[1], ss[1] = fast.open(1)[0], slow.open(1)[0]
            p = prompts_for("B", [25], seed=19)
            assert torch.equal(fast.step([sf[1]], p), slow.step([ss[1]], p))
            live = [1, 0, 2]
    assert len(fast.graphs.graphs) >= 2
    only_second = fast.step([sf[i] for i in live], [[1], [2], [3]], [[], [0], []])
    assert torch.equal(only_second, slow.step([ss[i] for i in live], [[1], [2], [3]], [[], [0], []])) and only_second.shape[0] == 1
