"""The step executor of the kernel library (csrc/host/engine.cpp) against the same steps run part by part from Python:
both launch the same kernels with the same arguments, so their logits are the same bits, whatever the step's shape;
where a long prompt's plain products go to the vendor's library, whose order of sums is its own, both are held to
the bound of such products."""
import copy
import ctypes

import pytest
import torch

from test_engine_gpu import ACTS, DEV, SHARP, prompts_for
from tiny_configs import TINY


def test_the_structures_of_the_executor_are_laid_out_alike():
    """No GPU needed: the built library says how large its structures are, the ctypes mirrors must agree."""
    from turboquant_cpp_amd.csrc import build, host_api
    for dtype in ("float32", "bfloat16"):
        path = build.find_library(dtype)
        if path is None:
            pytest.skip("the kernel library is not built here")
        lib = ctypes.CDLL(path)
        host_api.check_layout(lib)
        assert all(ctypes.sizeof(s) % 8 == 0 for s in host_api.STRUCTS)


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    from turboquant_cpp_amd.engine.model import load_model, write_random_model_dir
    made = {}

    def get(name, act):
        if (name, act) not in made:
            cfg, init = TINY[name]
            d = str(tmp_path_factory.mktemp(f"exec_{name}_{act}"))
            write_random_model_dir(d, cfg, init["seed"], SHARP, init["norm_std"], act)
            made[(name, act)] = load_model(d, act=act, device=DEV)
        return made[(name, act)]
    return get


def a_schedule_of_steps(eng, prompts):
    """Prompts of unequal lengths in one step, decode steps of all (eager, captured, replayed), of fewer after some
    have ended, a second chunk for two of them, and a prompt in slots used before; returns every step's logits."""
    out = []
    slots = eng.open(len(prompts))
    out.append(eng.step(slots, prompts, [list(range(len(p))) for p in prompts]).clone())
    for t in range(4):
        out.append(eng.step(slots, [[(3 * i + t) % 50] for i in range(len(prompts))]).clone())
    eng.close(slots[2:4])
    live = slots[:2] + slots[4:]
    for t in range(3):
        out.append(eng.step(live, [[(5 * i + t) % 50] for i in range(len(live))]).clone())
    out.append(eng.step(live[:2], [[1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20], [9, 8, 7]],
                        [[0, 19], [2]]).clone())
    eng.close(live)
    slots = eng.open(2)
    out.append(eng.step(slots, [prompts[-1][:40], prompts[0]], [[0, 39], []]).clone())
    out.append(eng.step(slots, [[4], [5]], [[], [0]]).clone())
    eng.close(slots)
    assert eng.cache.n_live == 0
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_the_executor_gives_the_bits_of_the_parts(name, act, models):
    from turboquant_cpp_amd.engine.step import Engine
    model = models(name, act)
    prompts = prompts_for(name, [1, 7, 33, 70, 150, 400], seed=61)
    by_executor = Engine(model, max_tokens=64 * 40)
    by_parts = Engine(model, max_tokens=64 * 40)
    assert by_executor.native is not None
    by_parts.native = None
    a, b = a_schedule_of_steps(by_executor, prompts), a_schedule_of_steps(by_parts, prompts)
    assert len(a) == len(b)
    for i, (x, y) in enumerate(zip(a, b)):
        assert x.shape == y.shape and torch.equal(x, y), (name, act, i, (x - y).abs().max().item())
    assert by_executor.graphs.graphs and by_parts.graphs.graphs           # both replayed their decode steps


@pytest.mark.gpu
@pytest.mark.parametrize("act", ACTS)
def test_the_executor_at_the_layer_sizes_of_a_real_checkpoint(act, monkeypatch):
    """Two layers of Qwen1.5-MoE-A2.7B's sizes: steps of 1, 8, 17, 64, 300, 900 and 1,100 tokens (the pair of products in one
    launch, the streaming and the tile kernels, units of 16 to 64 rows per expert and, in the longest, units of 64 two
    at a time, one and two streams), decode steps
    eager and replayed.  A step of 900 tokens hands its plain bfloat16 products to the vendor's library; the executor
    calls that library itself where the parts go through torch, and the two may be served by different kernels of it:
    there both are compared with each other at the bound of a bfloat16 product, and with every product in this
    library's kernels the bits agree again, also between the experts' units taken two at a time and one by one."""
    from turboquant_cpp_amd.csrc import ops
    from turboquant_cpp_amd.engine.model import random_model
    from turboquant_cpp_amd.engine.step import Engine
    V = 8000
    cfg = {"architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "vocab_size": V, "hidden_size": 2048,
           "num_hidden_layers": 2, "num_attention_heads": 16, "num_key_value_heads": 16, "intermediate_size": 5632,
           "moe_intermediate_size": 1408, "shared_expert_intermediate_size": 5632, "num_experts": 60,
           "num_experts_per_tok": 4, "norm_topk_prob": False, "decoder_sparse_step": 1, "mlp_only_layers": [],
           "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "use_sliding_window": False, "sliding_window": 32768,
           "max_window_layers": 2, "max_position_embeddings": 4096, "tie_word_embeddings": False, "torch_dtype": "float32"}
    model = random_model(cfg, seed=7, act=act, device=DEV)
    g = torch.Generator().manual_seed(62)
    lens = [1, 8, 17, 64, 300, 900, 1100]
    prompts = [torch.randint(0, V, (n,), generator=g).tolist() for n in lens]
    engines = [Engine(model, max_tokens=64 * 40), Engine(model, max_tokens=64 * 40)]
    engines[1].native = None
    launches = {}

    def run(eng):
        out = {}
        for n, p in zip(lens, prompts):
            slot = eng.open(1)
            out[n] = eng.step(slot, [p], [[0, n - 1]]).clone()
            if eng.native is not None:
                launches[n] = eng.native.last_launches
            eng.close(slot)
        slots = eng.open(3)
        eng.step(slots, [prompts[2], prompts[3], prompts[4]], [[], [], []])
        out["decode"] = torch.stack([eng.step(slots, [[t + 1], [t + 2], [t + 3]]).clone() for t in range(4)])
        eng.close(slots)
        return out

    a, b = run(engines[0]), run(engines[1])
    vendor = act == "bfloat16" and ops._VENDOR
    for key in a:
        if key in (900, 1100) and vendor:
            scale = b[key].abs().max().item()
            assert (a[key] - b[key]).abs().max().item() < 0.04 * scale, key
        else:
            assert torch.equal(a[key], b[key]), (act, key, (a[key] - b[key]).abs().max().item())
    # a layer is eight to thirteen calls of launchers, the step three more (embedding, last norm, vocabulary)
    assert all(2 * 8 + 3 <= launches[n] <= 2 * 14 + 3 for n in lens), launches
    if vendor:
        monkeypatch.setattr(ops, "_VENDOR", False)
        for n in (900, 1100):
            own = []
            for eng in engines:
                slot = eng.open(1)
                own.append(eng.step(slot, [prompts[lens.index(n)]], [[0, n - 1]]).clone())
                eng.close(slot)
            assert torch.equal(own[0], own[1])
            scale = own[0].abs().max().item()
            assert (own[0] - a[n]).abs().max().item() < 0.04 * scale
        # 1,100 tokens are 73 rows per expert: units of 64 two at a time; one by one they give the same bits
        monkeypatch.setattr(ops, "EXPERT_PAIRS_FROM", 1 << 30)
        for eng in engines:
            slot = eng.open(1)
            assert torch.equal(eng.step(slot, [prompts[-1]], [[0, 1099]]), own[0])
            eng.close(slot)


@pytest.mark.gpu
def test_a_model_with_a_part_that_the_executor_does_not_know_runs_part_by_part(models, monkeypatch):
    """A part without a form in the executor (here: the attention says it has none, as one with a norm of its heads
    does) leaves the engine without one, and its steps run through the parts as before."""
    from turboquant_cpp_amd.engine.step import Engine
    from turboquant_cpp_amd.parts.attention import GroupedQueryAttention
    model = models("A", "float32")
    want = Engine(model, max_tokens=256)
    assert want.native is not None
    monkeypatch.setattr(GroupedQueryAttention, "native", lambda self: None)
    eng = Engine(model, max_tokens=256)
    assert eng.native is None
    (p,) = prompts_for("A", [20], seed=63)
    outs = []
    for e in (want, eng):
        slot = e.open(1)
        outs.append(e.step(slot, [p], [list(range(20))]))
        e.close(slot)
    assert torch.equal(outs[0], outs[1])


@pytest.mark.gpu
@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("name", ["B", "D"])
def test_the_host_program_without_python_generates_what_the_library_does(name, act, tmp_path):
    """``bin/quant_c``: the host program in C++ (csrc/host/quant_main.cpp) reads the plan that the package writes from
    config.json, loads model.safetensors by tensor name, keeps a cache of its own and drives the step executor; its
    greedy tokens are those of the Python entry point, which runs the same kernels (unequal prompts, of which the
    shorter ones end earlier; B stops on its end tokens 7 and 11 if they come)."""
    import os
    import subprocess
    import sys
    from test_engine_gpu import ROOT
    from turboquant_cpp_amd import Model
    from turboquant_cpp_amd.engine.model import write_random_model_dir
    cfg, init = TINY[name]
    d = write_random_model_dir(str(tmp_path / "m"), cfg, init["seed"], SHARP, init["norm_std"], act)
    prompts = prompts_for(name, [5, 70, 1, 23], seed=64)
    text = ";".join(",".join(str(t) for t in p) for p in prompts)
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "quant_c"), d, "-p", text, "-n", "9", "--dtype", act],
                         capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    got = []
    for line in run.stdout.splitlines():
        head, reason = line.rsplit("(", 1)
        got.append(([int(t) for t in head.split("]")[1].split()], reason.rstrip(")")))
    with Model(d, dtype=act, temperature=0.0, rep_penalty=1.0, max_tokens=9, max_batch=4) as m:
        want = m.generate_detailed(prompts, loop_detection=False)
    assert got == [(r.tokens, r.finish_reason) for r in want]
    # a folder that does not fit the model is refused with the list of what is missing
    os.rename(os.path.join(d, "model.safetensors"), os.path.join(d, "kept"))
    from turboquant_cpp_amd.weights import SafetensorsFolder, write_safetensors
    with SafetensorsFolder(d, files=[os.path.join(d, "kept")]) as f:
        tensors = {n: f.read(n).clone() for n in f.names() if not n.endswith("model.norm.weight")}
    write_safetensors(os.path.join(d, "model.safetensors"), tensors)
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "quant_c"), d, "-p", "1,2", "--dtype", act],
                         capture_output=True, text=True, timeout=600)
    assert bad.returncode != 0 and "missing tensors (1): model.norm.weight" in bad.stderr


def test_the_plan_file_names_every_part_and_tensor():
    """No GPU: the plan that a host without Python reads lists every layer's parts with their constants, every
    parameter with the checkpoint tensors behind it, the table of rotation angles and the schedule."""
    from turboquant_cpp_amd.engine.model import model_from_config
    from turboquant_cpp_amd.engine.plan_file import plan_text
    model = model_from_config(TINY["B"][0], "bfloat16")
    text = plan_text(model)
    lines = text.splitlines()
    assert lines[0] == "tqplan 1" and lines[1].startswith("model Qwen2MoeForCausalLM act=bfloat16 vocab=384 hidden=144 n_layers=3")
    assert "stop 2 7 11" in lines
    assert [l for l in lines if l.startswith("entry ")] == [f"entry {i} layer={i} cache_of=-1" for i in range(3)]
    assert sum(l.startswith("part ") and " moe_swiglu " in l for l in lines) == 1
    assert any(l.startswith("part 1 mixer gqa_attention") and "window=24" in l for l in lines)
    assert any(l.startswith("part 0 mixer gqa_attention") and "window=" not in l for l in lines)
    named = {w for l in lines if l.startswith("param ") for w in l.split() if w.startswith("model.") or w.startswith("lm_head.")}
    assert named == set(model.tensor_table())
    table = [l for l in lines if l.startswith("table 0 mixer inv_freq 12 ")][0].split()[5:]
    assert len(table) == 12 and table[0] == "3f800000"
