"""Configuration from config.json, the architecture registry, weights by tensor name and their errors.  No GPU."""
import copy
import json
import os

import pytest
import torch

from tiny_configs import TINY, TINY_A, TINY_B
from turboquant_cpp_amd.config import ConfigError, config_from_dict, config_from_dir, known_architectures
from turboquant_cpp_amd.engine.model import model_from_config, write_random_model_dir
from turboquant_cpp_amd.weights import (SafetensorsError, SafetensorsFolder, TensorDict, WeightError, check,
                                        load_bindings, stored_dtype, write_safetensors)


# ------------------------------------------------------------------------------------------------ configuration
def test_config_reads_every_key_of_both_tiny_models():
    _, a = config_from_dict(TINY_A)
    _, b = config_from_dict(TINY_B)
    assert (a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (64, 4, 4, 16)
    assert (b.hidden_size, b.num_attention_heads, b.num_key_value_heads, b.head_dim) == (144, 6, 2, 24)
    assert a.norm_topk_prob is False and b.norm_topk_prob is True
    assert [a.layer_is_sparse(l) for l in range(2)] == [True, True]
    assert [b.layer_is_sparse(l) for l in range(3)] == [False, True, False]      # mlp_only [0], sparse step 2
    assert [a.layer_window(l) for l in range(2)] == [None, None]
    assert [b.layer_window(l) for l in range(3)] == [None, 24, 24]
    assert b.stop_token_ids == [7, 11] and a.stop_token_ids == []
    assert (a.rms_norm_eps, b.rms_norm_eps, a.rope_theta, b.rope_theta) == (1e-6, 1e-5, 1e4, 1e6)


def test_a_folder_as_newer_tools_write_it():
    """The layers' kinds listed one by one win over the rule of max_window_layers; the rotation's base is found inside
    rope_parameters; q, k, v without bias read no bias tensors; "dtype" names the stored type."""
    from tiny_configs import TINY_D
    arch, d = config_from_dict(TINY_D)
    assert [d.layer_window(l) for l in range(4)] == [19, None, 19, None]
    assert d.rope_theta == 250000.0 and d.qkv_bias is False and d.torch_dtype == "float32"
    plan = arch.plan(d)
    assert [l.parts["mixer"].args["window"] for l in plan.layers] == [19, None, 19, None]
    assert all("qkv_bias" not in l.parts["mixer"].tensors for l in plan.layers)
    names = model_from_config(TINY_D, "float32").tensor_table()
    assert not [n for n in names if n.endswith(".bias")]
    # what the configuration writes back reads as itself
    again = config_from_dict(arch.config_to_json(d))[1]
    assert again == d
    # without the list the rule of max_window_layers holds
    e = copy.deepcopy(TINY_D)
    del e["layer_types"]
    assert [config_from_dict(e)[1].layer_window(l) for l in range(4)] == [None, None, None, 19]
    # both places for the rotation's base may be there if they agree
    e["rope_theta"] = 250000.0
    assert config_from_dict(e)[1].rope_theta == 250000.0


@pytest.mark.parametrize("change,word", [
    ({"layer_types": ["full_attention"] * 3}, "layer_types"),
    ({"layer_types": ["full_attention", "chunked_attention", "full_attention", "full_attention"]}, "chunked_attention"),
    ({"sliding_window": None}, "sliding"),
    ({"rope_parameters": {"rope_type": "yarn", "rope_theta": 1e4, "factor": 2.0}}, "rope_type"),
    ({"rope_parameters": {"rope_type": "default"}}, "rope_theta"),
    ({"rope_theta": 1e4}, "differ"),
    ({"qkv_bias": "no"}, "true or false"),
])
def test_a_newer_folder_that_asks_for_what_is_not_built_is_refused(change, word):
    from tiny_configs import TINY_D
    d = copy.deepcopy(TINY_D)
    d.update(change)
    with pytest.raises(ConfigError, match=word):
        config_from_dict(d)


def test_head_dim_defaults_to_hidden_over_heads_and_kv_heads_to_heads():
    d = copy.deepcopy(TINY_A)
    del d["num_key_value_heads"]
    _, c = config_from_dict(d)
    assert c.head_dim == 16 and c.num_key_value_heads == 4


def test_changing_mlp_only_layers_changes_which_layers_are_sparse():
    d = copy.deepcopy(TINY_B)
    d["mlp_only_layers"] = []
    _, c = config_from_dict(d)
    assert [c.layer_is_sparse(l) for l in range(3)] == [False, True, False]       # the step rule alone
    d["decoder_sparse_step"] = 1
    _, c = config_from_dict(d)
    assert [c.layer_is_sparse(l) for l in range(3)] == [True, True, True]


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "intermediate_size", "moe_intermediate_size", "num_experts", "num_experts_per_tok",
                                 "rope_theta", "rms_norm_eps", "max_position_embeddings",
                                 "shared_expert_intermediate_size"])
def test_a_size_or_constant_that_is_missing_is_an_error_not_a_default(key):
    d = copy.deepcopy(TINY_A)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        config_from_dict(d)


@pytest.mark.parametrize("change,word", [
    ({"num_key_value_heads": 3}, "multiple"),
    ({"num_experts_per_tok": 9}, "exceeds"),
    ({"mlp_only_layers": [5]}, "mlp_only_layers"),
    ({"use_sliding_window": True, "sliding_window": 0}, "sliding_window"),
    ({"hidden_size": "64"}, "integer"),
    ({"norm_topk_prob": 1}, "true or false"),
    ({"head_dim": 15}, "even"),
    ({"architectures": ["LlamaForCausalLM"]}, "unknown architecture"),
    ({"architectures": []}, "architectures"),
    ({"rope_scaling": {"type": "yarn", "factor": 4.0}}, "rope_scaling"),
    ({"hidden_act": "gelu"}, "hidden_act"),
])
def test_inconsistent_configurations_are_refused(change, word):
    d = copy.deepcopy(TINY_A)
    d.update(change)
    with pytest.raises(ConfigError, match=word):
        config_from_dict(d)


def test_unknown_architecture_lists_the_known_ones():
    d = copy.deepcopy(TINY_A)
    d["architectures"] = ["Nope"]
    with pytest.raises(ConfigError) as e:
        config_from_dict(d)
    assert "Qwen2MoeForCausalLM" in str(e.value) and known_architectures() == ["Qwen2MoeForCausalLM"]


def test_config_from_dir_errors(tmp_path):
    with pytest.raises(ConfigError, match="no config.json"):
        config_from_dir(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        config_from_dir(str(tmp_path))


def test_plan_holds_the_layers_parts_by_kind():
    arch, c = config_from_dict(TINY_B)
    plan = arch.plan(c)
    assert [l.parts["ffn"].kind for l in plan.layers] == ["dense_swiglu", "moe_swiglu", "dense_swiglu"]
    assert [l.parts["mixer"].args["window"] for l in plan.layers] == [None, 24, 24]
    assert [e.layer for e in plan.schedule] == [0, 1, 2] and plan.stop_tokens == (7, 11)
    assert plan.layers[1].parts["ffn"].args["renormalize"] is True
    assert plan.layers[0].parts["ffn"].args["inner_size"] == 160


# ------------------------------------------------------------------------------------------------ safetensors
def test_safetensors_round_trip_against_the_safetensors_library(tmp_path):
    from safetensors import safe_open
    tensors = {"a": torch.randn(3, 5), "b.c": torch.randn(7).to(torch.bfloat16), "i": torch.arange(6, dtype=torch.int32).view(2, 3),
               "empty": torch.zeros(0, 4)}
    path = str(tmp_path / "model.safetensors")
    write_safetensors(path, tensors, metadata={"format": "pt"})
    with safe_open(path, framework="pt") as f:                   # the library reads what the writer wrote
        assert set(f.keys()) == set(tensors)
        for n, t in tensors.items():
            assert torch.equal(f.get_tensor(n), t)
    with SafetensorsFolder(str(tmp_path)) as folder:             # and the reader reads it by name
        for n, t in tensors.items():
            got = folder.read(n)
            assert got.dtype == t.dtype and torch.equal(got, t)


def test_safetensors_reader_reads_shards_and_refuses_broken_files(tmp_path):
    write_safetensors(str(tmp_path / "model-00001-of-00002.safetensors"), {"x": torch.ones(2)})
    write_safetensors(str(tmp_path / "model-00002-of-00002.safetensors"), {"y": torch.zeros(3)})
    with SafetensorsFolder(str(tmp_path)) as f:
        assert sorted(f.names()) == ["x", "y"] and f.read("y").shape == (3,)
    bad = tmp_path / "bad"
    bad.mkdir()
    with pytest.raises(SafetensorsError, match="no model.safetensors"):
        SafetensorsFolder(str(bad))
    (bad / "model.safetensors").write_bytes(b"\x00" * 4)
    with pytest.raises(SafetensorsError, match="too small"):
        SafetensorsFolder(str(bad))
    (bad / "model.safetensors").write_bytes((10 ** 6).to_bytes(8, "little") + b"{}")
    with pytest.raises(SafetensorsError, match="beyond the file"):
        SafetensorsFolder(str(bad))
    (bad / "model.safetensors").write_bytes((2).to_bytes(8, "little") + b"{x")
    with pytest.raises(SafetensorsError, match="not valid JSON"):
        SafetensorsFolder(str(bad))
    hdr = json.dumps({"t": {"dtype": "F8_E4M3", "shape": [1], "data_offsets": [0, 1]}}).encode()
    (bad / "model.safetensors").write_bytes(len(hdr).to_bytes(8, "little") + hdr + b"\x00")
    with pytest.raises(SafetensorsError, match="unsupported dtype"):
        SafetensorsFolder(str(bad))


# ------------------------------------------------------------------------------------------------ weights by name
def test_expected_tensor_names_and_shapes():
    table = model_from_config(TINY_B, "float32").tensor_table()
    assert table["model.embed_tokens.weight"] == ((384, 144), "table")
    assert table["model.layers.1.self_attn.q_proj.bias"] == ((144,), "bias")
    assert table["model.layers.1.self_attn.k_proj.weight"] == ((48, 144), "matrix")
    assert table["model.layers.1.mlp.gate.weight"] == ((12, 144), "router")
    assert table["model.layers.1.mlp.experts.11.down_proj.weight"] == ((144, 48), "matrix")
    assert table["model.layers.1.mlp.shared_expert_gate.weight"] == ((1, 144), "router")
    assert table["model.layers.0.mlp.up_proj.weight"] == ((160, 144), "matrix")
    assert table["model.layers.2.post_attention_layernorm.weight"] == ((144,), "scale")
    assert "model.layers.0.mlp.gate.weight" not in table and "lm_head.weight" in table


def test_tied_embeddings_read_no_lm_head():
    d = copy.deepcopy(TINY_A)
    d["tie_word_embeddings"] = True
    assert "lm_head.weight" not in model_from_config(d, "float32").tensor_table()


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    model = model_from_config(TINY_A, "float32")
    table = model.tensor_table()
    tensors = {n: torch.zeros(s) for n, (s, _r) in table.items()}
    del tensors["model.layers.0.mlp.gate.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.extra.weight"] = torch.zeros(1)
    tensors["model.layers.1.self_attn.o_proj.weight"] = torch.zeros(64, 63)
    with pytest.raises(WeightError) as e:
        load_bindings(model.bindings, TensorDict(tensors), "float32", "cpu")
    err = e.value
    assert sorted(err.missing) == ["model.layers.0.mlp.gate.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.extra.weight"]
    assert err.wrong_shape == [("model.layers.1.self_attn.o_proj.weight", (64, 63), (64, 64))]
    msg = str(err)
    for word in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (1)", "is (64, 63), model wants (64, 64)"):
        assert word in msg


def test_stored_types():
    bf, f32, f16 = torch.bfloat16, torch.float32, torch.float16
    assert stored_dtype([bf], "bfloat16") == bf and stored_dtype([f16], "bfloat16") == bf
    assert stored_dtype([f32], "bfloat16") == f32                 # stored in 32 bits: stays so, unless it is a matrix
    assert stored_dtype([bf, f32], "bfloat16") == f32
    for role, want in (("matrix", bf), ("table", bf), ("scale", f32), ("bias", f32), ("router", f32)):
        assert stored_dtype([f32], "bfloat16", role, "bfloat16") == want
        assert stored_dtype([f32], "bfloat16", role, "keep") == f32
        assert stored_dtype([f32], "float32", role, "bfloat16") == f32
    assert stored_dtype([bf], "float32") == f32 and stored_dtype([f32], "float32") == f32
    assert stored_dtype([torch.int64], "bfloat16") == torch.int32


def test_parameters_are_stacked_and_joined_from_their_tensors(model_dirs):
    d = model_dirs("B")
    model = model_from_config(TINY_B, "float32")
    with SafetensorsFolder(d) as f:
        model.load(f, "cpu")
        attn = model.blocks[1].mixer
        q, k, v = (f.read(f"model.layers.1.self_attn.{n}_proj.weight") for n in "qkv")
        assert torch.equal(attn.qkv_weight, torch.cat([q, k, v]))
        assert torch.equal(attn.qkv_bias, torch.cat([f.read(f"model.layers.1.self_attn.{n}_proj.bias") for n in "qkv"]))
        moe = model.blocks[1].ffn
        assert moe.expert_down.shape == (12, 144, 48)
        assert torch.equal(moe.expert_up[7], f.read("model.layers.1.mlp.experts.7.up_proj.weight"))
        assert torch.equal(model.lm_head, f.read("lm_head.weight"))


def test_a_bfloat16_model_rounds_32_bit_matrices_as_it_places_them_and_keeps_the_rest(tmp_path):
    """On the bfloat16 path a matrix of a product that the folder stores in 32 bits becomes bfloat16 at load, with one
    warning that counts them; norm weights, biases and the router's rows, which feed float32 arithmetic, stay as they
    are stored; ``f32_matrices="keep"`` leaves everything as stored and warns that those products are slow."""
    import warnings
    from turboquant_cpp_amd.weights.loader import RoundedWeights, SlowWeights
    d = write_random_model_dir(str(tmp_path / "m"), TINY_A, seed=3, dtype="bfloat16")
    with SafetensorsFolder(d) as f:
        tensors = {n: f.read(n).clone() for n in f.names()}
    in32 = ["model.norm.weight", "model.layers.0.mlp.gate.weight", "model.layers.0.self_attn.q_proj.bias",
            "model.layers.1.self_attn.o_proj.weight", "model.layers.0.mlp.experts.3.up_proj.weight"]
    for n in in32:
        tensors[n] = tensors[n].float() * 1.001          # values that bfloat16 does not hold
    write_safetensors(os.path.join(d, "model.safetensors"), tensors)
    model = model_from_config(TINY_A, "bfloat16")
    with SafetensorsFolder(d) as f, warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        model.load(f, "cpu")
    assert [str(x.message)[:10] for x in w if x.category is RoundedWeights] == ["2 matrices"]
    assert not [x for x in w if x.category is SlowWeights]
    assert model.final_norm.weight.dtype == torch.float32
    assert model.blocks[0].ffn.router.dtype == torch.float32
    assert model.blocks[0].mixer.qkv_bias.dtype == torch.float32        # one of its three pieces is stored in 32 bits
    assert model.blocks[1].mixer.qkv_bias.dtype == torch.bfloat16
    assert model.blocks[1].mixer.out_weight.dtype == torch.bfloat16     # rounded here
    assert torch.equal(model.blocks[1].mixer.out_weight, tensors["model.layers.1.self_attn.o_proj.weight"].bfloat16())
    assert model.blocks[0].ffn.expert_up.dtype == torch.bfloat16
    assert model.blocks[1].ffn.router.dtype == torch.bfloat16 and model.embedding.dtype == torch.bfloat16
    kept = model_from_config(TINY_A, "bfloat16")
    with SafetensorsFolder(d) as f, warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        kept.load(f, "cpu", f32_matrices="keep")
    assert [str(x.message)[:10] for x in w if x.category is SlowWeights] == ["2 matrices"]
    assert kept.blocks[1].mixer.out_weight.dtype == torch.float32 and kept.blocks[0].ffn.expert_up.dtype == torch.float32
    assert torch.equal(kept.blocks[1].mixer.out_weight, tensors["model.layers.1.self_attn.o_proj.weight"])
    with pytest.raises(ValueError, match="f32_matrices"):
        kept.load(TensorDict(tensors), "cpu", f32_matrices="half")
    m32 = model_from_config(TINY_A, "float32")
    with SafetensorsFolder(d) as f:
        m32.load(f, "cpu")
    assert all(getattr(b.owner, b.attr).dtype == torch.float32 for b in m32.bindings)


def test_random_weights_mode_writes_a_folder_that_the_seed_fixes(tmp_path):
    a = write_random_model_dir(str(tmp_path / "a"), TINY_B, seed=1, std=0.02, norm_std=0.02, dtype="float32")
    b = write_random_model_dir(str(tmp_path / "b"), TINY_B, seed=1, std=0.02, norm_std=0.02, dtype="float32")
    c = write_random_model_dir(str(tmp_path / "c"), TINY_B, seed=2, std=0.02, norm_std=0.02, dtype="float32")
    assert sorted(os.listdir(a)) == ["config.json", "model.safetensors"]
    assert json.load(open(os.path.join(a, "config.json")))["architectures"] == ["Qwen2MoeForCausalLM"]
    _, cfg = config_from_dir(a)
    assert cfg.sliding_window == 24 and cfg.stop_token_ids == [7, 11]
    with SafetensorsFolder(a) as fa, SafetensorsFolder(b) as fb, SafetensorsFolder(c) as fc:
        assert set(fa.names()) == set(model_from_config(TINY_B, "float32").tensor_table())
        w = "model.layers.1.mlp.experts.3.gate_proj.weight"
        assert torch.equal(fa.read(w), fb.read(w)) and not torch.equal(fa.read(w), fc.read(w))
        assert abs(float(fa.read(w).std()) - 0.02) < 0.004
        n = fa.read("model.layers.0.input_layernorm.weight")
        assert abs(float(n.mean()) - 1.0) < 0.01 and 0.01 < float(n.std()) < 0.03
    with SafetensorsFolder(write_random_model_dir(str(tmp_path / "d"), TINY_A, seed=0, dtype="bfloat16")) as fd:
        assert fd.read("model.norm.weight").dtype == torch.bfloat16 and bool((fd.read("model.norm.weight") == 1).all())


def test_tensors_that_the_model_does_not_read_are_a_warning_not_an_error():
    from turboquant_cpp_amd.weights.loader import UnexpectedTensors
    model = model_from_config(TINY_A, "float32")
    tensors = {n: torch.zeros(s) for n, (s, _r) in model.tensor_table().items()}
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    with pytest.warns(UnexpectedTensors, match="rotary_emb.inv_freq"):
        load_bindings(model.bindings, TensorDict(tensors), "float32", "cpu")
    assert model.blocks[0].mixer.qkv_weight.shape == (3 * 64, 64)


def test_random_weights_are_a_function_of_seed_tensor_and_element(tmp_path):
    """The generator's integer steps against splitmix64's published first outputs for state 0, pieces of a tensor
    against the whole, and a model drawn in memory against the folder written for the same seed."""
    from turboquant_cpp_amd.engine.model import random_model
    from turboquant_cpp_amd.weights import random_init as ri
    assert ri.splitmix64(0, 0) == 0xE220A8397B1DCDAF and ri.splitmix64(0, 1) == 0x6E789E6AA1B965F4
    words = ri.splitmix64_mix(torch.tensor([ri._signed(ri._GAMMA), ri._signed(2 * ri._GAMMA)]))
    assert [w % (1 << 64) for w in words.tolist()] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4]
    key = ri.tensor_key(5, 3)
    whole = ri.standard_normal(key, 0, 1000)
    assert torch.equal(torch.cat([ri.standard_normal(key, 0, 333), ri.standard_normal(key, 333, 667)]), whole)
    assert not torch.equal(ri.standard_normal(ri.tensor_key(5, 4), 0, 1000), whole)
    z = ri.standard_normal(key, 0, 400000)
    assert abs(float(z.mean())) < 0.01 and abs(float(z.var()) - 1) < 0.01 and abs(float((z ** 4).mean()) - 3) < 0.05
    assert abs(float((z[:-1] * z[1:]).mean())) < 0.01
    for dtype in ("float32", "bfloat16"):
        d = write_random_model_dir(str(tmp_path / dtype), TINY_B, seed=1, std=0.02, norm_std=0.02, dtype=dtype)
        drawn = random_model(TINY_B, 1, act=dtype, device="cpu", std=0.02, norm_std=0.02)
        loaded = model_from_config(TINY_B, dtype)
        with SafetensorsFolder(d) as f:
            loaded.load(f, "cpu")
        for a, b in zip(drawn.bindings, loaded.bindings):
            assert torch.equal(getattr(a.owner, a.attr), getattr(b.owner, b.attr)), a.path


def test_the_header_the_sources_and_the_python_face_name_the_same_entry_points():
    """Every exported function of the kernel sources is declared in `csrc/turboquant_kernels.h` (or `no_alloc.h`) with
    as many arguments as its definition has, and `ops.py` gives ctypes that many argument types."""
    import glob
    import os
    import re
    from turboquant_cpp_amd.csrc import ops
    csrc = os.path.dirname(ops.__file__)

    def declared(text, pattern):
        found = {}
        for m in re.finditer(pattern, text):
            args = " ".join(m.group(2).split())
            found[m.group(1)] = 0 if args in ("", "void") else args.count(",") + 1
        return found

    defined = {}
    for f in glob.glob(os.path.join(csrc, "*.hip")):
        defined.update(declared(open(f).read(), r"TQ_API\s+[\w\s\*]+?\s+(tq_\w+)\s*\(([^)]*)\)\s*\{"))
    header = {}
    for name in ("turboquant_kernels.h", "no_alloc.h"):
        header.update(declared(open(os.path.join(csrc, name)).read(), r"\b(tq_\w+)\s*\(([^)]*)\)\s*;"))
    assert defined == header, {k: (defined.get(k), header.get(k)) for k in set(defined) | set(header)
                               if defined.get(k) != header.get(k)}
    python = {**ops._SIGNATURES, **ops._OPTIONAL}
    for name, n_args in defined.items():
        if name in python:
            assert len(python[name]) == n_args, (name, len(python[name]), n_args)
    assert set(python) <= set(defined), set(python) - set(defined)
