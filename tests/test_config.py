"""Configuration and registry: every size and constant comes from config.json's keys,
errors name the key, and the architecture's name picks the model."""
import json
import os

import pytest

import common
import llama_cu_amd
from llama_cu_amd.config import (ConfigError, LlamaConfig, architecture_of, load_config, register_architecture,
                                 registered_architectures)
from llama_cu_amd.models.llama import llama_spec


def test_all_keys_are_read():
    cfg = LlamaConfig.from_dict(common.TINY_C)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
            cfg.intermediate_size, cfg.vocab_size, cfg.max_position_embeddings) == (1, 80, 6, 2, 48, 100, 301, 200)
    assert (cfg.rope_theta, cfg.rms_norm_eps, cfg.tie_word_embeddings, cfg.rope_interleaved) == (777.0, 1e-3, False, True)


def test_defaults_are_the_reference_s():
    """llama.cu/src/model/mod.rs:73-77: kv heads = heads, head size = width / heads,
    epsilon 1e-5, rotation base 1e4."""
    d = dict(architectures=["LlamaForCausalLM"], num_hidden_layers=1, hidden_size=96, num_attention_heads=6,
             intermediate_size=10, vocab_size=11, max_position_embeddings=12)
    cfg = LlamaConfig.from_dict(d)
    assert cfg.num_key_value_heads == 6 and cfg.head_dim == 16
    assert cfg.rope_theta == 1e4 and cfg.rms_norm_eps == 1e-5 and cfg.tie_word_embeddings is False


@pytest.mark.parametrize("key", ["num_hidden_layers", "hidden_size", "num_attention_heads", "intermediate_size",
                                 "vocab_size", "max_position_embeddings"])
def test_missing_required_key_is_named(key):
    d = dict(common.TINY_A)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        LlamaConfig.from_dict(d)


@pytest.mark.parametrize("key,value", [("hidden_size", 0), ("num_hidden_layers", -1), ("vocab_size", 3.5),
                                       ("rms_norm_eps", 0), ("rope_theta", -2.0), ("tie_word_embeddings", "yes"),
                                       ("num_attention_heads", True)])
def test_bad_value_is_named(key, value):
    d = dict(common.TINY_A)
    d[key] = value
    with pytest.raises(ConfigError, match=key):
        LlamaConfig.from_dict(d)


def test_inconsistent_sizes():
    with pytest.raises(ConfigError, match="num_key_value_heads"):
        LlamaConfig.from_dict(dict(common.TINY_A, num_key_value_heads=3))
    with pytest.raises(ConfigError, match="head_dim"):
        LlamaConfig.from_dict(dict(common.TINY_A, head_dim=15))
    d = dict(common.TINY_A, hidden_size=66)
    del d["head_dim"]
    with pytest.raises(ConfigError, match="head_dim"):
        LlamaConfig.from_dict(d)


@pytest.mark.parametrize("key,value", [("rope_scaling", {"rope_type": "llama3", "factor": 8.0}), ("hidden_act", "gelu"),
                                       ("attention_bias", True), ("mlp_bias", True), ("sliding_window", 4096)])
def test_keys_that_would_change_the_computation_are_refused(key, value):
    with pytest.raises(ConfigError, match=key):
        LlamaConfig.from_dict(dict(common.TINY_A, **{key: value}))
    # the harmless spellings are accepted
    LlamaConfig.from_dict(dict(common.TINY_A, rope_scaling=None, hidden_act="silu", attention_bias=False,
                               sliding_window=None, model_type="llama", torch_dtype="bfloat16", use_cache=True))


def test_eos_ids():
    assert LlamaConfig.from_dict(dict(common.TINY_A, eos_token_id=7)).eos_token_ids == (7,)
    assert LlamaConfig.from_dict(dict(common.TINY_A, eos_token_id=[7, 9])).eos_token_ids == (7, 9)
    assert LlamaConfig.from_dict(common.TINY_A).eos_token_ids == ()


def test_round_trip_through_config_json(tmp_path):
    cfg = LlamaConfig.from_dict(dict(common.TINY_B, eos_token_id=[3, 4], bos_token_id=1))
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    arch, back = load_config(str(tmp_path))
    assert arch.name == "LlamaForCausalLM" and back == cfg


def test_registry_picks_by_name_and_lists_what_it_knows(tmp_path):
    assert "LlamaForCausalLM" in registered_architectures()
    with pytest.raises(ConfigError, match="NoSuchModel.*LlamaForCausalLM"):
        architecture_of({"architectures": ["NoSuchModel"]})
    with pytest.raises(ConfigError, match="architectures"):
        architecture_of({"hidden_size": 3})
    with pytest.raises(ConfigError, match="config.json"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{ not json")
    with pytest.raises(ConfigError, match="JSON"):
        load_config(str(tmp_path))


def test_another_architecture_can_be_registered():
    seen = {}

    def from_dict(d):
        seen["dict"] = d
        return LlamaConfig.from_dict(dict(d, architectures=["LlamaForCausalLM"]))

    register_architecture("ToyForTesting", from_dict, llama_spec, replace=True)
    arch = architecture_of({"architectures": ["ToyForTesting"]})
    cfg = arch.config_from_dict(dict(common.TINY_A, architectures=["ToyForTesting"]))
    assert arch.build_spec(cfg).hidden_size == 64
    with pytest.raises(ValueError):
        register_architecture("ToyForTesting", from_dict, llama_spec)


def test_the_model_s_layout_holds_the_configuration_s_values_and_nothing_else():
    """Every size and constant of the parts comes from the configuration: two
    configurations that differ everywhere give layouts that differ everywhere."""
    for d in (common.TINY_A, common.TINY_B, common.TINY_C):
        cfg = LlamaConfig.from_dict(d)
        spec = llama_spec(cfg)
        assert (spec.hidden_size, spec.vocab_size, spec.max_positions) == (cfg.hidden_size, cfg.vocab_size, cfg.max_position_embeddings)
        assert len(spec.layers) == cfg.num_hidden_layers == len(spec.run_order)
        blk = spec.layers[-1].params
        assert blk["norm1"].params == {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps} == blk["norm2"].params
        m = blk["mixer"].params
        assert (m["heads"], m["kv_heads"], m["head_dim"], m["hidden_size"]) == (cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.hidden_size)
        assert m["scale"] == cfg.head_dim ** -0.5 and m["window"] == 0
        assert m["position"].params == {"head_dim": cfg.head_dim, "theta": cfg.rope_theta,
                                        "max_positions": cfg.max_position_embeddings, "interleaved": cfg.rope_interleaved}
        assert blk["ffn"].params == {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size}
        assert spec.head.params["tied"] == cfg.tie_word_embeddings
        assert spec.final_norm.params["eps"] == cfg.rms_norm_eps


def test_decode_attention_split_rule():
    """Into how many parts the decode attention cuts a request's keys: few requests fill the chip's
    256 compute units, many requests of long contexts fill whole waves of workgroups."""
    import llama_cu_amd  # noqa: F401
    from llama_cu_amd.kernels.ops import decode_splits
    assert decode_splits(1, 32, 8, 2100) == 8 and decode_splits(8, 32, 8, 2100) == 4 and decode_splits(16, 32, 8, 2100) == 2
    assert decode_splits(1, 32, 8, 100) == 1 and decode_splits(1, 32, 8, 200000) == 32
    for b in (28, 40, 48, 64, 128):
        assert decode_splits(b, 32, 8, 2100) == 1            # parts would fill the chip no better, or it is full
    for b in (20, 24, 28, 64):
        assert decode_splits(b, 32, 8, 1024) == 1            # up to 1k keys: one part
    assert decode_splits(17, 32, 8, 2100) == 3 and decode_splits(20, 32, 8, 2100) == 3 and decode_splits(24, 32, 8, 2100) == 4
    assert decode_splits(20, 32, 8, 8192) == 3 and decode_splits(48, 32, 8, 8192) == 1 and decode_splits(64, 32, 8, 8192) == 1
    assert decode_splits(20, 32, 8, 4097) == 3 and decode_splits(20, 32, 8, 1025) == 1


def test_a_module_of_the_user_s_registers_an_architecture_for_the_command_line(tmp_path):
    """--plugin MODULE (and LLAMA_CU_AMD_PLUGINS) import a module that is no file of the package before a model is
    looked up: an architecture and a part that only that module knows are then found by the registry, here by
    ``random-model``, which writes the folder of such a model."""
    import json
    import subprocess
    import sys
    from llama_cu_amd.config import ConfigError, load_plugins
    from llama_cu_amd.weights.safetensors_io import open_safetensors
    name, env = common.write_toy_plugin(str(tmp_path))
    cfg = dict(common.TINY_A, architectures=["ToyMeanForCausalLM"], mean_layer=1)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    tool = os.path.join(common.ROOT, "bin", "llama.cu_amd")
    # without the module: one line that says what is registered and how to name a module
    bare = subprocess.run([tool, "random-model", str(tmp_path / "config.json"), str(tmp_path / "m0")], capture_output=True, text=True, env=env)
    assert bare.returncode != 0 and "ToyMeanForCausalLM" in bare.stderr and "--plugin" in bare.stderr
    ok = subprocess.run([tool, "random-model", str(tmp_path / "config.json"), str(tmp_path / "m1"), "--plugin", name, "--dtype", "float32"],
                        capture_output=True, text=True, env=env)
    assert ok.returncode == 0, ok.stderr[-2000:]
    names = [n for f in open_safetensors(str(tmp_path / "m1")) for n in f.names()]
    assert "model.layers.1.toy.mix.weight" in names and "model.layers.1.self_attn.q_proj.weight" not in names
    assert "model.layers.0.self_attn.q_proj.weight" in names
    assert json.loads((tmp_path / "m1" / "config.json").read_text())["mean_layer"] == 1
    # the environment variable does the same for every entry point
    env2 = dict(env, LLAMA_CU_AMD_PLUGINS=name)
    via_env = subprocess.run([sys.executable, "-c", "import sys; sys.path.insert(0, %r); import llama_cu_amd; "
                              "from llama_cu_amd.config import registered_architectures; print(registered_architectures())" % common.ROOT],
                             capture_output=True, text=True, env=env2)
    assert via_env.returncode == 0 and "ToyMeanForCausalLM" in via_env.stdout, via_env.stderr[-2000:]
    # a module that cannot be imported is named
    with pytest.raises(ConfigError, match="no_such_module_anywhere"):
        load_plugins(["no_such_module_anywhere"])


def test_the_engines_constants_are_one_typed_record():
    """``EngineConfig``: defaults, replacement of single fields, and errors that name the field."""
    from llama_cu_amd import EngineConfig
    base = EngineConfig()
    assert (base.dtype, base.page_size, base.max_batch_tokens, base.run_ahead) == ("bfloat16", 16, 2048, True)
    ec = EngineConfig.of(base, dtype="float32", page_size=32, max_tokens=4096, prefill_chunk=48)
    assert ec.page_size == 32 and ec.runner_kwargs()["max_tokens"] == 4096 and "num_pages" not in ec.runner_kwargs()
    assert "prefill_chunk" not in ec.runner_kwargs() and "run_ahead" not in ec.runner_kwargs()
    for bad, word in ((dict(page_size=12), "page_size"), (dict(dtype="float16"), "dtype"), (dict(max_seqs=0), "max_seqs"),
                      (dict(num_pages=4, max_tokens=64), "num_pages"), (dict(kv_fraction=1.5), "kv_fraction"),
                      (dict(prefill_chunk=-1), "prefill_chunk")):
        with pytest.raises(ValueError, match=word):
            EngineConfig.of(**bad)
    with pytest.raises(TypeError, match="page_sise"):
        EngineConfig.of(page_sise=16)
