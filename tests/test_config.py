"""Configuration and registry (no GPU)."""

import json

import pytest

from helpers import TINY_A, TINY_B, TINY_C
from simple_inference_amd.config import (
    ConfigError, EngineConfig, LlamaConfig, UnknownArchitecture, architecture_of, get_architecture,
    known_architectures, preset, read_config_json, register_architecture, unregister_architecture,
)


def test_reads_every_size_from_the_json_keys():
    c = LlamaConfig.from_dict(TINY_B)
    assert (c.hidden_size, c.intermediate_size, c.num_hidden_layers, c.vocab_size) == (96, 224, 3, 384)
    assert (c.num_attention_heads, c.num_key_value_heads, c.head_dim, c.num_kv_groups) == (3, 1, 32, 3)
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 500000.0 and not c.tie_word_embeddings
    s = c.rope_scaling
    assert (s.rope_type, s.factor, s.low_freq_factor, s.high_freq_factor, s.original_max_position_embeddings) == \
        ("llama3", 8.0, 1.0, 4.0, 64)


def test_head_dim_is_derived_or_honoured():
    d = dict(TINY_A)
    del d["head_dim"]
    assert LlamaConfig.from_dict(d).head_dim == 64 // 4
    assert LlamaConfig.from_dict(TINY_C).head_dim == 48  # 5 heads of 48 on a hidden size of 120


def test_rope_scaling_null_means_none_and_defaults_follow_the_reference():
    assert LlamaConfig.from_dict(TINY_A).rope_scaling is None
    d = dict(TINY_A, rope_scaling={"rope_type": "llama3", "factor": 2.0})
    s = LlamaConfig.from_dict(d).rope_scaling
    assert (s.low_freq_factor, s.high_freq_factor, s.original_max_position_embeddings) == (1.0, 4.0, 8192)


def test_round_trip_through_json(tmp_path):
    for d in (TINY_A, TINY_B, TINY_C, preset("llama-3.2-3b")):
        c = LlamaConfig.from_dict(d)
        (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
        assert LlamaConfig.from_dict(read_config_json(tmp_path)) == c


def test_eos_may_be_a_list():
    c = LlamaConfig.from_dict(dict(TINY_A, eos_token_id=[2, 7, 9]))
    assert c.eos_token_ids == (2, 7, 9) and c.eos_token_id == 2


@pytest.mark.parametrize("change, word", [
    ({"hidden_act": "gelu"}, "hidden_act"), ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"), ({"num_key_value_heads": 3}, "divisible"),
    ({"head_dim": 15}, "even"), ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "yarn"), ({"torch_dtype": "int8"}, "torch_dtype"),
])
def test_refuses_what_it_does_not_implement(change, word):
    with pytest.raises(ConfigError, match=word):
        LlamaConfig.from_dict(dict(TINY_A, **change))


def test_missing_keys_are_all_named():
    d = dict(TINY_A)
    del d["rope_theta"], d["vocab_size"]
    with pytest.raises(ConfigError) as e:
        LlamaConfig.from_dict(d)
    assert "rope_theta" in str(e.value) and "vocab_size" in str(e.value)


def test_registry_maps_the_architecture_name_to_its_model():
    assert "LlamaForCausalLM" in known_architectures()
    arch = architecture_of(TINY_A)
    assert arch is get_architecture("LlamaForCausalLM")
    plan = arch.build_plan(arch.parse_config(TINY_B))
    assert len(plan.layers) == 3 and plan.head.params["tied"] is False
    assert plan.layers[2].mixer.weights["q"] == "model.layers.2.self_attn.q_proj.weight"
    with pytest.raises(UnknownArchitecture, match="LlamaForCausalLM"):
        architecture_of({"architectures": ["MysteryForCausalLM"]})
    with pytest.raises(UnknownArchitecture):
        architecture_of({})
    register_architecture("TestOnly", lambda d: d, lambda c: None)
    try:
        with pytest.raises(ValueError):
            register_architecture("TestOnly", lambda d: d, lambda c: None)
        assert "TestOnly" in known_architectures()
    finally:
        unregister_architecture("TestOnly")


def test_engine_config():
    e = EngineConfig(max_running=3, max_seq_len=100, block_size=16)
    assert e.pages_per_request() == 7 and e.resolved_num_kv_blocks() == 21 and e.resolved_token_budget() == 300
    for bad in ({"block_size": 12}, {"max_running": 0}, {"dtype": "float16"}, {"chunk_tokens": 0}):
        with pytest.raises(ValueError):
            EngineConfig(**bad)


def test_no_model_size_stands_in_the_package_code():
    """The 3B shape's telltale numbers appear in the presets (data) only."""
    import pathlib
    import re
    root = pathlib.Path(__file__).resolve().parent.parent / "simple-inference_amd"
    hits = []
    for path in list(root.rglob("*.py")) + list(root.rglob("*.hip")) + list(root.rglob("*.h")):
        if path.name == "presets.py":
            continue
        code = "\n".join(line.split("#")[0].split("//")[0] for line in path.read_text().splitlines()
                         if not line.lstrip().startswith(("#", "//", '"""', "*")))
        if re.search(r"\b(128256|3072|8192|500000|131072)\b", code):
            hits.append(path.name)
    assert hits in ([], ["model_config.py"]), hits  # model_config.py: defaults 8192 of the reference's RopeScalingConfig
