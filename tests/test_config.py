"""Configuration parsing and the architecture registry (no GPU)."""

import json

import pytest

import tiny
from mini_infer_amd.config import EngineConfig, Llama3RopeScaling, ModelConfig, read_rope_parameters
from mini_infer_amd.exceptions import ConfigError
from mini_infer_amd.models import architecture_for
from mini_infer_amd.registry import ARCHITECTURES, MIXERS, Registry


def test_tiny_configs_differ_in_every_size_and_option():
    a, b = ModelConfig.from_dict(tiny.TINY_A), ModelConfig.from_dict(tiny.TINY_B)
    for field in (
        "vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
        "num_key_value_heads", "head_dim", "rms_norm_eps", "rope_theta", "tie_word_embeddings",
        "max_position_embeddings", "rope_scaling",
    ):
        assert getattr(a, field) != getattr(b, field), field
    assert a.num_attention_heads // a.num_key_value_heads != b.num_attention_heads // b.num_key_value_heads


def test_every_number_comes_from_the_file():
    cfg = ModelConfig.from_dict(tiny.TINY_B)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.intermediate_size) == (384, 96, 256)
    assert (cfg.num_hidden_layers, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim) == (3, 3, 1, 32)
    assert cfg.rms_norm_eps == 1e-5 and cfg.rope_theta == 500000.0 and not cfg.tie_word_embeddings
    assert cfg.rope_scaling == Llama3RopeScaling(8.0, 1.0, 4.0, 64)
    assert cfg.max_position_embeddings == 512
    assert cfg.architecture == "LlamaForCausalLM"


def test_head_dim_defaults_to_hidden_over_heads():
    raw = dict(tiny.TINY_A)
    del raw["head_dim"]
    assert ModelConfig.from_dict(raw).head_dim == 64 // 4
    raw["head_dim"] = None
    assert ModelConfig.from_dict(raw).head_dim == 16


def test_rope_parameters_in_either_place():
    # newer files: `rope_parameters` with theta inside; older: `rope_scaling` beside `rope_theta`
    theta, scaling = read_rope_parameters(tiny.TINY_C)
    assert theta == 20000.0 and scaling.factor == 4.0 and scaling.original_max_position_embeddings == 32
    theta, scaling = read_rope_parameters({"rope_theta": 123.0, "rope_scaling": None})
    assert theta == 123.0 and scaling is None
    theta, scaling = read_rope_parameters({})
    assert theta == 10000.0 and scaling is None
    legacy = {"rope_scaling": {"type": "llama3", "factor": 2, "low_freq_factor": 1, "high_freq_factor": 4,
                               "original_max_position_embeddings": 16}}
    assert read_rope_parameters(legacy)[1].factor == 2.0


@pytest.mark.parametrize("kind", ["linear", "dynamic", "yarn"])
def test_other_rope_types_are_refused(kind):
    with pytest.raises(NotImplementedError, match=kind):
        read_rope_parameters({"rope_scaling": {"rope_type": kind, "factor": 2.0}})


def test_llama3_rope_needs_all_its_fields():
    with pytest.raises(ConfigError, match="low_freq_factor"):
        read_rope_parameters({"rope_scaling": {"rope_type": "llama3", "factor": 8.0}})
    with pytest.raises(ConfigError):
        Llama3RopeScaling(8.0, 4.0, 1.0, 64)
    with pytest.raises(ConfigError):
        Llama3RopeScaling(0.0, 1.0, 4.0, 64)


def test_missing_keys_and_biases_are_refused():
    raw = dict(tiny.TINY_A)
    del raw["intermediate_size"]
    with pytest.raises(ConfigError, match="intermediate_size"):
        ModelConfig.from_dict(raw)
    with pytest.raises(NotImplementedError, match="attention_bias"):
        ModelConfig.from_dict({**tiny.TINY_A, "attention_bias": True})
    with pytest.raises(NotImplementedError, match="mlp_bias"):
        ModelConfig.from_dict({**tiny.TINY_A, "mlp_bias": True})
    with pytest.raises(ConfigError, match="multiple"):
        ModelConfig.from_dict({**tiny.TINY_A, "num_key_value_heads": 3})
    with pytest.raises(ConfigError, match="architectures"):
        ModelConfig.from_dict({**tiny.TINY_A, "architectures": []})


def test_config_round_trips_through_json(tmp_path):
    cfg = ModelConfig.from_dict(tiny.TINY_B)
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    assert ModelConfig.from_json(tmp_path) == cfg


def test_registry_lookup_and_errors():
    assert architecture_for(tiny.TINY_A) is ARCHITECTURES.lookup("LlamaForCausalLM")
    with pytest.raises(ValueError, match="supported.*LlamaForCausalLM"):
        architecture_for({"architectures": ["NoSuchForCausalLM"]})
    with pytest.raises(ValueError, match="architectures"):
        architecture_for({})
    import mini_infer_amd.parts  # noqa: F401

    assert "gqa_attention" in MIXERS
    reg = Registry("thing")
    with pytest.raises(ValueError):
        reg.register("", object())
    with pytest.raises(ValueError, match="no thing named"):
        reg.lookup("x")


def test_llama_spec_is_data():
    arch = architecture_for(tiny.TINY_B)
    spec = arch.build_spec(arch.parse_config(tiny.TINY_B))
    assert len(spec.layers) == 3 and [c.layer for c in spec.order] == [0, 1, 2]
    mixer = spec.layers[0].block["mixer"]
    assert mixer["kind"] == "gqa_attention" and mixer["num_kv_heads"] == 1 and mixer["head_dim"] == 32
    assert mixer["position"]["llama3"]["factor"] == 8.0
    assert spec.layers[0].block["feed_forward"] == {
        "kind": "swiglu", "hidden_size": 96, "intermediate_size": 256, "activation": "silu"}
    assert not spec.tie_word_embeddings


def test_a_spec_needs_only_what_its_embedding_and_head_need():
    """The checkpoint names of the plain table and the plain head are a short form: a spec that
    describes its own embedding and head parts gives neither, one that gives nothing is told so."""
    import dataclasses

    from mini_infer_amd.models.spec import ModelSpec

    arch = architecture_for(tiny.TINY_A)
    llama = arch.build_spec(arch.parse_config(tiny.TINY_A))
    own = ModelSpec(vocab_size=7, hidden_size=8, layers=[], order=[], final_norm=llama.final_norm, final_norm_prefix="n.",
                    embedding={"kind": "my_embedding"}, head={"kind": "my_head"})
    assert own.embedding_description() == {"kind": "my_embedding"} and own.head_description() == {"kind": "my_head"}
    bare = dataclasses.replace(own, embedding=None, head=None)
    with pytest.raises(ValueError, match="embedding_name"):
        bare.embedding_description()
    with pytest.raises(ValueError, match="head_name"):
        bare.head_description()
    assert dataclasses.replace(bare, tie_word_embeddings=True).head_description()["tied"]


def test_engine_config_checks():
    assert EngineConfig().block_size == 16 and EngineConfig().num_blocks == 1024
    with pytest.raises(ValueError):
        EngineConfig(dtype="float16")
    with pytest.raises(ValueError):
        EngineConfig(block_size=0)
