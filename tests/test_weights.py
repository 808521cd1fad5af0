"""Weights by tensor name: errors, dtype rules, shards, the random-weights mode (no GPU)."""

import json

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

import tiny
from mini_infer_amd.exceptions import WeightLoadError
from mini_infer_amd.models import DecoderModel, architecture_for
from mini_infer_amd.parts.base import ParamSpec
from mini_infer_amd.weights import (
    CheckpointReader,
    check_names_and_shapes,
    load_checkpoint,
    random_tensors,
    shard_paths,
    write_random_model,
)
from mini_infer_amd.weights.loader import target_dtype


def _model(cfg, dtype=torch.float32):
    arch = architecture_for(cfg)
    return DecoderModel(arch.build_spec(arch.parse_config(cfg)), dtype, "cpu")


@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F"])
def test_model_names_are_the_checkpoint_names(name):
    cfg, _ = tiny.CONFIGS[name]
    specs = _model(cfg).param_specs()
    assert {k: v.shape for k, v in specs.items()} == tiny.tensor_shapes(cfg)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg, _ = tiny.CONFIGS["B"]
    weights = tiny.make_weights(cfg, 0)
    del weights["model.layers.1.mlp.up_proj.weight"]
    del weights["model.norm.weight"]
    weights["model.layers.7.extra.weight"] = np.zeros((2, 2), dtype=np.float32)
    weights["model.layers.0.self_attn.k_proj.weight"] = np.zeros((16, 96), dtype=np.float32)
    folder = tiny.write_model_dir(tmp_path, cfg, weights)
    with pytest.raises(WeightLoadError) as caught:
        load_checkpoint(_model(cfg), folder)
    text = str(caught.value)
    assert "model.layers.1.mlp.up_proj.weight" in text and "model.norm.weight" in text
    assert "model.layers.7.extra.weight" in text
    assert "model.layers.0.self_attn.k_proj.weight: found (16, 96), expected (32, 96)" in text
    assert text.index("missing") < text.index("unexpected") < text.index("wrong_shape")


def test_tied_head_may_be_present_or_absent(tmp_path):
    cfg, _ = tiny.CONFIGS["A"]
    weights = tiny.make_weights(cfg, 0)
    assert "lm_head.weight" not in weights
    model = _model(cfg)
    load_checkpoint(model, tiny.write_model_dir(tmp_path / "without", cfg, weights))
    assert model.head.weight is model.embedding.weight
    weights["lm_head.weight"] = weights["model.embed_tokens.weight"]
    load_checkpoint(_model(cfg), tiny.write_model_dir(tmp_path / "with", cfg, weights))
    # untied: the head is required
    cfg_b, _ = tiny.CONFIGS["B"]
    weights_b = tiny.make_weights(cfg_b, 0)
    del weights_b["lm_head.weight"]
    with pytest.raises(WeightLoadError, match="lm_head.weight"):
        load_checkpoint(_model(cfg_b), tiny.write_model_dir(tmp_path / "untied", cfg_b, weights_b))


def test_merged_projections_are_q_k_v_and_gate_up_in_order(tmp_path):
    cfg, _ = tiny.CONFIGS["A"]
    weights = tiny.make_weights(cfg, 3)
    model = _model(cfg)
    load_checkpoint(model, tiny.write_model_dir(tmp_path, cfg, weights))
    p = "model.layers.1."
    qkv = model.blocks[1].mixer.qkv.weight.numpy()
    expected = np.concatenate([weights[p + f"self_attn.{n}_proj.weight"] for n in "qkv"], axis=0)
    assert np.array_equal(qkv, expected)
    gate_up = model.blocks[1].feed_forward.gate_up.weight.numpy()
    expected = np.concatenate([weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.up_proj.weight"]], axis=0)
    assert np.array_equal(gate_up, expected)


def test_dtype_rules():
    compute = torch.bfloat16
    assert target_dtype(ParamSpec((1,)), torch.float32, compute) == torch.bfloat16
    assert target_dtype(ParamSpec((1,)), torch.float16, compute) == torch.bfloat16
    assert target_dtype(ParamSpec((1,), dtype="float32"), torch.bfloat16, compute) == torch.float32
    assert target_dtype(ParamSpec((1,), dtype="int32"), torch.int64, compute) == torch.int32
    assert target_dtype(ParamSpec((1,)), torch.int64, compute) == torch.int32
    assert target_dtype(ParamSpec((1,)), torch.bfloat16, torch.float32) == torch.float32


def test_weights_are_kept_in_the_engine_dtype(tmp_path):
    cfg, _ = tiny.CONFIGS["B"]
    weights = tiny.make_weights(cfg, 1)
    folder = tiny.write_model_dir(tmp_path, cfg, weights, dtype=torch.float32)
    model = _model(cfg, torch.bfloat16)
    load_checkpoint(model, folder)
    assert model.embedding.weight.dtype == torch.bfloat16
    assert model.blocks[0].mixer_norm.weight.dtype == torch.bfloat16
    # bf16-exact values survive the trip through a float32 file
    assert np.array_equal(model.final_norm.weight.float().numpy(), weights["model.norm.weight"])


def test_sharded_checkpoint_and_missing_files(tmp_path):
    cfg, _ = tiny.CONFIGS["A"]
    weights = {k: torch.from_numpy(v) for k, v in tiny.make_weights(cfg, 2).items()}
    names = sorted(weights)
    half = len(names) // 2
    save_file({n: weights[n] for n in names[:half]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({n: weights[n] for n in names[half:]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    weight_map = {n: "model-00001-of-00002.safetensors" for n in names[:half]}
    weight_map.update({n: "model-00002-of-00002.safetensors" for n in names[half:]})
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    assert [p.name for p in shard_paths(tmp_path)] == [
        "model-00001-of-00002.safetensors", "model-00002-of-00002.safetensors"]
    model = _model(cfg)
    load_checkpoint(model, tmp_path)
    assert np.array_equal(model.embedding.weight.numpy(), weights["model.embed_tokens.weight"].numpy())
    with pytest.raises(FileNotFoundError, match="model.safetensors"):
        shard_paths(tmp_path / "nowhere")


def test_check_names_and_shapes_passes_when_all_fit():
    specs = {"a": ParamSpec((2, 3)), "b": ParamSpec((4,))}
    check_names_and_shapes(specs, {"c"}, {"a": (2, 3), "b": (4,), "c": (9,)})


def test_random_weights_mode_writes_a_loadable_folder(tmp_path):
    cfg, _ = tiny.CONFIGS["B"]
    folder = write_random_model(cfg, 7, tmp_path / "m")
    assert json.loads((folder / "config.json").read_text()) == cfg
    reader = CheckpointReader(folder)
    assert {n: reader.shapes[n] for n in reader.names()} == tiny.tensor_shapes(cfg)
    assert set(reader.dtypes.values()) == {"BF16"}
    model = _model(cfg)
    load_checkpoint(model, folder)
    embed = model.embedding.weight.numpy()
    assert abs(embed.std() - 0.02) < 0.002 and abs(embed.mean()) < 0.001
    norm = model.final_norm.weight.numpy()
    assert abs(norm.mean() - 1.0) < 0.05 and 0.03 < norm.std() < 0.2
    # same seed, same values; another seed, other values
    again = write_random_model(cfg, 7, tmp_path / "again")
    other = write_random_model(cfg, 8, tmp_path / "other")
    name = "model.layers.2.mlp.down_proj.weight"
    assert torch.equal(CheckpointReader(again).read(name), reader.read(name))
    assert not torch.equal(CheckpointReader(other).read(name), reader.read(name))


def test_random_tensors_follow_the_specs():
    specs = {"w": ParamSpec((64, 32)), "n": ParamSpec((32,), init="norm_weight"),
             "f": ParamSpec((8,), dtype="float32")}
    out = random_tensors(specs, 0, std=0.5, norm_jitter=0.0, dtype=torch.bfloat16)
    assert out["w"].dtype == torch.bfloat16 and out["f"].dtype == torch.float32
    assert torch.all(out["n"] == 1.0)
    assert 0.4 < out["w"].float().std() < 0.6
