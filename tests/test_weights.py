"""Weights: random model folders, loading by name, the one error that lists
everything wrong, storage dtypes."""

from __future__ import annotations

import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from conftest import TINY
from forge_engine_amd.config import load_model_config
from forge_engine_amd.engine import load_model
from forge_engine_amd.weights import WeightsError, storage_dtype, write_random_model


@pytest.fixture()
def folder(tmp_path):
    write_random_model(load_model_config(TINY["B"]), 7, tmp_path)
    return tmp_path


def rewrite(folder, change):
    tensors = load_file(str(folder / "model.safetensors"))
    change(tensors)
    save_file(tensors, str(folder / "model.safetensors"))


def test_random_folder_has_every_tensor_of_the_reference_schema(folder):
    # names and shapes of src/forge_engine/weights.py:253-282 plus lm_head for an untied model
    tensors = load_file(str(folder / "model.safetensors"))
    config = TINY["B"]
    assert len(tensors) == 11 * config["num_hidden_layers"] + 3
    assert tensors["model.layers.1.self_attn.q_proj.weight"].shape == (192, 96)
    assert tensors["model.layers.1.self_attn.k_norm.weight"].shape == (32,)
    assert tensors["model.layers.2.mlp.down_proj.weight"].shape == (96, 224)
    assert tensors["lm_head.weight"].shape == (384, 96)
    assert all(t.dtype == torch.bfloat16 for t in tensors.values())
    assert abs(float(tensors["model.norm.weight"].float().mean()) - 1.0) < 0.05
    assert 0.015 < float(tensors["model.embed_tokens.weight"].float().std()) < 0.025
    assert json.loads((folder / "config.json").read_text())["architectures"] == ["Qwen3ForCausalLM"]
    # seeded: the same seed writes the same file, another seed another
    again = folder / "again"
    write_random_model(load_model_config(config), 7, again)
    assert all(torch.equal(tensors[k], v) for k, v in load_file(str(again / "model.safetensors")).items())
    write_random_model(load_model_config(config), 8, again)
    assert not torch.equal(tensors["lm_head.weight"], load_file(str(again / "model.safetensors"))["lm_head.weight"])


def test_tied_model_has_no_head_tensor(tmp_path):
    write_random_model(load_model_config(TINY["A"]), 1, tmp_path)
    tensors = load_file(str(tmp_path / "model.safetensors"))
    assert "lm_head.weight" not in tensors and len(tensors) == 11 * 2 + 2
    _, model = load_model(tmp_path, dtype="float32", device="cpu")
    assert model.head.matrix() is model.embedding.weight
    # a checkpoint that repeats the tied matrix under lm_head.weight still loads
    rewrite(tmp_path, lambda t: t.update({"lm_head.weight": t["model.embed_tokens.weight"].clone()}))
    load_model(tmp_path, dtype="float32", device="cpu")


@pytest.mark.parametrize("dtype,matrix_dtype", [("bfloat16", torch.bfloat16), ("float32", torch.float32)])
def test_loading_keeps_values_and_fuses_projections(folder, dtype, matrix_dtype):
    tensors = load_file(str(folder / "model.safetensors"))
    _, model = load_model(folder, dtype=dtype, device="cpu")
    mixer = model.layers[1].mixer
    assert mixer.qkv_weight.dtype == matrix_dtype and mixer.qkv_weight.shape == (192 + 64 + 64, 96)
    for module, part in mixer.split_qkv_weight().items():
        assert torch.equal(part.float(), tensors[f"model.layers.1.self_attn.{module}.weight"].float())
    ffn = model.layers[2].feed_forward
    assert torch.equal(ffn.gate_up_weight[:224].float(), tensors["model.layers.2.mlp.gate_proj.weight"].float())
    assert torch.equal(ffn.gate_up_weight[224:].float(), tensors["model.layers.2.mlp.up_proj.weight"].float())
    assert model.final_norm.weight.dtype == torch.float32      # norm weights are widened (exactly)
    assert torch.equal(model.final_norm.weight, tensors["model.norm.weight"].float())


def test_storage_policy():
    assert storage_dtype("matrix", torch.bfloat16, torch.bfloat16) == torch.bfloat16
    assert storage_dtype("matrix", torch.bfloat16, torch.float32) == torch.float32
    assert storage_dtype("matrix", torch.float32, torch.bfloat16) == torch.float32   # 32-bit stays 32-bit
    assert storage_dtype("vector", torch.bfloat16, torch.bfloat16) == torch.float32
    assert storage_dtype("int_table", torch.int64, torch.bfloat16) == torch.int32


def test_tensor_stored_in_32_bit_stays_so(folder):
    rewrite(folder, lambda t: t.update({"model.layers.0.mlp.down_proj.weight": t["model.layers.0.mlp.down_proj.weight"].float()}))
    _, model = load_model(folder, dtype="bfloat16", device="cpu")
    assert model.layers[0].feed_forward.down_weight.dtype == torch.float32
    assert model.layers[1].feed_forward.down_weight.dtype == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_wrong_shapes(folder):
    def change(t):
        del t["model.layers.0.self_attn.q_norm.weight"]
        del t["model.norm.weight"]
        t["model.layers.9.mlp.up_proj.weight"] = torch.zeros(2, 2)
        t["model.layers.1.mlp.gate_proj.weight"] = torch.zeros(224, 95, dtype=torch.bfloat16)
        t["model.embed_tokens.weight"] = torch.zeros(383, 96, dtype=torch.bfloat16)
    rewrite(folder, change)
    with pytest.raises(WeightsError) as caught:
        load_model(folder, dtype="float32", device="cpu")
    error = caught.value
    assert sorted(error.missing) == ["model.layers.0.self_attn.q_norm.weight", "model.norm.weight"]
    assert error.unexpected == ["model.layers.9.mlp.up_proj.weight"]
    assert len(error.wrong_shape) == 2 and any("(224, 95)" in w and "(224, 96)" in w for w in error.wrong_shape)
    message = str(error)
    for piece in ("missing tensors", "model.norm.weight", "unexpected tensors", "model.layers.9.mlp.up_proj.weight",
                  "wrong shapes", "model.embed_tokens.weight"):
        assert piece in message


def test_non_finite_values_are_refused(folder):
    def change(t):
        t["model.layers.0.mlp.up_proj.weight"][3, 4] = float("nan")
    rewrite(folder, change)
    with pytest.raises(WeightsError, match="non-finite"):
        load_model(folder, dtype="float32", device="cpu")


def test_sharded_checkpoint_with_index(folder):
    tensors = load_file(str(folder / "model.safetensors"))
    names = sorted(tensors)
    half = len(names) // 2
    shards = {"model-00001-of-00002.safetensors": names[:half], "model-00002-of-00002.safetensors": names[half:]}
    weight_map = {}
    for shard, members in shards.items():
        save_file({n: tensors[n] for n in members}, str(folder / shard))
        weight_map.update({n: shard for n in members})
    (folder / "model.safetensors").unlink()
    (folder / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    _, model = load_model(folder, dtype="bfloat16", device="cpu")
    assert torch.equal(model.embedding.weight, tensors["model.embed_tokens.weight"])
    (folder / "model-00002-of-00002.safetensors").unlink()
    with pytest.raises(WeightsError, match="not in"):
        load_model(folder, dtype="bfloat16", device="cpu")


def test_no_weights_at_all(tmp_path):
    load_model_config(TINY["A"]).save(tmp_path)
    with pytest.raises(WeightsError, match="no safetensors"):
        load_model(tmp_path, dtype="float32", device="cpu")
