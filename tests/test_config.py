"""Configuration and registry."""

from __future__ import annotations

import json

import pytest

from conftest import TINY
from forge_engine_amd.config import ConfigError, Qwen3Config, SchedulerConfig, load_model_config
from forge_engine_amd.registry import architecture, architectures, part_class, register_architecture


def test_reads_every_key_of_config_json(tmp_path):
    for raw in TINY.values():
        config = load_model_config(raw)
        assert isinstance(config, Qwen3Config)
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings",
                    "rms_norm_eps", "rope_theta", "tie_word_embeddings", "attention_bias"):
            assert getattr(config, key) == raw[key]
        assert config.q_size == raw["num_attention_heads"] * raw["head_dim"]
        assert config.groups == raw["num_attention_heads"] // raw["num_key_value_heads"]
    # the pinned checkpoint's sizes (reference src/forge_engine/qwen3.py:66-80) load like any other
    qwen3_4b = dict(TINY["A"], vocab_size=151936, hidden_size=2560, intermediate_size=9728,
                    num_hidden_layers=36, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                    max_position_embeddings=262144, rope_theta=5e6, eos_token_id=151645)
    path = tmp_path / "config.json"
    path.write_text(json.dumps(qwen3_4b))
    config = load_model_config(path)
    assert (config.q_size, config.kv_size, config.eos_token_ids) == (4096, 1024, frozenset({151645}))
    assert load_model_config(tmp_path) == config          # a folder works too
    assert load_model_config(config.to_dict()) == config  # round trip


def test_defaults_and_lists():
    raw = {k: v for k, v in TINY["A"].items() if k not in ("head_dim", "tie_word_embeddings", "attention_bias", "eos_token_id")}
    config = load_model_config(raw)
    assert config.head_dim == 16 and config.tie_word_embeddings is False and config.eos_token_ids == frozenset()
    assert load_model_config(dict(TINY["A"], eos_token_id=[3, 4])).eos_token_ids == frozenset({3, 4})


@pytest.mark.parametrize("change,match", [
    ({"model_type": "llama"}, "model_type"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"sliding_window": 128}, "sliding-window"),
    ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"vocab_size": 0}, "at least 1"),
    ({"rms_norm_eps": -1.0}, "positive"),
    ({"hidden_size": "64"}, "integer"),
    ({"architectures": ["NoSuchModel"]}, "unknown architecture"),
    ({"architectures": []}, "architectures"),
])
def test_rejections(change, match):
    with pytest.raises(ConfigError, match=match):
        load_model_config(dict(TINY["A"], **change))


def test_missing_key_is_named():
    raw = dict(TINY["A"])
    del raw["rope_theta"]
    with pytest.raises(ConfigError, match="rope_theta"):
        load_model_config(raw)


def test_registry():
    assert "Qwen3ForCausalLM" in architectures()
    entry = architecture("Qwen3ForCausalLM")
    plan = entry.plan(load_model_config(TINY["B"]))
    assert len(plan.layers) == 3 and len(plan.schedule) == 3
    assert plan.layers[0].mixer.kind == "gqa_attention" and plan.layers[0].feed_forward.kind == "swiglu"
    assert plan.layers[2].mixer.prefix == "model.layers.2.self_attn"
    assert part_class("norm", "rms_norm").__name__ == "RMSNorm"
    with pytest.raises(ValueError, match="already registered"):
        register_architecture("Qwen3ForCausalLM", Qwen3Config, entry.plan)
    with pytest.raises(ConfigError, match="unknown mixer"):
        part_class("mixer", "nope")


def test_schedule_may_repeat_and_share():
    from forge_engine_amd.parts import LayerCall
    import dataclasses
    plan = architecture("Qwen3ForCausalLM").plan(load_model_config(TINY["A"]))
    shared = dataclasses.replace(plan, schedule=(LayerCall(0), LayerCall(1), LayerCall(0), LayerCall(1, cache=1, writes_cache=False)))
    resolved = shared.resolved_schedule()
    assert [c.cache for c in resolved] == [0, 1, 2, 1] and [c.writes_cache for c in resolved] == [True, True, True, False]
    bad = dataclasses.replace(plan, schedule=(LayerCall(0, cache=1, writes_cache=False), LayerCall(1)))
    with pytest.raises(ValueError, match="no earlier entry"):
        bad.resolved_schedule()
    with pytest.raises(ValueError, match="must not write"):
        dataclasses.replace(plan, schedule=(LayerCall(0), LayerCall(1, cache=0))).resolved_schedule()


def test_scheduler_config_limits():
    assert SchedulerConfig().token_budget == 256 and SchedulerConfig().block_capacity == 1024
    for field in ("max_requests", "max_batch_size", "token_budget", "block_size", "block_capacity"):
        with pytest.raises(ValueError, match=field):
            SchedulerConfig(**{field: 0})
    with pytest.raises(ValueError, match="admission"):
        SchedulerConfig(admission="swap")
