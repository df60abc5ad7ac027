"""Qwen3 dense as a plan over the generic parts.

Layer structure and tensor names follow the reference
(src/forge_engine/qwen3.py:230-342; names and shapes weights.py:253-282):
token embedding; L pre-norm layers of grouped-query attention with per-head
q/k RMSNorm and rotary positions, and a SwiGLU feed-forward; final RMSNorm;
head tied to the embedding or ``lm_head.weight``.
"""

from __future__ import annotations

from ..config.qwen3 import Qwen3Config
from ..parts.plan import LayerCall, LayerSpec, ModelPlan, PartSpec
from ..registry import register_architecture


def qwen3_plan(config: Qwen3Config) -> ModelPlan:
    def norm(prefix: str) -> PartSpec:
        return PartSpec("rms_norm", {"size": config.hidden_size, "eps": config.rms_norm_eps}, prefix)

    position = PartSpec("rotary", {"head_dim": config.head_dim, "theta": config.rope_theta})
    layers = []
    for index in range(config.num_hidden_layers):
        prefix = f"model.layers.{index}"
        mixer = PartSpec("gqa_attention", {
            "hidden_size": config.hidden_size,
            "num_heads": config.num_attention_heads,
            "num_kv_heads": config.num_key_value_heads,
            "head_dim": config.head_dim,
            "qk_norm_eps": config.rms_norm_eps,
            "bias": config.attention_bias,
            "position": position,
        }, f"{prefix}.self_attn")
        feed_forward = PartSpec("swiglu", {
            "hidden_size": config.hidden_size,
            "intermediate_size": config.intermediate_size,
        }, f"{prefix}.mlp")
        layers.append(LayerSpec("pre_norm", mixer, feed_forward, {
            "input": norm(f"{prefix}.input_layernorm"),
            "post_mixer": norm(f"{prefix}.post_attention_layernorm"),
        }))
    sizes = {"vocab_size": config.vocab_size, "hidden_size": config.hidden_size}
    return ModelPlan(
        hidden_size=config.hidden_size,
        vocab_size=config.vocab_size,
        embedding=PartSpec("token_embedding", dict(sizes), "model.embed_tokens"),
        layers=tuple(layers),
        schedule=tuple(LayerCall(index) for index in range(config.num_hidden_layers)),
        final_norm=norm("model.norm"),
        head=PartSpec("lm_head", dict(sizes, tied=config.tie_word_embeddings), "lm_head"),
        eos_token_ids=config.eos_token_ids,
        max_positions=config.max_position_embeddings,
    )


register_architecture(Qwen3Config.architecture, Qwen3Config, qwen3_plan)
