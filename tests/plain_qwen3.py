"""Plain, slow Qwen3 dense forward pass: whole sequences, no cache, one function per part.

Written from the formulas of the reference model (paths are relative to the
reference checkout, ``src/forge_engine/``).  It shares no code with the engine:
it takes a dict of tensors under their checkpoint names and a dict with the
config.json keys, and works on one whole sequence at a time in the dtype of the
tensors it is given (float32 in the tests).
"""

from __future__ import annotations

import torch
from torch import Tensor


def rms_norm(x: Tensor, weight: Tensor, eps: float) -> Tensor:
    """``w * (x * rsqrt(mean(x^2) + eps))`` over the last dim, statistics in
    float32 (qwen3.py:99-105)."""
    xf = x.float()
    variance = xf.square().mean(dim=-1, keepdim=True)
    return weight * (xf * torch.rsqrt(variance + eps)).to(x.dtype)


def add_rms_norm(residual: Tensor, update: Tensor, weight: Tensor, eps: float):
    """Sum first, then normalise the sum; returns (sum, normalised)
    (kernels/__init__.py:12-26)."""
    summed = residual + update
    return summed, rms_norm(summed, weight, eps)


def rotary_tables(positions: Tensor, head_dim: int, theta: float):
    """cos/sin of ``pos * theta^(-2j/D)``, the D/2 phases repeated twice along
    the last dim (qwen3.py:345-363)."""
    exponent = torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim
    inv_freq = 1.0 / (theta**exponent)
    phases = positions.float().unsqueeze(-1) * inv_freq
    emb = torch.cat((phases, phases), dim=-1)
    return emb.cos(), emb.sin()


def rotate_half(x: Tensor) -> Tensor:
    """``cat(-x[D/2:], x[:D/2])`` (qwen3.py:366-369)."""
    first, second = x.chunk(2, dim=-1)
    return torch.cat((-second, first), dim=-1)


def apply_rotary(x: Tensor, cos: Tensor, sin: Tensor) -> Tensor:
    """``x * cos + rotate_half(x) * sin``; x is [heads, T, D], tables [T, D]
    (qwen3.py:372-381)."""
    return x * cos.unsqueeze(0) + rotate_half(x) * sin.unsqueeze(0)


def causal_attention(q: Tensor, k: Tensor, v: Tensor, scale: float,
                     window: int | None = None) -> Tensor:
    """Grouped-query causal attention over one whole sequence.

    q [Hq, T, D], k and v [Hkv, T, D].  Query head h reads kv head h // G
    (``repeat_interleave(G, dim=1)``, qwen3.py:187-188); scores are scaled after
    the product (189-190); key j is visible from query i iff j <= i
    (qwen3.py:384-406 with past_length 0); softmax in float32 (200).  ``window``
    is not part of Qwen3 dense (the reference rejects it, qwen3.py:44-45); it is
    here for the tests of the general attention kernel: key j is then visible
    only if also j > i - window.
    """
    groups = q.shape[0] // k.shape[0]
    kk = k.repeat_interleave(groups, dim=0)
    vv = v.repeat_interleave(groups, dim=0)
    scores = torch.matmul(q, kk.transpose(1, 2)) * scale
    length = q.shape[1]
    i = torch.arange(length).unsqueeze(1)
    j = torch.arange(length).unsqueeze(0)
    allowed = j <= i
    if window is not None:
        allowed = allowed & (j > i - window)
    scores = scores.masked_fill(~allowed, float("-inf"))
    probabilities = torch.softmax(scores, dim=-1, dtype=torch.float32).to(q.dtype)
    return torch.matmul(probabilities, vv)


def attention_block(x: Tensor, weights: dict, prefix: str, config: dict,
                    positions: Tensor) -> Tensor:
    """q/k/v projections, per-head q/k RMSNorm before RoPE, attention, output
    projection (qwen3.py:132-207).  x is [T, H]."""
    heads = config["num_attention_heads"]
    kv_heads = config["num_key_value_heads"]
    head_dim = config["head_dim"]
    eps = config["rms_norm_eps"]
    length = x.shape[0]

    def project(name: str) -> Tensor:
        y = x @ weights[f"{prefix}.{name}.weight"].T
        bias = weights.get(f"{prefix}.{name}.bias")
        return y if bias is None else y + bias

    q = project("q_proj").view(length, heads, head_dim)
    k = project("k_proj").view(length, kv_heads, head_dim)
    v = project("v_proj").view(length, kv_heads, head_dim)
    q = rms_norm(q, weights[f"{prefix}.q_norm.weight"], eps).transpose(0, 1)
    k = rms_norm(k, weights[f"{prefix}.k_norm.weight"], eps).transpose(0, 1)
    v = v.transpose(0, 1)
    cos, sin = rotary_tables(positions, head_dim, config["rope_theta"])
    cos, sin = cos.to(x.dtype), sin.to(x.dtype)
    q = apply_rotary(q, cos, sin)
    k = apply_rotary(k, cos, sin)
    out = causal_attention(q, k, v, head_dim**-0.5)
    out = out.transpose(0, 1).reshape(length, heads * head_dim)
    y = out @ weights[f"{prefix}.o_proj.weight"].T
    bias = weights.get(f"{prefix}.o_proj.bias")
    return y if bias is None else y + bias


def swiglu_mlp(x: Tensor, weights: dict, prefix: str) -> Tensor:
    """``down(silu(gate(x)) * up(x))`` without biases (qwen3.py:225-227)."""
    gate = x @ weights[f"{prefix}.gate_proj.weight"].T
    up = x @ weights[f"{prefix}.up_proj.weight"].T
    return (torch.nn.functional.silu(gate) * up) @ weights[f"{prefix}.down_proj.weight"].T


def decoder_layer(h: Tensor, weights: dict, index: int, config: dict,
                  positions: Tensor) -> Tensor:
    """Pre-norm block: attention on the normalised stream, add, normalise the
    sum, feed-forward, add (qwen3.py:240-261)."""
    prefix = f"model.layers.{index}"
    eps = config["rms_norm_eps"]
    x = rms_norm(h, weights[f"{prefix}.input_layernorm.weight"], eps)
    attn = attention_block(x, weights, f"{prefix}.self_attn", config, positions)
    h, y = add_rms_norm(h, attn, weights[f"{prefix}.post_attention_layernorm.weight"], eps)
    return h + swiglu_mlp(y, weights, f"{prefix}.mlp")


def lm_head(z: Tensor, weights: dict, config: dict) -> Tensor:
    """Tied: ``z @ E^T`` (qwen3.py:336).  Untied ``lm_head.weight`` follows the
    checkpoint naming; the reference is always tied."""
    if config.get("tie_word_embeddings", False):
        matrix = weights["model.embed_tokens.weight"]
    else:
        matrix = weights["lm_head.weight"]
    return (z @ matrix.T).float()


def forward(weights: dict, config: dict, token_ids, first_position: int = 0,
            return_hidden: bool = False, rows=None):
    """Logits [T, V] (float32) for one whole sequence (qwen3.py:297-342).

    ``first_position`` shifts every position by a constant; with rotary
    positions only distances count, so the result must not change.  ``rows``:
    logits of these positions only (the head of a large vocabulary is most of
    the work on a CPU); the reference computes all and its callers slice.
    """
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    positions = torch.arange(first_position, first_position + ids.numel())
    h = weights["model.embed_tokens.weight"][ids]
    hidden = []
    for index in range(config["num_hidden_layers"]):
        h = decoder_layer(h, weights, index, config, positions)
        hidden.append(h)
    if rows is not None:
        h = h[torch.as_tensor(rows, dtype=torch.long)]
    z = rms_norm(h, weights["model.norm.weight"], config["rms_norm_eps"])
    logits = lm_head(z, weights, config)
    return (logits, hidden) if return_hidden else logits


def greedy_generate(weights: dict, config: dict, prompt, new_tokens: int) -> list[int]:
    """Recompute the whole sequence for every new token; argmax of the last row."""
    ids = list(prompt)
    out = []
    for _ in range(new_tokens):
        token = int(forward(weights, config, ids)[-1].argmax())
        out.append(token)
        ids.append(token)
    return out


def filter_logits(logits: Tensor, temperature: float, top_k=None, top_p=1.0,
                  min_p=0.0) -> Tensor:
    """Temperature, top-k, top-p, min-p in that order (sampling.py:83-140)."""
    x = logits.float()
    x = (x - x.max(dim=-1, keepdim=True).values) / temperature
    neg = float("-inf")
    if top_k is not None and top_k < x.shape[-1]:
        values, indices = torch.topk(x, k=top_k, dim=-1)
        x = torch.full_like(x, neg).scatter(-1, indices, values)
    if top_p < 1.0:
        sorted_x, order = torch.sort(x, dim=-1, descending=True)
        probs = torch.softmax(sorted_x, dim=-1, dtype=torch.float32)
        remove = probs.cumsum(dim=-1) > top_p
        remove[..., 1:] = remove[..., :-1].clone()
        remove[..., 0] = False
        sorted_x = sorted_x.masked_fill(remove, neg)
        x = torch.full_like(x, neg).scatter(-1, order, sorted_x)
    if min_p > 0.0:
        probs = torch.softmax(x, dim=-1, dtype=torch.float32)
        threshold = probs.max(dim=-1, keepdim=True).values
        x = x.masked_fill(probs < threshold * min_p, neg)
    return x


def random_weights(config: dict, seed: int, dtype=torch.float32) -> dict:
    """Seeded weights under checkpoint names: matrices N(0, 0.02), norm weights
    1 + N(0, 0.05).  Names and shapes as in weights.py:253-282, plus
    ``lm_head.weight`` when the embeddings are not tied.  The values are an
    independent draw; tests that need the engine's own random model read its
    safetensors file instead."""
    g = torch.Generator().manual_seed(seed)
    hidden = config["hidden_size"]
    inter = config["intermediate_size"]
    q_size = config["num_attention_heads"] * config["head_dim"]
    kv_size = config["num_key_value_heads"] * config["head_dim"]

    def matrix(*shape):
        return (torch.randn(*shape, generator=g) * 0.02).to(dtype)

    def norm(size):
        return (1.0 + torch.randn(size, generator=g) * 0.05).to(dtype)

    w = {"model.embed_tokens.weight": matrix(config["vocab_size"], hidden)}
    for i in range(config["num_hidden_layers"]):
        p = f"model.layers.{i}"
        w[f"{p}.input_layernorm.weight"] = norm(hidden)
        w[f"{p}.self_attn.q_proj.weight"] = matrix(q_size, hidden)
        w[f"{p}.self_attn.k_proj.weight"] = matrix(kv_size, hidden)
        w[f"{p}.self_attn.v_proj.weight"] = matrix(kv_size, hidden)
        w[f"{p}.self_attn.o_proj.weight"] = matrix(hidden, q_size)
        w[f"{p}.self_attn.q_norm.weight"] = norm(config["head_dim"])
        w[f"{p}.self_attn.k_norm.weight"] = norm(config["head_dim"])
        w[f"{p}.post_attention_layernorm.weight"] = norm(hidden)
        w[f"{p}.mlp.gate_proj.weight"] = matrix(inter, hidden)
        w[f"{p}.mlp.up_proj.weight"] = matrix(inter, hidden)
        w[f"{p}.mlp.down_proj.weight"] = matrix(hidden, inter)
    w["model.norm.weight"] = norm(hidden)
    if not config.get("tie_word_embeddings", False):
        w["lm_head.weight"] = matrix(config["vocab_size"], hidden)
    return w
