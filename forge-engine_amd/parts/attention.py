"""Grouped-query causal self-attention over the paged cache.

In order (reference: src/forge_engine/qwen3.py:132-207): q, k, v projections
(one fused product here); RMSNorm of each q and k head over the head dim with a
weight shared by all heads, before the rotation; rotary positions; attention of
each query head h over the keys of kv head h // G with scale head_dim^-0.5 and
the causal mask; output projection.  The keys and values of the step's tokens
go into their pages first, and attention then reads everything through the
block table, so a step may hold any portion of any request.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..cache.spec import CacheNeeds, CacheView, PagedKV
from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, Mixer, ParamSpec, build_part
from .plan import PartSpec


class GroupedQueryAttention(Mixer):
    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, num_heads: int,
                 num_kv_heads: int, head_dim: int, position: PartSpec, qk_norm_eps: float | None = None,
                 bias: bool = False, window: int | None = None, scale: float | None = None) -> None:
        super().__init__(ctx, prefix)
        if num_heads % num_kv_heads:
            raise ValueError("query heads must be a multiple of kv heads")
        if head_dim % 2 or not 2 <= head_dim <= 256:
            raise ValueError(f"head size {head_dim} is not supported: even sizes from 2 to 256")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.q_size = num_heads * head_dim
        self.kv_size = num_kv_heads * head_dim
        self.qk_norm_eps = qk_norm_eps
        self.bias = bias
        self.window = window
        self.scale = head_dim ** -0.5 if scale is None else float(scale)
        self.position = build_part("position", position, ctx)
        width = self.q_size + 2 * self.kv_size
        self._rows = {"q_proj": (0, self.q_size), "k_proj": (self.q_size, self.kv_size),
                      "v_proj": (self.q_size + self.kv_size, self.kv_size)}
        self._width = width
        self.qkv_weight: Tensor | None = None
        self.qkv_bias: Tensor | None = None
        self.o_weight: Tensor | None = None
        self.o_bias: Tensor | None = None
        self.q_norm: Tensor | None = None
        self.k_norm: Tensor | None = None

    # ------------------------------------------------------------ tensors
    def param_specs(self):
        specs = {
            self.name("q_proj.weight"): ParamSpec((self.q_size, self.hidden_size)),
            self.name("k_proj.weight"): ParamSpec((self.kv_size, self.hidden_size)),
            self.name("v_proj.weight"): ParamSpec((self.kv_size, self.hidden_size)),
            self.name("o_proj.weight"): ParamSpec((self.hidden_size, self.q_size)),
        }
        if self.bias:
            specs[self.name("q_proj.bias")] = ParamSpec((self.q_size,), kind="vector", init="zeros")
            specs[self.name("k_proj.bias")] = ParamSpec((self.kv_size,), kind="vector", init="zeros")
            specs[self.name("v_proj.bias")] = ParamSpec((self.kv_size,), kind="vector", init="zeros")
            specs[self.name("o_proj.bias")] = ParamSpec((self.hidden_size,), kind="vector", init="zeros")
        if self.qk_norm_eps is not None:
            specs[self.name("q_norm.weight")] = ParamSpec((self.head_dim,), kind="vector", init="norm")
            specs[self.name("k_norm.weight")] = ParamSpec((self.head_dim,), kind="vector", init="norm")
        return specs

    def set_param(self, name: str, tensor: Tensor) -> None:
        local = name[len(self.prefix) + 1:] if self.prefix else name
        module, _, leaf = local.rpartition(".")
        if module in self._rows:
            start, size = self._rows[module]
            if leaf == "weight":
                if self.qkv_weight is None:  # the three projections share one matrix: one product per step
                    self.qkv_weight = torch.empty((self._width, self.hidden_size), dtype=tensor.dtype,
                                                  device=tensor.device)
                if tensor.dtype != self.qkv_weight.dtype:
                    raise ValueError(f"{name}: q, k and v projections must be stored in one dtype")
                self.qkv_weight[start:start + size].copy_(tensor)
            else:
                if self.qkv_bias is None:
                    self.qkv_bias = torch.zeros(self._width, dtype=torch.float32, device=tensor.device)
                self.qkv_bias[start:start + size].copy_(tensor)
        elif local == "o_proj.weight":
            self.o_weight = tensor
        elif local == "o_proj.bias":
            self.o_bias = tensor
        elif local == "q_norm.weight":
            self.q_norm = tensor
        elif local == "k_norm.weight":
            self.k_norm = tensor
        else:
            raise KeyError(name)

    def finalize(self) -> None:
        if self.qkv_bias is not None and self.qkv_weight.dtype != torch.float32:
            self.qkv_bias = self.qkv_bias.to(self.qkv_weight.dtype)
        if self.o_bias is not None and self.o_weight.dtype != torch.float32:
            self.o_bias = self.o_bias.to(self.o_weight.dtype)

    def split_qkv_weight(self) -> dict[str, Tensor]:
        """The three projection matrices back out of the fused one."""
        return {module: self.qkv_weight[start:start + size] for module, (start, size) in self._rows.items()}

    # ------------------------------------------------------------ running
    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(paged=PagedKV(self.num_kv_heads, self.head_dim, self.window))

    takes_stream = True

    def forward(self, x: Tensor, batch, cache: CacheView, writes_cache: bool = True,
                stream: Tensor | None = None) -> Tensor | None:
        rotary = self.position.rotary()
        inv_freq, rotary_dim = rotary if rotary is not None else (None, 0)
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 1.0
        if writes_cache:
            if self._single_tokens_only(batch, x, cache, rotary_dim):
                # norms, rotation, cache write and attention in one launch, which also adds up
                # the projection's partial sums where the product is faster with K in parts
                qkv = ops.linear_in_parts(x, self.qkv_weight) if self.qkv_bias is None else None
                if qkv is None:
                    qkv = ops.linear(x, self.qkv_weight, self.qkv_bias)
                attn = torch.empty((x.shape[0], self.q_size), dtype=x.dtype, device=x.device)
                ops.decode_attention_prepare(
                    qkv, self.q_norm, self.k_norm, inv_freq, cache.key_pages, cache.value_pages, attn,
                    batch.cu_q, batch.ctx_len, cache.block_table, q_heads=self.num_heads,
                    kv_heads=self.num_kv_heads, head_dim=self.head_dim, eps=eps, scale=self.scale,
                    window=self.window, max_ctx=batch.max_ctx)
                return ops.linear_update(attn, self.o_weight, self.o_bias, stream)
            qkv = ops.linear(x, self.qkv_weight, self.qkv_bias)
        else:  # another call wrote the keys and values this one reads: only q is needed
            bias = None if self.qkv_bias is None else self.qkv_bias[:self.q_size]
            qkv = ops.linear(x, self.qkv_weight[:self.q_size], bias)
        ops.qk_norm_rope_write(
            qkv, self.q_norm, self.k_norm, inv_freq, batch.positions, batch.token_seq,
            cache.block_table, cache.key_pages, cache.value_pages, q_heads=self.num_heads,
            kv_heads=self.num_kv_heads, head_dim=self.head_dim, rotary_dim=rotary_dim, eps=eps,
            write_kv=writes_cache)
        attn = torch.empty((x.shape[0], self.q_size), dtype=x.dtype, device=x.device)
        ops.paged_attention(
            qkv, cache.key_pages, cache.value_pages, attn, batch.cu_q, batch.ctx_len, cache.block_table,
            num_seqs=batch.num_seqs, max_q_len=batch.max_q_len, q_heads=self.num_heads,
            kv_heads=self.num_kv_heads, head_dim=self.head_dim, scale=self.scale, window=self.window,
            num_decode=batch.num_decode, max_ctx=batch.max_ctx)
        return ops.linear_update(attn, self.o_weight, self.o_bias, stream)   # float32 update for the residual sum

    def _single_tokens_only(self, batch, x: Tensor, cache: CacheView, rotary_dim: int) -> bool:
        """Every sequence of the step brings one token, and the sizes are ones that the
        decode kernel prepares queries and keys for itself."""
        return (batch.num_decode is not None and batch.num_decode == batch.num_seqs == x.shape[0]
                and ops.decode_prepare_supported(
                    x.dtype, q_heads=self.num_heads, kv_heads=self.num_kv_heads, head_dim=self.head_dim,
                    rotary_dim=rotary_dim, block_size=cache.key_pages.shape[2]))

    def token_inputs(self):
        return self.position.token_inputs()

    def kernel_libraries(self):
        return {"qk_rope", "attention_generic", "attention_decode", "attention_prefill", "gemm_f32", "gemm_skinny", "gemm_mid", "gemm_wide"}


register_part("mixer", "gqa_attention", GroupedQueryAttention)
