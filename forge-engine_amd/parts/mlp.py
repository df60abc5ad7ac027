"""Gated SiLU feed-forward: ``down(silu(gate(x)) * up(x))``, no biases
(reference: src/forge_engine/qwen3.py:210-227).  gate and up share one fused
matrix [2I, H] so that a step makes one product for both."""

from __future__ import annotations

import torch
from torch import Tensor

from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, FeedForward, ParamSpec


class SwiGLU(FeedForward):
    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, intermediate_size: int) -> None:
        super().__init__(ctx, prefix)
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up_weight: Tensor | None = None
        self.down_weight: Tensor | None = None

    def param_specs(self):
        inter, hidden = self.intermediate_size, self.hidden_size
        return {
            self.name("gate_proj.weight"): ParamSpec((inter, hidden)),
            self.name("up_proj.weight"): ParamSpec((inter, hidden)),
            self.name("down_proj.weight"): ParamSpec((hidden, inter)),
        }

    def set_param(self, name: str, tensor: Tensor) -> None:
        inter = self.intermediate_size
        if name in (self.name("gate_proj.weight"), self.name("up_proj.weight")):
            if self.gate_up_weight is None:
                self.gate_up_weight = torch.empty((2 * inter, self.hidden_size), dtype=tensor.dtype,
                                                  device=tensor.device)
            if tensor.dtype != self.gate_up_weight.dtype:
                raise ValueError(f"{name}: gate and up projections must be stored in one dtype")
            start = 0 if name == self.name("gate_proj.weight") else inter
            self.gate_up_weight[start:start + inter].copy_(tensor)
        elif name == self.name("down_proj.weight"):
            self.down_weight = tensor
        else:
            raise KeyError(name)

    takes_stream = True

    def forward(self, x: Tensor, batch=None, stream: Tensor | None = None) -> Tensor | None:
        act = ops.linear_swiglu(x, self.gate_up_weight)
        return ops.linear_update(act, self.down_weight, stream=stream)   # the update stays float32 for the residual sum

    def kernel_libraries(self):
        return {"rowwise", "gemm_f32", "gemm_skinny", "gemm_mid", "gemm_wide", "gemm_tile"}


register_part("feed_forward", "swiglu", SwiGLU)
