"""RMSNorm over the residual stream, fused with the add of the pending update.

``y = sum * rsqrt(mean(sum^2) + eps) * w`` with ``sum = h + update``
(reference: src/forge_engine/qwen3.py:99-105 and kernels/__init__.py:12-26).
The reference rounds the normalised value to the model dtype before the weight
product; here the whole expression is float32 with one rounding at the store.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, Norm, ParamSpec, Residual


class RMSNorm(Norm):
    def __init__(self, ctx: BuildContext, prefix: str, *, size: int, eps: float) -> None:
        super().__init__(ctx, prefix)
        self.size = size
        self.eps = float(eps)
        self.weight: Tensor | None = None

    def param_specs(self):
        return {self.name("weight"): ParamSpec((self.size,), kind="vector", init="norm")}

    def set_param(self, name: str, tensor: Tensor) -> None:
        if name != self.name("weight"):
            raise KeyError(name)
        self.weight = tensor

    def forward(self, residual: Residual, rows: Tensor | None = None) -> Tensor:
        if rows is not None:    # the chosen rows of stream + pending update; both are left as they are
            h = residual.h
            out = torch.empty((rows.numel(), self.size), dtype=self.ctx.dtype, device=h.device)
            return ops.add_rmsnorm(h, residual.pending, self.weight, self.eps, out, rows=rows, store_sum=False)
        update, residual.pending = residual.pending, None
        out = torch.empty((residual.h.shape[0], self.size), dtype=self.ctx.dtype, device=residual.h.device)
        return ops.add_rmsnorm(residual.h, update, self.weight, self.eps, out)

    def kernel_libraries(self):
        return {"rowwise"}


register_part("norm", "rms_norm", RMSNorm)
