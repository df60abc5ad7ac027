"""Token embedding and the language-model head.

Embedding: ``h0 = E[ids]`` (reference: src/forge_engine/qwen3.py:325), widened
to the float32 residual stream.  Head: ``logits = z @ W^T`` in float32, with W
the embedding matrix when tied (qwen3.py:336) or ``lm_head.weight`` otherwise;
only the rows that the step asks for are multiplied.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, Embedding, Head, ParamSpec, Residual


class TokenEmbedding(Embedding):
    def __init__(self, ctx: BuildContext, prefix: str, *, vocab_size: int, hidden_size: int) -> None:
        super().__init__(ctx, prefix)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.weight: Tensor | None = None

    def param_specs(self):
        return {self.name("weight"): ParamSpec((self.vocab_size, self.hidden_size))}

    def set_param(self, name: str, tensor: Tensor) -> None:
        if name != self.name("weight"):
            raise KeyError(name)
        self.weight = tensor

    def forward(self, batch) -> Residual:
        h = torch.empty((batch.num_tokens, self.hidden_size), dtype=torch.float32, device=self.weight.device)
        ops.embed_rows(batch.token_ids, self.weight, h)
        return Residual(h)

    def kernel_libraries(self):
        return {"rowwise"}


class LMHead(Head):
    def __init__(self, ctx: BuildContext, prefix: str, *, vocab_size: int, hidden_size: int,
                 tied: bool = False) -> None:
        super().__init__(ctx, prefix)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied = tied
        self.weight: Tensor | None = None
        self._embedding: TokenEmbedding | None = None

    def tie(self, embedding: TokenEmbedding) -> None:
        self._embedding = embedding

    def param_specs(self):
        if self.tied:
            return {}
        return {self.name("weight"): ParamSpec((self.vocab_size, self.hidden_size))}

    def set_param(self, name: str, tensor: Tensor) -> None:
        if self.tied or name != self.name("weight"):
            raise KeyError(name)
        self.weight = tensor

    def matrix(self) -> Tensor:
        return self._embedding.weight if self.tied else self.weight

    def forward(self, z: Tensor) -> Tensor:
        # float32 accumulation and float32 logits in both modes (no rounding of the logits)
        return ops.linear(z, self.matrix(), out_dtype=torch.float32)

    def kernel_libraries(self):
        return {"gemm_f32", "gemm_skinny"}


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "lm_head", LMHead)
