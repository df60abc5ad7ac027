"""Rotary position encoding: the table of inverse frequencies that attention
rotates q and k with.

``inv_freq[j] = 1 / theta^(2j / R)``, j < R/2, in float32, computed with the
same expression as the reference (src/forge_engine/qwen3.py:352-360) so that the
angles ``float(position) * inv_freq[j]`` are bit-equal to its own.  R is the
number of rotated dims (the whole head unless ``rotary_dim`` says less); the
partner of dim j is j + R/2 (rotate-half pairing, qwen3.py:366-381).
"""

from __future__ import annotations

import torch

from ..registry import register_part
from .base import BuildContext, PositionEncoding


class RotaryPosition(PositionEncoding):
    def __init__(self, ctx: BuildContext, prefix: str = "", *, head_dim: int, theta: float,
                 rotary_dim: int | None = None) -> None:
        super().__init__(ctx, prefix)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {head_dim}")
        exponent = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
        self.inv_freq = (1.0 / (float(theta) ** exponent)).to(ctx.device)

    def rotary(self):
        return self.inv_freq, self.rotary_dim


class NoPosition(PositionEncoding):
    """No position information inside the mixer."""

    def __init__(self, ctx: BuildContext, prefix: str = "") -> None:
        super().__init__(ctx, prefix)


register_part("position", "rotary", RotaryPosition)
register_part("position", "none", NoPosition)
