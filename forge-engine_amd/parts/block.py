"""Arrangements of a mixer, a feed-forward and norms in one layer."""

from __future__ import annotations

from ..cache.spec import CacheView
from ..registry import register_part
from .base import Block, Residual


class PreNormBlock(Block):
    """``h += mixer(norm_in(h)); h += ffn(norm_post(h))`` (reference:
    src/forge_engine/qwen3.py:240-261).  Each add is left pending on the stream
    and fused into the next norm, unless the part's last product added it itself."""

    NORMS = ("input", "post_mixer")

    def forward(self, residual: Residual, batch, cache: CacheView | None, writes_cache: bool = True) -> None:
        x = self.norms["input"].forward(residual)
        if self.mixer.takes_stream:
            residual.add(self.mixer.forward(x, batch, cache, writes_cache, stream=residual.open()))
        else:
            residual.add(self.mixer.forward(x, batch, cache, writes_cache))
        y = self.norms["post_mixer"].forward(residual)
        if self.feed_forward.takes_stream:
            residual.add(self.feed_forward.forward(y, batch, stream=residual.open()))
        else:
            residual.add(self.feed_forward.forward(y, batch))


register_part("block", "pre_norm", PreNormBlock)
