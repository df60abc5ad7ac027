"""Interfaces of the parts a decoder is put together from.

A part knows its own sizes and constants (constructor arguments), the tensors it
needs (``param_specs``) and how to run on a step's flat batch.  It never knows
which model it is in.  Roles:

* ``Embedding``:    token ids -> float32 residual stream [T, H]
* ``Norm``:         residual stream (+ pending update) -> normalised activations
* ``Mixer``:        activations [T, H] -> update [T, H]; may use the cache
* ``FeedForward``:  activations [T, H] -> update [T, H]
* ``PositionEncoding``: what a mixer needs to encode positions
* ``Block``:        the arrangement of the above in one layer
* ``Head``:         normalised rows -> float32 logits
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch
from torch import Tensor

from ..cache.spec import CacheNeeds, CacheView
from ..kernels import ops


@dataclass(frozen=True)
class ParamSpec:
    """One tensor a part reads from the checkpoint.

    kind: ``matrix`` (kept in the compute dtype), ``vector`` (norm weights and
    biases, widened to float32, which is exact), ``int_table`` (int32).
    ``init``: how the random-weights mode draws it: ``normal`` N(0, 0.02),
    ``norm`` 1 + N(0, 0.05), ``zeros``.
    """

    shape: tuple[int, ...]
    kind: str = "matrix"
    init: str = "normal"
    optional: bool = False


@dataclass
class BuildContext:
    device: torch.device
    dtype: torch.dtype  # compute dtype of activations and matrices: bfloat16 or float32


class Residual:
    """The float32 residual stream of one step with at most one update that has
    not been added yet, so that the add can be fused into the next norm."""

    def __init__(self, h: Tensor) -> None:
        self.h = h
        self.pending: Tensor | None = None

    def add(self, update: Tensor | None) -> None:
        """Leave an update pending; None: the part has added it into the stream itself."""
        self.flush()
        self.pending = update

    def open(self) -> Tensor:
        """The stream with nothing pending, for a part that adds its update itself."""
        return self.flush()

    def flush(self) -> Tensor:
        if self.pending is not None:
            ops.add_rows(self.h, self.pending)
            self.pending = None
        return self.h


class Part:
    role = ""
    # False for a part whose forward decides anything on the host from the step's
    # contents (lengths, slots): its steps are not replayed from a captured graph.
    graph_safe = True

    def __init__(self, ctx: BuildContext, prefix: str = "") -> None:
        self.ctx = ctx
        self.prefix = prefix

    def name(self, local: str) -> str:
        return f"{self.prefix}.{local}" if self.prefix else local

    def param_specs(self) -> dict[str, ParamSpec]:
        """Checkpoint name -> spec, for every tensor this part (and its
        sub-parts) reads."""
        return {}

    def set_param(self, name: str, tensor: Tensor) -> None:
        """Receive one loaded tensor (already on the device, already in the
        dtype its kind and storage call for)."""
        raise KeyError(name)

    def finalize(self) -> None:
        """Called once after every tensor was set."""

    def kernel_libraries(self) -> set[str]:
        return set()

    def token_inputs(self) -> dict[str, int]:
        """Per-token integers that this part reads beside the positions: name -> integers a token
        (a position encoding with several axes, a token type).  A step's entries bring them
        (``StepEntry.inputs``) and the part finds them as ``batch.inputs[name]``, int32 [T, width];
        tokens whose entry brings none get their position on every axis."""
        return {}


class Embedding(Part):
    role = "embedding"

    def forward(self, batch) -> Residual:
        raise NotImplementedError


class Norm(Part):
    role = "norm"

    def forward(self, residual: Residual, rows: Tensor | None = None) -> Tensor:
        """Add the pending update into the stream and return the normalised
        activations (of the rows listed, if given) in the compute dtype."""
        raise NotImplementedError


class PositionEncoding(Part):
    role = "position"

    def rotary(self) -> tuple[Tensor, int] | None:
        """(inv_freq float32 [rotary_dim / 2], rotary_dim) for mixers that rotate
        q and k, or None."""
        return None


class Mixer(Part):
    role = "mixer"
    # True for a part whose forward takes ``stream=`` (the float32 residual stream, nothing pending):
    # it may add its update into the stream itself, where its last product can do so for free, and
    # then returns None instead of the update.
    takes_stream = False

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds()

    def forward(self, x: Tensor, batch, cache: CacheView | None, writes_cache: bool = True) -> Tensor | None:
        raise NotImplementedError


class FeedForward(Part):
    role = "feed_forward"
    takes_stream = False   # as for a mixer

    def forward(self, x: Tensor, batch) -> Tensor | None:
        raise NotImplementedError


class Head(Part):
    role = "head"

    def forward(self, z: Tensor) -> Tensor:
        raise NotImplementedError


class Block(Part):
    role = "block"

    def __init__(self, ctx: BuildContext, mixer: Mixer, feed_forward: FeedForward,
                 norms: dict[str, Norm]) -> None:
        super().__init__(ctx)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms

    def children(self) -> list[Part]:
        return [self.mixer, self.feed_forward, *self.norms.values()]

    def forward(self, residual: Residual, batch, cache: CacheView | None, writes_cache: bool = True) -> None:
        raise NotImplementedError


def build_part(role: str, spec, ctx: BuildContext, **extra: Any) -> Part:
    """Instantiate the registered class for ``spec.kind`` with the spec's
    parameters."""
    from ..registry import part_class

    return part_class(role, spec.kind)(ctx, spec.prefix, **spec.params, **extra)
