"""The data that describes a model: which parts, with which sizes, under which
checkpoint names, run in which order.  An architecture is a function from its
configuration to a ``ModelPlan``; the decoder is built from the plan alone.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


@dataclass(frozen=True)
class PartSpec:
    """One part: its kind in the registry, its sizes and constants, and the
    prefix of its tensors' names in the checkpoint."""

    kind: str
    params: dict[str, Any] = field(default_factory=dict)
    prefix: str = ""


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a block arrangement over a mixer, a feed-forward and norms.
    Different layers of one model may name different kinds."""

    block: str
    mixer: PartSpec
    feed_forward: PartSpec
    norms: dict[str, PartSpec]


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.  ``layer`` indexes ``ModelPlan.layers`` (a
    layer may be named more than once).  ``cache`` names the cache slot the
    call uses: by default its own, else that of an earlier call, in which case
    ``writes_cache`` is False and the mixer only reads what the other wrote."""

    layer: int
    cache: int | None = None
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelPlan:
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    schedule: tuple[LayerCall, ...]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: frozenset = frozenset()
    max_positions: int | None = None

    def resolved_schedule(self) -> tuple[LayerCall, ...]:
        """The run order with every cache slot made explicit and checked."""
        calls = []
        for index, call in enumerate(self.schedule):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"schedule entry {index} names layer {call.layer} of {len(self.layers)}")
            slot = index if call.cache is None else call.cache
            if call.cache is not None and call.cache != index:
                if call.writes_cache:
                    raise ValueError(f"schedule entry {index} shares cache slot {slot} and must not write it")
                if not (0 <= slot < index) or not calls[slot].writes_cache:
                    raise ValueError(f"schedule entry {index} reads cache slot {slot}, which no earlier entry writes")
            calls.append(LayerCall(call.layer, slot, call.writes_cache))
        return tuple(calls)
