"""A decoder built from a ``ModelPlan``: embedding, layers run in the order of
the plan's schedule, final norm, head.  It knows no architecture: which parts,
which sizes and which order all come from the plan.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..cache.spec import CacheNeeds, CacheView
from ..parts.base import Block, BuildContext, ParamSpec, Part, build_part
from ..parts.plan import LayerCall, ModelPlan
from ..registry import part_class


class DecoderModel:
    def __init__(self, plan: ModelPlan, ctx: BuildContext) -> None:
        self.plan = plan
        self.ctx = ctx
        self.schedule: tuple[LayerCall, ...] = plan.resolved_schedule()
        self.embedding = build_part("embedding", plan.embedding, ctx)
        self.layers: list[Block] = []
        for spec in plan.layers:
            mixer = build_part("mixer", spec.mixer, ctx)
            feed_forward = build_part("feed_forward", spec.feed_forward, ctx)
            norms = {role: build_part("norm", norm_spec, ctx) for role, norm_spec in spec.norms.items()}
            self.layers.append(part_class("block", spec.block)(ctx, mixer, feed_forward, norms))
        self.final_norm = build_part("norm", plan.final_norm, ctx)
        self.head = build_part("head", plan.head, ctx)
        if getattr(self.head, "tied", False):
            self.head.tie(self.embedding)
        self._owners: dict[str, Part] = {}
        self._specs: dict[str, ParamSpec] = {}
        for part in self.parts():
            for name, spec in part.param_specs().items():
                if name in self._owners:
                    raise ValueError(f"tensor name '{name}' is claimed by two parts")
                self._owners[name] = part
                self._specs[name] = spec
        self._assigned: set[str] = set()

    # ------------------------------------------------------------- structure
    def parts(self) -> list[Part]:
        found: list[Part] = [self.embedding]
        for layer in self.layers:
            found.extend(layer.children())
        found.extend([self.final_norm, self.head])
        return found

    def param_specs(self) -> dict[str, ParamSpec]:
        return dict(self._specs)

    def ignorable_names(self) -> set[str]:
        """Tensors a checkpoint may hold that the model does not read: the head
        matrix of a model whose head is tied to the embedding."""
        if getattr(self.head, "tied", False):
            return {self.head.name("weight")}
        return set()

    def set_param(self, name: str, tensor: Tensor) -> None:
        self._owners[name].set_param(name, tensor)
        self._assigned.add(name)

    def finalize(self) -> None:
        missing = [n for n, s in self._specs.items() if n not in self._assigned and not s.optional]
        if missing:
            raise ValueError(f"tensors never loaded: {missing[:5]}")
        for part in self.parts():
            part.finalize()

    @property
    def graph_safe(self) -> bool:
        """Whether a decode step of this model may be captured and replayed."""
        return all(part.graph_safe for part in self.parts())

    def kernel_libraries(self) -> set[str]:
        names: set[str] = set()
        for part in self.parts():
            names |= part.kernel_libraries()
        return names

    def token_inputs(self) -> dict[str, int]:
        """The per-token inputs that the model's parts ask for, name -> integers a token."""
        asked: dict[str, int] = {}
        for part in self.parts():
            for name, width in part.token_inputs().items():
                if asked.setdefault(name, int(width)) != int(width):
                    raise ValueError(f"parts ask for the token input '{name}' at widths {asked[name]} and {width}")
        return asked

    def cache_needs(self) -> list[CacheNeeds]:
        """One entry per schedule call (what its mixer asks of the cache)."""
        return [self.layers[call.layer].mixer.cache_needs() for call in self.schedule]

    # --------------------------------------------------------------- running
    def forward(self, batch, cache_views: list[CacheView | None]) -> Tensor:
        """Run the step's tokens through every scheduled layer; float32 logits
        [len(batch.want_rows), vocab] at the wanted rows."""
        residual = self.embedding.forward(batch)
        for index, call in enumerate(self.schedule):
            self.layers[call.layer].forward(residual, batch, cache_views[index], call.writes_cache)
        if batch.num_wanted == 0:
            residual.flush()
            return torch.empty((0, self.plan.vocab_size), dtype=torch.float32, device=residual.h.device)
        z = self.final_norm.forward(residual, rows=batch.want_rows)
        return self.head.forward(z)
