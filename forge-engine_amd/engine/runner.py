"""The step function: one batch of (request, its next tokens) through the
model, from the cache that earlier steps left, to the logits at the wanted
places.  The runner owns the device side of the cache (page tensors, state
tensors) and drives the host-side cache manager; generation, the scheduler and
trace replay all go through ``ModelRunner.step``.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..cache import CacheCapacityError, CacheManager, CacheView, plan_groups
from ..kernels import library
from ..models.decoder import DecoderModel
from .batch import StepBatch, StepEntry, build_batch


class ModelRunner:
    def __init__(self, model: DecoderModel, *, block_size: int, block_capacity: int,
                 num_state_slots: int) -> None:
        self.model = model
        self.device = model.ctx.device
        self.dtype = model.ctx.dtype
        self.block_size = block_size
        needs = model.cache_needs()
        groups, self._where = plan_groups(needs, model.schedule)
        self.cache = CacheManager(groups, block_size=block_size, block_capacity=block_capacity,
                                  num_state_slots=num_state_slots)
        if self.device.type == "cuda":
            library.ensure_built(sorted(model.kernel_libraries()))
        # pages of a group: [slot in group, key|value, page, kv head, position in page, head dim]
        self.pages = [
            torch.zeros((len(g.slots), 2, block_capacity, g.kv_heads, block_size, g.head_dim),
                        dtype=self.dtype, device=self.device)
            for g in groups
        ]
        self.states: list[Tensor | None] = []
        for need in needs:
            if need.state is None:
                self.states.append(None)
            else:
                self.states.append(torch.zeros((num_state_slots, *need.state.shape),
                                               dtype=need.state.dtype or torch.float32, device=self.device))
        self.steps_run = 0

    # ------------------------------------------------------------ requests
    def begin(self, request_id: str) -> None:
        self.cache.begin(request_id)

    def end(self, request_id: str) -> None:
        self.cache.end(request_id)

    def length(self, request_id: str) -> int:
        return self.cache.length(request_id)

    # ---------------------------------------------------------------- step
    def _check(self, entries: list[StepEntry]) -> None:
        if not entries:
            raise ValueError("a step needs at least one entry")
        vocab = self.model.plan.vocab_size
        seen = set()
        for entry in entries:
            if entry.request_id in seen:
                raise ValueError(f"request '{entry.request_id}' appears twice in one step")
            seen.add(entry.request_id)
            if entry.request_id not in self.cache:
                raise KeyError(f"request '{entry.request_id}' was not begun")
            if not entry.tokens:
                raise ValueError(f"request '{entry.request_id}' brings no tokens")
            for token in entry.tokens:
                if not 0 <= token < vocab:
                    raise ValueError(f"token id {token} is outside the vocabulary of {vocab}")
            for place in entry.want:
                if not 0 <= place < len(entry.tokens):
                    raise ValueError(f"wanted place {place} is outside the {len(entry.tokens)} tokens of '{entry.request_id}'")

    def prepare(self, entries: list[StepEntry]) -> StepBatch:
        """Lease the pages the step needs (all or none) and build its batch."""
        self._check(entries)
        before = [self.cache.length(e.request_id) for e in entries]
        self.cache.reserve({e.request_id: before[i] + len(e.tokens) for i, e in enumerate(entries)})
        records = [self.cache.request(e.request_id) for e in entries]
        tables = [[record.tables[g] for record in records] for g in range(len(self.cache.groups))]
        return build_batch(entries, before, [r.state_slot for r in records], tables, self.device)

    def cache_views(self, batch: StepBatch) -> list[CacheView | None]:
        views: list[CacheView | None] = []
        for index, call in enumerate(self.model.schedule):
            state = self.states[index]
            if call.cache in self._where:
                g, j = self._where[call.cache]
                group = self.cache.groups[g]
                views.append(CacheView(self.pages[g][j, 0], self.pages[g][j, 1], batch.block_tables[g],
                                       self.block_size, group.window, state))
            elif state is not None:
                views.append(CacheView(state=state))
            else:
                views.append(None)
        return views

    @torch.inference_mode()
    def step(self, entries: list[StepEntry]) -> Tensor:
        """Run the entries' tokens as one batch; float32 logits [wanted, vocab]
        in the order of the entries and of each entry's ``want``.  Raises
        ``CacheCapacityError`` (and changes nothing) if pages run out."""
        batch = self.prepare(entries)
        logits = self.model.forward(batch, self.cache_views(batch))
        for i, entry in enumerate(entries):
            self.cache.commit(entry.request_id, batch.ctx_before_host[i] + batch.q_lens[i])
        self.steps_run += 1
        return logits


__all__ = ["CacheCapacityError", "ModelRunner", "StepEntry"]
