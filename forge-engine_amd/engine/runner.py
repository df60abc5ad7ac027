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
from .batch import StepBatch, StepEntry, build_batch, static_batch_size

GRAPH_MAX_REQUESTS = 64      # decode steps of up to this many requests replay a captured graph
GRAPH_TABLE_STEP = 64        # block-table widths of graphs are multiples of this many pages
GRAPH_LIMIT = 24             # captured graphs kept (least recently used goes first)


class _DecodeGraph:
    """One captured decode step: fixed request count and block-table widths.
    The step's metadata lives in a static buffer that each replay refills."""

    def __init__(self, num_seqs: int, widths, device) -> None:
        size = static_batch_size(num_seqs, widths)
        self.host = torch.empty(size, dtype=torch.int32).pin_memory()
        self.dev = torch.zeros(size, dtype=torch.int32, device=device)
        self.widths = list(widths)
        self.graph = None
        self.logits = None
        self.views = None
        self.copied = torch.cuda.Event()   # the last upload of the host buffer


class ModelRunner:
    def __init__(self, model: DecoderModel, *, block_size: int, block_capacity: int,
                 num_state_slots: int, use_graphs: bool = True) -> None:
        self.model = model
        self.use_graphs = use_graphs and model.ctx.device.type == "cuda" and model.graph_safe
        self._graphs: dict[tuple, _DecodeGraph] = {}
        self.graph_replays = 0
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

    def _graphable(self, entries: list[StepEntry]) -> bool:
        return (self.use_graphs and len(entries) <= GRAPH_MAX_REQUESTS
                and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries))

    def _graph_step(self, entries: list[StepEntry]) -> Tensor:
        """A decode-only step (one token and one wanted row per request) as a
        replay of a captured HIP graph: the launches of a step cost more host
        time than the step takes on the GPU."""
        self._check(entries)
        before = [self.cache.length(e.request_id) for e in entries]
        self.cache.reserve({e.request_id: before[i] + 1 for i, e in enumerate(entries)})
        records = [self.cache.request(e.request_id) for e in entries]
        tables = [[record.tables[g] for record in records] for g in range(len(self.cache.groups))]
        widths = tuple(-(-max(1, max(len(t) for t in group)) // GRAPH_TABLE_STEP) * GRAPH_TABLE_STEP
                       for group in tables)
        key = (len(entries), widths)
        slot = self._graphs.pop(key, None)
        if slot is None:
            if len(self._graphs) >= GRAPH_LIMIT:
                self._graphs.pop(next(iter(self._graphs)))
            slot = _DecodeGraph(len(entries), widths, self.device)
        self._graphs[key] = slot   # most recently used last
        bound = max(widths, default=GRAPH_TABLE_STEP) * self.block_size
        slot.copied.synchronize()          # the pinned buffer is free to be rewritten
        batch = build_batch(entries, before, [r.state_slot for r in records], tables, self.device,
                            widths=widths, static=(slot.host, slot.dev), max_ctx=bound)
        slot.copied.record(torch.cuda.current_stream(self.device))
        if slot.graph is None:
            views = self.cache_views(batch)
            side = torch.cuda.Stream(device=self.device)
            side.wait_stream(torch.cuda.current_stream(self.device))
            with torch.cuda.stream(side):      # once eagerly: libraries load, scratch gets its size
                self.model.forward(batch, views)
            torch.cuda.current_stream(self.device).wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                slot.logits = self.model.forward(batch, views)
            slot.graph, slot.views = graph, views
        slot.graph.replay()
        self.graph_replays += 1
        for i, entry in enumerate(entries):
            self.cache.commit(entry.request_id, before[i] + 1)
        self.steps_run += 1
        return slot.logits

    @torch.inference_mode()
    def step(self, entries: list[StepEntry]) -> Tensor:
        """Run the entries' tokens as one batch; float32 logits [wanted, vocab]
        in the order of the entries and of each entry's ``want``.  Raises
        ``CacheCapacityError`` (and changes nothing) if pages run out.  The
        result of a decode-only step lives in a buffer that the next such step
        of the same shape overwrites."""
        if self._graphable(entries):
            return self._graph_step(entries)
        batch = self.prepare(entries)
        logits = self.model.forward(batch, self.cache_views(batch))
        for i, entry in enumerate(entries):
            self.cache.commit(entry.request_id, batch.ctx_before_host[i] + batch.q_lens[i])
        self.steps_run += 1
        return logits


__all__ = ["CacheCapacityError", "ModelRunner", "StepEntry"]
