"""The step function: one batch of (request, its next tokens) through the
model, from the cache that earlier steps left, to the logits at the wanted
places.  The runner owns the device side of the cache (page tensors, state
tensors) and drives the host-side cache manager; generation, the scheduler and
trace replay all go through ``ModelRunner.step``.
"""

from __future__ import annotations

import numpy as np
import torch
from torch import Tensor

from ..cache import CacheCapacityError, CacheManager, CacheView, plan_groups
from ..kernels import library, ops
from ..models.decoder import DecoderModel
from .batch import BatchLayout, StepBatch, StepEntry, build_batch, static_batch, token_input_values

GRAPH_MAX_REQUESTS = 256     # steps of up to this many requests replay a captured graph
GRAPH_TABLE_STEP = 64        # block-table widths of graphs are multiples of this many pages
GRAPH_LIMIT = 24             # captured graphs kept (least recently used goes first)
PORTION_GRAPH_MAX_TOKENS = 4096   # steps with prompt portions of up to this many tokens may be captured
PORTION_GRAPH_SEQ_STEP = 8        # ... for a number of sequences rounded up to a multiple of this
PORTION_GRAPH_WANT_STEP = 8       # ... and of wanted rows likewise (none stays none)
# A capture costs two more runs of the step (the warm-up and the replay after a capture that runs
# nothing), and a replay saves the host's launches only: measured 0.2 ms a step, 3 % of a step of 256
# tokens and 1 % of one of 2,048.  So a shape is captured once it has come this often, the more often
# the larger the step: a workload of mixed prompts repeats few of its large shapes, and capturing each
# on its second sighting cost it 6 % of its time.
PORTION_GRAPH_SIGHTINGS = 2       # a shape is captured on this sighting ...
PORTION_GRAPH_SIGHTINGS_PER = 128  # ... plus one for every so many tokens of the step


class _DecodeGraph:
    """One captured decode step: fixed request count and block-table widths.
    The step's metadata lives in a static buffer (laid out as ``build_batch``
    lays out a batch of single tokens) that each replay refills; block-table
    rows are rewritten only when a request's table changed (a request that ended and began again
    under the same name holds another lease and other pages)."""

    def __init__(self, num_seqs: int, widths, device, token_inputs=None) -> None:
        n = num_seqs
        self.layout = BatchLayout.of(n, n, n, widths, token_inputs)
        self.host = torch.empty(self.layout.size, dtype=torch.int32).pin_memory()
        self.dev = torch.zeros(self.layout.size, dtype=torch.int32, device=device)
        self.np = self.host.numpy()
        self.part = self.layout.views(self.np)          # the pinned buffer's parts by name
        self.widths = list(widths)
        self.n = n
        self.np[:] = -1
        self.part["token_seq"][:] = np.arange(n)
        self.part["cu_q"][:] = np.arange(n + 1)
        self.part["want_rows"][:] = np.arange(n)
        self.row_keys = [[None] * n for _ in self.widths]
        self.graph = None
        self.logits = None
        self.views = None
        self.batch = None
        self.copied = torch.cuda.Event()   # the last upload of the host buffer

    def fill_inputs(self, entries, positions) -> None:
        """The per-token inputs of a step of single tokens at ``positions``."""
        for name, width in self.layout.token_inputs:
            rows = self.part[("input", name)]
            for i, entry in enumerate(entries):
                rows[i] = token_input_values(entry, name, width, int(positions[i]))

    def fill(self, tokens, before, records, entries) -> None:
        part = self.part
        before = np.asarray(before, dtype=np.int32)
        self.fill_inputs(entries, before)
        part["token_ids"][:] = tokens
        part["positions"][:] = before
        part["ctx_len"][:] = before + 1
        part["ctx_before"][:] = before
        part["state_slots"][:] = [r.state_slot for r in records]
        for g in range(len(self.widths)):
            keys, rows = self.row_keys[g], part[("table", g)]
            for i, record in enumerate(records):
                table = record.tables[g]
                key = (record.lease, len(table), record.first_block[g])   # pages are only ever appended or given back from the front
                if keys[i] != key:
                    rows[i, :len(table)] = table
                    rows[i, len(table):] = -1
                    keys[i] = key

    def move_on(self, tokens, entries) -> None:
        """The same requests again, each one token further: only the tokens change and every
        position moves on by one."""
        part = self.part
        part["token_ids"][:] = tokens
        part["positions"] += 1
        part["ctx_len"] += 1
        part["ctx_before"] += 1
        self.fill_inputs(entries, part["positions"])

    def feed(self, device_tokens: Tensor) -> None:
        """Tokens that are still on the device go into the step's buffer there."""
        tokens = self.dev[self.layout.span("token_ids")]
        tokens.copy_(device_tokens[:tokens.numel()])


class _SteadyDecode:
    """What the last decode step left for the next one, if that brings the same requests again:
    their records, the graph they replay, and how many more tokens fit into every request's last
    page (no page to reserve, no table row to rewrite until then)."""

    def __init__(self, ids, records, slot, room: int) -> None:
        self.ids, self.records, self.slot, self.room = ids, records, slot, room


class _PortionGraph:
    """One captured step that holds prompt portions (beside single tokens or not): fixed token
    count, sequence count and wanted-row count rounded up, block-table widths rounded up.
    Sequences beyond the step's own are empty (no tokens, so every kernel skips them), wanted
    rows beyond the step's own repeat row 0 and are cut off the result."""

    def __init__(self, num_tokens: int, num_seqs: int, num_wanted: int, widths, device, pad_state_slot: int = 0,
                 token_inputs=None) -> None:
        self.pad_state_slot = pad_state_slot
        self.layout = BatchLayout.of(num_tokens, num_seqs, num_wanted, widths, token_inputs)
        self.host = torch.empty(self.layout.size, dtype=torch.int32).pin_memory()
        self.dev = torch.zeros(self.layout.size, dtype=torch.int32, device=device)
        self.np = self.host.numpy()
        self.part = self.layout.views(self.np)
        self.np[:] = 0
        for g in range(len(self.layout.widths)):
            self.part[("table", g)][:] = -1
        self.graph = None
        self.logits = None
        self.copied = torch.cuda.Event()

    def fill(self, entries, before, records) -> None:
        part = self.part
        n = len(entries)
        at = rows = 0
        cu, want = part["cu_q"], part["want_rows"]
        for i, entry in enumerate(entries):
            count = len(entry.tokens)
            part["token_ids"][at:at + count] = entry.tokens
            part["positions"][at:at + count] = np.arange(before[i], before[i] + count)
            part["token_seq"][at:at + count] = i
            cu[i] = at
            for place in entry.want:
                want[rows] = at + place
                rows += 1
            for name, width in self.layout.token_inputs:
                part[("input", name)][at:at + count] = np.asarray(
                    token_input_values(entry, name, width, before[i]), dtype=np.int32).reshape(count, width)
            at += count
        cu[n:] = at                                                   # the other sequences are empty
        want[rows:] = 0
        part["ctx_len"][:n] = [before[i] + len(e.tokens) for i, e in enumerate(entries)]
        part["ctx_len"][n:] = 0
        part["ctx_before"][:n] = before
        part["ctx_before"][n:] = 0
        part["state_slots"][:n] = [r.state_slot for r in records]
        part["state_slots"][n:] = self.pad_state_slot
        for g in range(len(self.layout.widths)):
            table_rows = part[("table", g)]
            for i, record in enumerate(records):
                table = record.tables[g]
                table_rows[i, :len(table)] = table
                table_rows[i, len(table):] = -1
            table_rows[n:] = -1


class ModelRunner:
    def __init__(self, model: DecoderModel, *, block_size: int, block_capacity: int | list[int] | tuple[int, ...],
                 num_state_slots: int, use_graphs: bool = True, eager_sightings: int | None = None) -> None:
        """``block_capacity``: pages of every cache group's pool, or one count per group (a group
        whose window bounds what a request holds needs fewer).  ``eager_sightings``: how often a shape of a step with prompt portions runs eagerly before
        it is captured (None: by the step's size, see ``PORTION_GRAPH_SIGHTINGS``; a loop that repeats
        one shape, a benchmark for instance, passes 1)."""
        self.model = model
        self.eager_sightings = eager_sightings
        self.use_graphs = use_graphs and model.ctx.device.type == "cuda" and model.graph_safe
        self._graphs: dict[tuple, _DecodeGraph] = {}
        self._steady: _SteadyDecode | None = None
        self.steady_steps = 0
        self._portion_graphs: dict[tuple, _PortionGraph] = {}
        self._portion_seen: dict[tuple, int] = {}
        self.graph_replays = 0
        self.portion_graph_replays = 0
        self.device = model.ctx.device
        self.dtype = model.ctx.dtype
        self.block_size = block_size
        self.token_inputs = model.token_inputs()     # per-token integers beside the positions, name -> width
        needs = model.cache_needs()
        groups, self._where = plan_groups(needs, model.schedule)
        self.cache = CacheManager(groups, block_size=block_size, block_capacity=block_capacity,
                                  num_state_slots=num_state_slots)
        if self.device.type == "cuda":
            library.ensure_built(sorted(model.kernel_libraries()))
        # pages of a group, per cache slot: keys [page, kv head, position in page, head dim],
        # values transposed [page, kv head, value width, position in page]; a group that keeps keys
        # only has no value pages
        capacities = [pool.capacity for pool in self.cache.pools]
        self.key_pages = [
            torch.zeros((len(g.slots), capacity, g.kv_heads, block_size, g.head_dim),
                        dtype=self.dtype, device=self.device) for g, capacity in zip(groups, capacities)]
        self.value_pages = [
            torch.zeros((len(g.slots), capacity, g.kv_heads, g.value_width, block_size),
                        dtype=self.dtype, device=self.device) if g.value_width else None
            for g, capacity in zip(groups, capacities)]
        # fixed-size states of every schedule call, by name, each with its own shape and dtype; one row
        # more than there are slots: the empty sequences that pad a captured step point there, so that
        # a mixer that writes its state back never touches a live slot
        self.states: list[dict[str, Tensor]] = [
            {name: torch.zeros((num_state_slots + 1, *state.shape), dtype=state.dtype or torch.float32, device=self.device)
             for name, state in need.states().items()} for need in needs]
        self.pad_state_slot = num_state_slots
        self.steps_run = 0
        self.workspace = ops.Workspace()    # scratch that this runner's launches (and its captured graphs) share

    # ------------------------------------------------------------ requests
    def begin(self, request_id: str) -> None:
        """Lease a state slot and empty tables for the request.  The slot's fixed-size state starts
        at zero: the runner clears it here, so a mixer never has to know a request's first step."""
        record = self.cache.begin(request_id)
        for states in self.states:
            for state in states.values():
                state[record.state_slot].zero_()

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
            self._check_inputs(entry)

    def _check_inputs(self, entry: StepEntry) -> None:
        for name in entry.inputs or ():
            if name not in self.token_inputs:
                raise ValueError(f"request '{entry.request_id}' brings the token input '{name}', which no part of the model "
                                 f"asks for (asked for: {sorted(self.token_inputs)})")

    def prepare(self, entries: list[StepEntry]) -> StepBatch:
        """Lease the pages the step needs (all or none) and build its batch."""
        self._check(entries)
        before = [self.cache.length(e.request_id) for e in entries]
        self.cache.reserve({e.request_id: before[i] + len(e.tokens) for i, e in enumerate(entries)})
        records = [self.cache.request(e.request_id) for e in entries]
        tables = [[record.tables[g] for record in records] for g in range(len(self.cache.groups))]
        return build_batch(entries, before, [r.state_slot for r in records], tables, self.device, token_inputs=self.token_inputs)

    def cache_views(self, batch: StepBatch, scratch_state: bool = False) -> list[CacheView | None]:
        """What each schedule call sees of the cache in this step.  ``scratch_state``: fixed-size
        state is handed out as a copy, for a run whose effects on it must not stay."""
        views: list[CacheView | None] = []
        for index, call in enumerate(self.model.schedule):
            states = self.states[index]
            if scratch_state:
                states = {name: state.clone() for name, state in states.items()}
            if call.cache in self._where:
                g, j = self._where[call.cache]
                group = self.cache.groups[g]
                values = self.value_pages[g]
                views.append(CacheView(self.key_pages[g][j], None if values is None else values[j], batch.block_tables[g],
                                       self.block_size, group.window, states))
            elif states:
                views.append(CacheView(states=states))
            else:
                views.append(None)
        return views

    def _graphable(self, entries: list[StepEntry]) -> bool:
        return (self.use_graphs and len(entries) <= GRAPH_MAX_REQUESTS
                and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries))

    def _graph_step(self, entries: list[StepEntry], device_tokens: Tensor | None = None) -> Tensor:
        """A decode-only step (one token and one wanted row per request) as a
        replay of a captured HIP graph: the launches of a step cost more host
        time than the step takes on the GPU.  With ``device_tokens`` (int32
        [requests], on the device) the tokens of the entries are ignored and
        those are fed instead, by a copy on the device: the host need not have
        seen them yet."""
        cache = self.cache
        vocab = self.model.plan.vocab_size
        tokens = [e.tokens[0] for e in entries]
        if device_tokens is not None:
            if device_tokens.dtype != torch.int32 or device_tokens.device != self.device or device_tokens.numel() < len(entries):
                raise ValueError("device_tokens must be int32 on the runner's device, one per entry")
            tokens = [0] * len(entries)
        elif min(tokens) < 0 or max(tokens) >= vocab:
            raise ValueError(f"a token id is outside the vocabulary of {vocab}")
        for entry in entries:
            if entry.inputs:
                self._check_inputs(entry)
        steady = self._steady
        if (steady is not None and steady.room > 0 and len(entries) == len(steady.ids)
                and all(e.request_id == name for e, name in zip(entries, steady.ids))
                and cache.holds(steady.records)):
            # the same requests as the last step, none ended since, every one with room in its last
            # page: only the tokens change and every position moves on by one
            slot = steady.slot
            slot.copied.synchronize()
            slot.move_on(tokens, entries)
            slot.dev.copy_(slot.host, non_blocking=True)
            slot.copied.record(torch.cuda.current_stream(self.device))
            if device_tokens is not None:
                slot.feed(device_tokens)
            slot.graph.replay()
            for record in steady.records:
                record.length += 1
            steady.room -= 1
            self.steady_steps += 1
            self.graph_replays += 1
            self.steps_run += 1
            return slot.logits
        self._steady = None
        records = [cache.request(e.request_id) for e in entries]
        if len({e.request_id for e in entries}) != len(entries):
            raise ValueError("a request appears twice in one step")
        before = [r.length for r in records]
        need = {r.request_id: b + 1 for r, b in zip(records, before)
                if any(len(t) * self.block_size <= b for t in r.tables)}
        if need:
            cache.reserve(need)
        groups = range(len(cache.groups))
        widths = tuple(-(-max(1, max(len(r.tables[g]) for r in records)) // GRAPH_TABLE_STEP) * GRAPH_TABLE_STEP
                       for g in groups)
        key = (len(entries), widths)
        slot = self._graphs.pop(key, None)
        if slot is None:
            if len(self._graphs) >= GRAPH_LIMIT:
                self._graphs.pop(next(iter(self._graphs)))
            slot = _DecodeGraph(len(entries), widths, self.device, self.token_inputs)
        self._graphs[key] = slot   # most recently used last
        slot.copied.synchronize()          # the pinned buffer is free to be rewritten
        slot.fill(tokens, before, records, entries)
        slot.dev.copy_(slot.host, non_blocking=True)
        slot.copied.record(torch.cuda.current_stream(self.device))
        if slot.graph is None:
            bound = max(widths, default=GRAPH_TABLE_STEP) * self.block_size
            tables = [[record.tables[g] for record in records] for g in groups]
            batch = build_batch(entries, before, [r.state_slot for r in records], tables, self.device,
                                widths=widths, static=(slot.host, slot.dev), max_ctx=bound, token_inputs=self.token_inputs)
            views = self.cache_views(batch)
            self._warm_up(batch)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                slot.logits = self.model.forward(batch, views)
            slot.graph, slot.views, slot.batch = graph, views, batch
        if device_tokens is not None:
            slot.feed(device_tokens)
        slot.graph.replay()
        self.graph_replays += 1
        cache.commit_single_tokens(records)
        self.steps_run += 1
        if not any(group.window is not None for group in cache.groups):   # a window gives pages back as it moves
            room = min(len(table) * self.block_size - record.length for record in records for table in record.tables)
            self._steady = _SteadyDecode(tuple(e.request_id for e in entries), records, slot, room)
        return slot.logits

    def _warm_up(self, batch: StepBatch) -> None:
        """Run the step once eagerly before it is captured (libraries load, scratch gets its
        size).  The step is then captured (which runs nothing) and replayed, so its effects would
        happen twice: writes of keys and values into pages give the same pages both times, but a
        mixer's update of its fixed-size state does not, so this run gets a copy of the state."""
        views = self.cache_views(batch, scratch_state=True)
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(side):
            self.model.forward(batch, views)
        torch.cuda.current_stream(self.device).wait_stream(side)

    def _portion_key(self, entries: list[StepEntry]):
        """The shape under which a step with prompt portions may be captured, or None."""
        if not self.use_graphs or len(entries) > GRAPH_MAX_REQUESTS:
            return None
        tokens = sum(len(e.tokens) for e in entries)
        if tokens > PORTION_GRAPH_MAX_TOKENS:
            return None
        seqs = -(-len(entries) // PORTION_GRAPH_SEQ_STEP) * PORTION_GRAPH_SEQ_STEP
        wanted = sum(len(e.want) for e in entries)
        wanted = -(-wanted // PORTION_GRAPH_WANT_STEP) * PORTION_GRAPH_WANT_STEP
        singles = any(len(e.tokens) == 1 for e in entries)    # a step without single tokens launches no kernel for them
        return tokens, seqs, wanted, singles

    def _portion_graph_step(self, entries: list[StepEntry], shape) -> Tensor | None:
        """A step with prompt portions as a replay of a captured graph, once its shape (token
        count, sequence and wanted-row counts rounded up, table widths rounded up) has come
        often enough: a scheduler that fills its token budget repeats few shapes.  None if the
        step is to run eagerly (the first sightings of a shape)."""
        cache = self.cache
        self._check(entries)
        records = [cache.request(e.request_id) for e in entries]
        before = [r.length for r in records]
        groups = range(len(cache.groups))
        after = [b + len(e.tokens) for b, e in zip(before, entries)]
        pages = -(-max(after) // self.block_size)
        widths = tuple(-(-pages // GRAPH_TABLE_STEP) * GRAPH_TABLE_STEP for _ in groups)
        key = (*shape, widths)
        slot = self._portion_graphs.pop(key, None)
        if slot is None:
            seen = self._portion_seen.pop(key, 0)
            if len(self._portion_seen) >= 4 * GRAPH_LIMIT:
                self._portion_seen.pop(next(iter(self._portion_seen)))
            self._portion_seen[key] = seen + 1
            eager = self.eager_sightings
            if eager is None:
                eager = PORTION_GRAPH_SIGHTINGS - 1 + shape[0] // PORTION_GRAPH_SIGHTINGS_PER
            if seen < eager:
                return None
            if len(self._portion_graphs) >= GRAPH_LIMIT:
                self._portion_graphs.pop(next(iter(self._portion_graphs)))
            slot = _PortionGraph(shape[0], shape[1], shape[2], widths, self.device, self.pad_state_slot, self.token_inputs)
        self._portion_graphs[key] = slot
        cache.reserve({e.request_id: n for e, n in zip(entries, after)})
        records = [cache.request(e.request_id) for e in entries]
        slot.copied.synchronize()
        slot.fill(entries, before, records)
        slot.dev.copy_(slot.host, non_blocking=True)
        slot.copied.record(torch.cuda.current_stream(self.device))
        if slot.graph is None:
            batch = static_batch(slot.dev, slot.layout, max_q_len=shape[0],
                                 max_ctx=widths[0] * self.block_size if widths else 0,
                                 num_decode=None if shape[3] else 0)
            views = self.cache_views(batch)
            self._warm_up(batch)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                slot.logits = self.model.forward(batch, views)
            slot.graph, slot.views, slot.batch = graph, views, batch
        slot.graph.replay()
        self.portion_graph_replays += 1
        for entry, length in zip(entries, after):
            cache.commit(entry.request_id, length)
        self.steps_run += 1
        return slot.logits[:sum(len(e.want) for e in entries)]

    @torch.inference_mode()
    def step(self, entries: list[StepEntry], device_tokens: Tensor | None = None) -> Tensor:
        """Run the entries' tokens as one batch; float32 logits [wanted, vocab]
        in the order of the entries and of each entry's ``want``.  Raises
        ``CacheCapacityError`` (and changes nothing) if pages run out.  The
        result of a step that replays a captured graph lives in a buffer that
        the next step of the same shape overwrites.

        ``device_tokens`` (int32 [entries] on the device): for a step of single
        tokens that replays a graph (``feeds_from_device``), the token of entry i
        is ``device_tokens[i]`` whatever the entry holds, so that a step can be
        launched before the host has read the tokens that the step before
        sampled."""
        with ops.use_workspace(self.workspace):
            if device_tokens is not None:
                if not self._graphable(entries):
                    raise ValueError("tokens are fed from the device only into steps of single tokens that replay a graph")
                return self._graph_step(entries, device_tokens)
            return self._step(entries)

    def feeds_from_device(self, entries: list[StepEntry]) -> bool:
        """Whether ``step(entries, device_tokens=...)`` serves this step."""
        return self._graphable(entries)

    def _step(self, entries: list[StepEntry]) -> Tensor:
        if self._graphable(entries):
            return self._graph_step(entries)
        self._steady = None        # any other step may move the requests that the last decode step left
        shape = self._portion_key(entries) if entries else None
        if shape is not None:
            logits = self._portion_graph_step(entries, shape)
            if logits is not None:
                return logits
        batch = self.prepare(entries)
        logits = self.model.forward(batch, self.cache_views(batch))
        for i, entry in enumerate(entries):
            self.cache.commit(entry.request_id, batch.ctx_before_host[i] + batch.q_lens[i])
        self.steps_run += 1
        return logits


__all__ = ["CacheCapacityError", "ModelRunner", "StepEntry"]
