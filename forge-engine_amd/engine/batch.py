"""The flat batch of one step: the tokens of every request in it, one after the
other, with the metadata the kernels index by."""

from __future__ import annotations

from dataclasses import dataclass, field
from functools import cached_property

import torch
from torch import Tensor


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens (a portion of its prompt,
    or one decoded token) and the places among them whose logits are wanted."""

    request_id: str
    tokens: list[int]
    want: list[int] = field(default_factory=list)
    # per-token integers by name, for models whose parts ask for them (``token_inputs``): a row
    # (or one integer) for each of ``tokens``.  A name that is left out gets the token's position
    # on every axis.
    inputs: dict | None = None


@dataclass
class StepBatch:
    num_tokens: int
    num_seqs: int
    num_wanted: int
    max_q_len: int
    max_ctx: int
    num_decode: int | None  # sequences that bring exactly one token (None: not known on the host)
    token_ids: Tensor       # int32 [T]
    positions: Tensor       # int32 [T]   absolute position of each token in its request
    token_seq: Tensor       # int32 [T]   index of the token's request within the batch
    cu_q: Tensor            # int32 [B+1] prefix sums of the requests' token counts
    ctx_len: Tensor         # int32 [B]   tokens the request holds after this step
    ctx_before: Tensor      # int32 [B]   tokens it held before
    state_slots: Tensor     # int32 [B]   slot of its fixed-size state
    want_rows: Tensor       # int32 [W]   flat token indices whose logits are returned
    block_tables: list      # per cache group: int32 [B, max_blocks], -1 where no page
    inputs: dict            # name -> int32 [T, width]: what the model's parts asked for beside the positions
    request_ids: list       # host copies, for parts that decide on the host
    q_lens: list
    ctx_before_host: list
    state_slots_host: list


@dataclass(frozen=True)
class BatchLayout:
    """Where each part of a step's metadata lies in the step's one int32 buffer: what there is per
    token, per request, the wanted rows, a block table per cache group, and the per-token inputs
    that the model's parts asked for, name after name.  ``build_batch`` packs a step this way, and
    the buffers of captured steps are refilled through the same description."""

    num_tokens: int
    num_seqs: int
    num_wanted: int
    widths: tuple            # block-table width of every cache group
    token_inputs: tuple = ()   # (name, integers a token), in the order of the names

    @classmethod
    def of(cls, num_tokens: int, num_seqs: int, num_wanted: int, widths, token_inputs=None) -> "BatchLayout":
        return cls(num_tokens, num_seqs, num_wanted, tuple(widths), tuple(sorted((token_inputs or {}).items())))

    def parts(self):
        """(key, int32 entries) in the order of the buffer; a block table's key is ("table", group),
        a per-token input's ("input", name)."""
        t, b = self.num_tokens, self.num_seqs
        yield from (("token_ids", t), ("positions", t), ("token_seq", t), ("cu_q", b + 1), ("ctx_len", b),
                    ("ctx_before", b), ("state_slots", b), ("want_rows", self.num_wanted))
        for group, width in enumerate(self.widths):
            yield ("table", group), b * width
        for name, width in self.token_inputs:
            yield ("input", name), t * width

    @cached_property
    def spans(self) -> dict:
        found, offset = {}, 0
        for key, size in self.parts():
            found[key] = slice(offset, offset + size)
            offset += size
        return found

    @property
    def size(self) -> int:
        return sum(size for _, size in self.parts())

    def span(self, key) -> slice:
        return self.spans[key]

    def views(self, flat) -> dict:
        """The buffer's parts by key (of a tensor or an array): block tables as [requests, width],
        per-token inputs as [tokens, integers a token]."""
        found = {key: flat[span] for key, span in self.spans.items()}
        for group, width in enumerate(self.widths):
            found[("table", group)] = found[("table", group)].reshape(self.num_seqs, width)
        for name, width in self.token_inputs:
            found[("input", name)] = found[("input", name)].reshape(self.num_tokens, width)
        return found

    def batch(self, flat: Tensor, *, max_q_len: int, max_ctx: int, num_decode: int | None, request_ids=(), q_lens=(),
              ctx_before_host=(), state_slots_host=()) -> "StepBatch":
        """The step's batch over the device buffer ``flat``."""
        v = self.views(flat)
        return StepBatch(
            num_tokens=self.num_tokens, num_seqs=self.num_seqs, num_wanted=self.num_wanted, max_q_len=max_q_len,
            max_ctx=max_ctx, num_decode=num_decode, token_ids=v["token_ids"], positions=v["positions"],
            token_seq=v["token_seq"], cu_q=v["cu_q"], ctx_len=v["ctx_len"], ctx_before=v["ctx_before"],
            state_slots=v["state_slots"], want_rows=v["want_rows"],
            block_tables=[v[("table", group)] for group in range(len(self.widths))],
            inputs={name: v[("input", name)] for name, _ in self.token_inputs}, request_ids=list(request_ids),
            q_lens=list(q_lens), ctx_before_host=list(ctx_before_host), state_slots_host=list(state_slots_host))


def token_input_values(entry: StepEntry, name: str, width: int, start: int) -> list[int]:
    """One named per-token input for an entry's tokens, row after row: what the entry brings, else
    the token's position (``start`` is the first token's) on every axis."""
    count = len(entry.tokens)
    given = None if entry.inputs is None else entry.inputs.get(name)
    if given is None:
        return [position for position in range(start, start + count) for _ in range(width)]
    rows = [list(row) if isinstance(row, (list, tuple)) else [row] for row in given]
    if len(rows) != count or any(len(row) != width for row in rows):
        raise ValueError(f"input '{name}' of request '{entry.request_id}' must hold {count} rows of {width} integers")
    return [int(value) for row in rows for value in row]


def build_batch(entries, lengths_before, state_slots, tables_per_group, device, *, widths=None,
                static=None, max_ctx=None, token_inputs=None) -> StepBatch:
    """Pack the step's metadata into one int32 buffer and copy it to the
    device in one transfer.  ``tables_per_group[g][i]`` is request i's page
    list in cache group g.

    ``widths`` fixes the block tables' widths (else: the longest table);
    ``static`` = (pinned host buffer, device buffer) makes the batch live at
    fixed addresses, refilled in place, which is what a captured graph reads;
    ``max_ctx`` overrides the host-side context bound (a graph is captured for
    a bound, not for one step's lengths); ``token_inputs`` (name -> integers a token) are the
    per-token inputs that the model's parts asked for, laid out behind the block tables in the
    order of their names."""
    num_seqs = len(entries)
    q_lens = [len(e.tokens) for e in entries]
    total = sum(q_lens)
    token_ids, positions, token_seq, want_rows = [], [], [], []
    cu_q = [0]
    for i, entry in enumerate(entries):
        start = lengths_before[i]
        token_ids.extend(entry.tokens)
        positions.extend(range(start, start + q_lens[i]))
        token_seq.extend([i] * q_lens[i])
        want_rows.extend(cu_q[-1] + w for w in entry.want)
        cu_q.append(cu_q[-1] + q_lens[i])
    ctx_len = [lengths_before[i] + q_lens[i] for i in range(num_seqs)]
    if widths is None:
        widths = [max(1, max((len(t) for t in tables), default=1)) for tables in tables_per_group]
    layout = BatchLayout.of(total, num_seqs, len(want_rows), widths, token_inputs)
    values = {"token_ids": token_ids, "positions": positions, "token_seq": token_seq, "cu_q": cu_q, "ctx_len": ctx_len,
              "ctx_before": list(lengths_before), "state_slots": list(state_slots), "want_rows": want_rows}
    for group, (tables, width) in enumerate(zip(tables_per_group, widths)):
        flat_table = values[("table", group)] = []
        for table in tables:
            if len(table) > width:
                raise ValueError(f"a block table of {len(table)} pages does not fit the width {width}")
            flat_table.extend(table)
            flat_table.extend([-1] * (width - len(table)))
    for name, width in layout.token_inputs:
        values[("input", name)] = [v for i, entry in enumerate(entries)
                                   for v in token_input_values(entry, name, width, lengths_before[i])]
    host = torch.tensor([v for key, _ in layout.parts() for v in values[key]], dtype=torch.int32)
    if static is not None:
        host_static, flat = static
        if host.numel() > flat.numel():
            raise ValueError("the step does not fit its static buffer")
        host_static[:host.numel()].copy_(host)
        flat[:host.numel()].copy_(host_static[:host.numel()], non_blocking=True)
    else:
        if device.type == "cuda":
            host = host.pin_memory()
        flat = host.to(device, non_blocking=True)
    return layout.batch(flat, max_q_len=max(q_lens), max_ctx=max(ctx_len) if max_ctx is None else max_ctx,
                        num_decode=sum(1 for n in q_lens if n == 1), request_ids=[e.request_id for e in entries],
                        q_lens=q_lens, ctx_before_host=lengths_before, state_slots_host=state_slots)


def static_batch(flat: Tensor, layout: BatchLayout, *, max_q_len: int, max_ctx: int, num_decode: int | None = None) -> StepBatch:
    """The batch of a captured step: views into a device buffer at fixed addresses, for
    ``layout.num_seqs`` sequences of which some may be empty.  What the kernels cannot read from
    the buffer is a bound (``max_q_len``, ``max_ctx``) or unknown (how many sequences bring one
    token, unless the caller knows that none ever does: ``num_decode=0``); the host-side lists are
    not filled in, so a model with a part that reads them is not captured."""
    return layout.batch(flat, max_q_len=max_q_len, max_ctx=max_ctx, num_decode=num_decode)
