"""The flat batch of one step: the tokens of every request in it, one after the
other, with the metadata the kernels index by."""

from __future__ import annotations

from dataclasses import dataclass, field

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
    token_inputs = dict(sorted((token_inputs or {}).items()))
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
    flat_tables = []
    for tables, width in zip(tables_per_group, widths):
        for table in tables:
            if len(table) > width:
                raise ValueError(f"a block table of {len(table)} pages does not fit the width {width}")
            flat_tables.extend(table)
            flat_tables.extend([-1] * (width - len(table)))
    sections = [token_ids, positions, token_seq, cu_q, ctx_len, list(lengths_before), list(state_slots),
                want_rows, flat_tables]
    for name, width in token_inputs.items():
        sections.append([v for i, entry in enumerate(entries) for v in token_input_values(entry, name, width, lengths_before[i])])
    host = torch.tensor([v for section in sections for v in section], dtype=torch.int32)
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
    views = []
    offset = 0
    for section in sections:
        views.append(flat[offset:offset + len(section)])
        offset += len(section)
    block_tables = []
    table_flat = views[8]
    offset = 0
    for width in widths:
        block_tables.append(table_flat[offset:offset + num_seqs * width].view(num_seqs, width))
        offset += num_seqs * width
    inputs = {name: views[9 + i].view(total, width) for i, (name, width) in enumerate(token_inputs.items())}
    return StepBatch(
        num_tokens=total, num_seqs=num_seqs, num_wanted=len(want_rows), max_q_len=max(q_lens),
        max_ctx=max(ctx_len) if max_ctx is None else max_ctx,
        num_decode=sum(1 for n in q_lens if n == 1), token_ids=views[0], positions=views[1],
        token_seq=views[2], cu_q=views[3], ctx_len=views[4], ctx_before=views[5], state_slots=views[6],
        want_rows=views[7], block_tables=block_tables, inputs=inputs, request_ids=[e.request_id for e in entries],
        q_lens=q_lens, ctx_before_host=list(lengths_before), state_slots_host=list(state_slots))


def static_batch_size(num_seqs: int, widths, num_tokens: int | None = None, num_wanted: int | None = None,
                      token_inputs=None) -> int:
    """int32 entries of a batch of ``num_seqs`` requests (by default with one token and one
    wanted row each)."""
    tokens = num_seqs if num_tokens is None else num_tokens
    wanted = num_seqs if num_wanted is None else num_wanted
    return 3 * tokens + 4 * num_seqs + 1 + wanted + num_seqs * sum(widths) + tokens * sum((token_inputs or {}).values())


def token_input_places(num_seqs: int, widths, num_tokens: int, num_wanted: int, token_inputs) -> dict:
    """name -> (first int32 entry, integers a token) of the per-token inputs in a batch's buffer."""
    offset = static_batch_size(num_seqs, widths, num_tokens, num_wanted)
    places = {}
    for name, width in sorted((token_inputs or {}).items()):
        places[name] = (offset, width)
        offset += num_tokens * width
    return places


def static_batch(flat: Tensor, *, num_tokens: int, num_seqs: int, num_wanted: int, widths, max_q_len: int,
                 max_ctx: int, num_decode: int | None = None, token_inputs=None) -> StepBatch:
    """The batch of a captured step: views into a device buffer at fixed addresses, laid out as
    ``build_batch`` lays a batch out, for ``num_seqs`` sequences of which some may be empty.
    What the kernels cannot read from the buffer is a bound (``max_q_len``, ``max_ctx``) or
    unknown (how many sequences bring one token, unless the caller knows that none ever does:
    ``num_decode=0``); the host-side lists are not filled in, so a model with a part that reads
    them is not captured."""
    sizes = [num_tokens, num_tokens, num_tokens, num_seqs + 1, num_seqs, num_seqs, num_seqs, num_wanted]
    views, offset = [], 0
    for size in sizes:
        views.append(flat[offset:offset + size])
        offset += size
    block_tables = []
    for width in widths:
        block_tables.append(flat[offset:offset + num_seqs * width].view(num_seqs, width))
        offset += num_seqs * width
    inputs = {name: flat[at:at + num_tokens * width].view(num_tokens, width)
              for name, (at, width) in token_input_places(num_seqs, widths, num_tokens, num_wanted, token_inputs).items()}
    return StepBatch(
        num_tokens=num_tokens, num_seqs=num_seqs, num_wanted=num_wanted, max_q_len=max_q_len, max_ctx=max_ctx,
        num_decode=num_decode, token_ids=views[0], positions=views[1], token_seq=views[2], cu_q=views[3],
        ctx_len=views[4], ctx_before=views[5], state_slots=views[6], want_rows=views[7],
        block_tables=block_tables, inputs=inputs, request_ids=[], q_lens=[], ctx_before_host=[], state_slots_host=[])
