"""Continuous batching above the step function.

The public surface follows the reference's concurrent engine
(src/forge_engine/scheduler.py:137-363): ``submit``, ``step``,
``run_until_idle``, ``cancel``, ``request``, ``forget``, ``snapshot``, ``idle``,
with the same states, the same round-robin order (every visited request goes to
the back of the queue, 365-385), the same admission by worst-case page
reservation (220-244) and the same finishing order (472-519).  What differs is
what a step is: the reference runs one model call per group of equal shapes
and never splits a prompt; here every selected request contributes to one flat
batch (portions of prompts beside single decoded tokens) and the token budget
cuts prompts into portions.

Overlapped decoding (``overlap_decode``).  While the same requests decode step after step
(greedily or with draws: a draw is keyed by the request's seed and the count of its tokens, which
the host knows without reading any), a step is launched with the tokens that the step before sampled still on the device, and
the host reads those tokens while the new step runs: the GPU does not wait for the scheduler
between two steps.  What the host sees is one step late: events come a step later, and a
request that samples its end-of-sequence token still rides in the step that was already
launched (its result there is dropped).  A request that reaches its token limit is known in
advance and never rides along.  Any other kind of step (a prompt portion, another set of
requests) first reads what is in flight.  The tokens that
requests generate are the same either way.

When pages run out.  ``admission="reserve"`` (default, the reference's policy):
a request is admitted only if the pages for its prompt plus ``max_new_tokens``
are unreserved, so a running request can never run out; ``submit`` raises
``OverloadedError`` instead.  ``admission="preempt"``: nothing is reserved; if a
step finds too few free pages, the request admitted last among those holding
pages gives its pages back and is queued again; it later recomputes its prompt
and the tokens it had generated.  Sampling is keyed by (seed, token index), so
a preempted request continues exactly as it would have.
"""

from __future__ import annotations

import secrets
from collections import deque
from dataclasses import dataclass, field
from enum import Enum
from typing import Sequence

from ..cache import CacheCapacityError
from ..config.engine import SchedulerConfig
from ..sampling.params import SamplingParams
from .batch import StepEntry
from .detokenizer import IncrementalDetokenizer


class RequestStatus(str, Enum):
    WAITING = "waiting"      # its prompt (or, after preemption, its history) is not yet in the cache
    RUNNING = "running"      # decoding: one token per step
    FINISHED = "finished"
    CANCELLED = "cancelled"
    FAILED = "failed"

    @property
    def terminal(self) -> bool:
        return self in (RequestStatus.FINISHED, RequestStatus.CANCELLED, RequestStatus.FAILED)


class OverloadedError(RuntimeError):
    """Admission cannot take the request now (request limit or pages)."""


@dataclass(frozen=True)
class RequestView:
    request_id: str
    status: RequestStatus
    prompt_tokens: int
    sampled_tokens: int
    reserved_blocks: int
    finish_reason: str | None
    error: str | None
    output_token_ids: tuple[int, ...] = ()
    text: str = ""


@dataclass(frozen=True)
class StreamEvent:
    request_id: str
    text: str
    status: RequestStatus
    token_ids: tuple[int, ...] = ()


@dataclass(frozen=True)
class SchedulerSnapshot:
    iteration: int
    waiting: int
    running: int
    terminal: int
    reserved_blocks: int
    allocated_blocks: int
    last_batch: tuple[str, ...]
    model_batches: tuple[tuple[str, ...], ...]
    last_batch_tokens: tuple[int, ...] = ()
    preemptions: int = 0


@dataclass
class _Request:
    request_id: str
    prompt: list[int]
    params: SamplingParams
    seed: int
    eos_ids: frozenset
    detokenizer: IncrementalDetokenizer | None
    reserved_blocks: list[int]                         # per cache group
    admitted: int
    status: RequestStatus = RequestStatus.WAITING
    outputs: list[int] = field(default_factory=list)   # sampled tokens that go back into the model
    fed: int = 0                                       # tokens of prompt + outputs already in the cache
    sampled_tokens: int = 0
    text: str = ""
    finish_reason: str | None = None
    error: str | None = None
    reservation_released: bool = False
    holds_cache: bool = False
    in_flight: bool = False                            # its last sampled token is still on the device, unread
    inputs: dict | None = None                         # per-token integers of the prompt by name (``StepEntry.inputs``)

    def feed(self) -> list[int]:
        return self.prompt + self.outputs

    def next_tokens(self, count: int) -> list[int]:
        """The next ``count`` tokens that go into the model: what follows ``fed`` in prompt +
        outputs, without building that list (a decoding request asks for one token a step)."""
        start, prompt = self.fed, self.prompt
        if start >= len(prompt):
            return self.outputs[start - len(prompt):start - len(prompt) + count]
        if start + count <= len(prompt):
            return prompt[start:start + count]
        return prompt[start:] + self.outputs[:start + count - len(prompt)]

    def next_inputs(self, count: int) -> dict | None:
        """The per-token inputs of the next ``count`` tokens: the prompt's rows as submitted; sampled
        tokens bring none (they get their position on every axis)."""
        if not self.inputs:
            return None
        start, found = self.fed, {}
        for name, rows in self.inputs.items():
            width = len(rows[0]) if isinstance(rows[0], (list, tuple)) else 1
            part = list(rows[start:start + count])
            part.extend([position] * width for position in range(start + len(part), start + count))
            found[name] = part
        return found

    def remaining(self) -> int:
        return len(self.prompt) + len(self.outputs) + (1 if self.in_flight else 0) - self.fed


class ConcurrentGenerationEngine:
    """Runs admitted requests in round-robin, token-budgeted steps."""

    def __init__(self, runner, sampler, default_sampling_params: SamplingParams | None = None,
                 scheduler_config: SchedulerConfig | None = None, tokenizer=None,
                 eos_token_ids=None) -> None:
        self._runner = runner
        self._sampler = sampler
        self._default_params = default_sampling_params or SamplingParams()
        self._config = scheduler_config or SchedulerConfig()
        self._tokenizer = tokenizer
        if eos_token_ids is None:
            eos_token_ids = getattr(runner.model.plan, "eos_token_ids", frozenset())
        self._eos_ids = frozenset(eos_token_ids)
        cache = runner.cache
        self._capacities = self._config.capacities(len(cache.pools))     # pages of each cache group's pool
        if cache.block_size != self._config.block_size or [pool.capacity for pool in cache.pools] != self._capacities:
            raise ValueError("the runner's cache pool does not match the scheduler configuration")
        self._requests: dict[str, _Request] = {}
        self._order: deque[str] = deque()
        self._reserved = [0] * len(self._capacities)                     # pages reserved in each group
        self._next_number = 1
        self._admitted = 0
        self._iteration = 0
        self._preemptions = 0
        self._last_batch: tuple[str, ...] = ()
        self._last_tokens: tuple[int, ...] = ()
        # the step whose sampled tokens the host has not read yet: (its requests, tokens and status on the device)
        self._flight: tuple[list[_Request], object] | None = None
        self.overlapped_steps = 0

    # ----------------------------------------------------------- properties
    @property
    def idle(self) -> bool:
        return self._flight is None and all(r.status.terminal for r in self._requests.values())

    @property
    def cache_pool(self):
        """The cache manager (page pools, tables, state slots)."""
        return self._runner.cache

    @property
    def config(self) -> SchedulerConfig:
        return self._config

    # ------------------------------------------------------------ admission
    def _tokens_of(self, prompt) -> list[int]:
        if isinstance(prompt, str):
            if self._tokenizer is None:
                raise ValueError("a text prompt needs a tokenizer; pass token ids")
            encoded = self._tokenizer.encode(prompt)
            prompt = getattr(encoded, "ids", encoded)
        tokens = [int(t) for t in prompt]
        if not tokens:
            raise ValueError("each request must contain one non-empty prompt")
        vocab = self._runner.model.plan.vocab_size
        for token in tokens:
            if not 0 <= token < vocab:
                raise ValueError(f"token id {token} is outside the vocabulary of {vocab}")
        return tokens

    def submit(self, prompt, *, request_id: str | None = None,
               sampling_params: SamplingParams | None = None, inputs: dict | None = None) -> str:
        """Admit a request (token ids, or text if a tokenizer is present).
        Raises ``OverloadedError`` if the request limit is reached or, under
        ``admission="reserve"``, its worst-case pages are not unreserved.
        ``inputs``: per-token integers of the prompt by name, for a model whose parts ask for
        them (a row for every prompt token)."""
        config = self._config
        active = sum(not r.status.terminal for r in self._requests.values())
        if active >= config.max_requests:
            raise OverloadedError(f"request limit {config.max_requests} is full")
        assigned = self._new_id() if request_id is None else request_id
        if assigned in self._requests:
            raise ValueError(f"duplicate request_id: {assigned}")
        params = sampling_params or self._default_params
        tokens = self._tokens_of(prompt)
        if inputs:
            asked = getattr(self._runner, "token_inputs", {})
            for name, rows in inputs.items():
                if name not in asked:
                    raise ValueError(f"the model asks for no token input '{name}' (it asks for {sorted(asked)})")
                if len(rows) != len(tokens):
                    raise ValueError(f"input '{name}' must hold a row for each of the {len(tokens)} prompt tokens")
        total = len(tokens) + params.max_new_tokens
        if config.max_context is not None and total > config.max_context:
            raise OverloadedError(f"request needs {total} positions but max_context is {config.max_context}")
        portion = min(config.token_budget, config.prefill_chunk or config.token_budget)
        # every cache group has a pool of its own: a group whose window bounds what a request holds
        # needs, and reserves, less than one that keeps every key
        needed = self._runner.cache.worst_case_pages(total, step_tokens=portion)
        for need, capacity in zip(needed, self._capacities):
            if need > capacity:
                raise OverloadedError(f"request needs {need} KV blocks but pool capacity is {capacity}")
        reserved = [0] * len(needed)
        if config.admission == "reserve":
            for need, capacity, taken in zip(needed, self._capacities, self._reserved):
                if need > capacity - taken:
                    raise OverloadedError(
                        f"request needs {need} KV blocks but only {capacity - taken} are unreserved")
            reserved = needed
        detokenizer = None
        if self._tokenizer is not None:
            detokenizer = IncrementalDetokenizer(self._tokenizer, params.stop_strings)
        elif params.stop_strings:
            raise ValueError("stop strings need a tokenizer")
        seed = params.seed if params.seed is not None else secrets.randbits(63)
        self._runner.begin(assigned)
        self._admitted += 1
        self._requests[assigned] = _Request(assigned, tokens, params, seed, self._eos_ids, detokenizer,
                                            reserved, self._admitted, holds_cache=True, inputs=inputs or None)
        self._order.append(assigned)
        self._reserved = [taken + more for taken, more in zip(self._reserved, reserved)]
        return assigned

    def cancel(self, request_id: str) -> bool:
        request = self._request(request_id)
        if request.status.terminal:
            return False
        request.status = RequestStatus.CANCELLED
        request.finish_reason = "cancelled"
        self._cleanup(request)
        return True

    # ----------------------------------------------------------------- step
    def _select_batch(self) -> list[tuple[_Request, int]]:
        """Round-robin: visit requests from the front of the queue; a decoding
        request costs one token, a waiting one a portion of what it still has
        to feed, cut to ``prefill_chunk`` and to the budget left (at least one
        token; a first pick is never refused).  Every visited request goes to
        the back, chosen or not."""
        config = self._config
        selected: list[tuple[_Request, int]] = []
        budget = config.token_budget
        for _ in range(len(self._order)):
            request_id = self._order.popleft()
            request = self._requests[request_id]
            if request.status.terminal:
                continue
            self._order.append(request_id)
            cost = min(request.remaining(), budget)   # budget >= 1 here: the loop ends when it is spent
            if config.prefill_chunk is not None:
                cost = min(cost, config.prefill_chunk)
            selected.append((request, cost))
            budget -= cost
            if len(selected) >= config.max_batch_size or budget == 0:
                break
        return selected

    def _pick_victim(self, keep: _Request | None) -> _Request | None:
        """The request admitted last among those that hold pages."""
        holders = [r for r in self._requests.values()
                   if not r.status.terminal and r.fed > 0 and r is not keep]
        return max(holders, key=lambda r: r.admitted) if holders else None

    def _preempt(self, request: _Request) -> None:
        self._runner.end(request.request_id)
        self._runner.begin(request.request_id)
        request.fed = 0
        request.status = RequestStatus.WAITING
        self._preemptions += 1

    # ------------------------------------------------- overlapped decode steps
    def _land(self) -> list[StreamEvent]:
        """Read the tokens of the step in flight and consume them."""
        events: list[StreamEvent] = []
        if self._flight is None:
            return events
        requests, both = self._flight
        self._flight = None
        try:
            tokens = self._sampler.read(both)
        except Exception as error:
            for request in requests:
                request.in_flight = False
            events.extend(self._fail([r for r in requests if not r.status.terminal], error))
            self._drop_terminal()
            return events
        for request, token in zip(requests, tokens):
            request.in_flight = False
            if not request.status.terminal:       # cancelled meanwhile, or ended in the step before: dropped
                events.extend(self._consume(request, token))
        self._drop_terminal()
        return events

    def _may_overlap(self, selected: list[tuple[_Request, int]]) -> bool:
        """A step of single tokens, every one the last of its request's history, none of which
        ends its request by the token limit, that the runner can feed from the device."""
        if not self._config.overlap_decode or not hasattr(self._sampler, "sample_on_device"):
            return False
        for request, count in selected:
            if count != 1 or request.remaining() != 1:
                return False
            if request.sampled_tokens + (1 if request.in_flight else 0) + 1 > request.params.max_new_tokens:
                return False
        feeds = getattr(self._runner, "feeds_from_device", None)
        return feeds is not None and feeds([StepEntry(r.request_id, [0], [0]) for r, _ in selected])

    def _overlapped_step(self, selected: list[tuple[_Request, int]]) -> list[StreamEvent] | None:
        """Launch the step on the tokens in flight (or, for the first of a run, on host tokens),
        sample on the device, then read and consume the step before.  None if it cannot be done
        (the caller then lands what is in flight and takes the plain path)."""
        requests = [r for r, _ in selected]
        if self._flight is not None:
            flying, both = self._flight
            if len(flying) != len(requests) or any(a is not b for a, b in zip(flying, requests)):
                return None
            entries = [StepEntry(r.request_id, [0], [0]) for r in requests]
            feed = both[0]
        else:
            entries = [StepEntry(r.request_id, r.next_tokens(1), [0]) for r in requests]
            feed = None
        try:
            logits = self._runner.step(entries, device_tokens=feed) if feed is not None else self._runner.step(entries)
        except CacheCapacityError:
            return None                             # nothing was changed: pages are reserved all or none
        except Exception as error:
            return self._land() + self._fail_batch(requests, error)
        # from here on the step has run: the cache holds one token more for every request
        for request in requests:
            request.fed += 1
        try:
            # a request with a token in flight has drawn one more than it has consumed
            launched = self._sampler.sample_on_device(
                logits, [r.params for r in requests], [r.seed for r in requests],
                [r.sampled_tokens + (1 if r.in_flight else 0) for r in requests])
        except Exception as error:
            return self._land() + self._fail_batch(requests, error)
        self._last_batch = tuple(r.request_id for r in requests)
        self._last_tokens = tuple(1 for _ in requests)
        events = self._land()                       # the step before, read while this one runs
        for request in requests:
            request.in_flight = True
        self._flight = (requests, launched)
        self.overlapped_steps += 1
        return events

    def step(self) -> list[StreamEvent]:
        """One model step over a fresh batch; returns what it produced."""
        order_before = deque(self._order)
        selected = self._select_batch()
        self._iteration += 1
        events: list[StreamEvent] = []
        if selected and self._may_overlap(selected):
            produced = self._overlapped_step(selected)
            if produced is not None:
                return produced
        if self._flight is not None:
            # another kind of step follows: first learn what the step in flight sampled, then choose again,
            # from the queue as it stood (a selection that did not run must not cost anyone a turn)
            events.extend(self._land())
            self._order = order_before
            self._drop_terminal()
            selected = self._select_batch()
        while True:
            self._last_batch = tuple(r.request_id for r, _ in selected)
            self._last_tokens = tuple(n for _, n in selected)
            if not selected:
                return events
            entries, wanted = [], []
            for request, count in selected:
                tokens = request.next_tokens(count)
                complete = count == request.remaining()
                entries.append(StepEntry(request.request_id, tokens, [count - 1] if complete else [], request.next_inputs(count)))
                if complete:
                    wanted.append(request)
            try:
                logits = self._runner.step(entries)
                for request, count in selected:
                    request.fed += count
                tokens = self._sampler.sample(
                    logits, [r.params for r in wanted], [r.seed for r in wanted],
                    [r.sampled_tokens for r in wanted])
                break
            except CacheCapacityError as error:
                if self._config.admission != "preempt":
                    events.extend(self._fail([r for r, _ in selected], error))
                    self._drop_terminal()
                    return events
                oldest = min((r for r, _ in selected), key=lambda r: r.admitted)
                victim = self._pick_victim(keep=oldest)
                if victim is not None:
                    self._preempt(victim)
                elif len(selected) > 1:  # nobody left to take pages from: the youngest waits a step
                    victim = max((r for r, _ in selected), key=lambda r: r.admitted)
                else:
                    events.extend(self._fail([oldest], error))
                    self._drop_terminal()
                    return events
                selected = [(r, n) for r, n in selected if r is not victim]
            except Exception as error:  # the whole batch shares one model call
                events.extend(self._fail([r for r, _ in selected], error))
                self._drop_terminal()
                return events
        for request, token in zip(wanted, tokens):
            events.extend(self._consume(request, token))
        self._drop_terminal()
        return events

    def run_until_idle(self) -> list[StreamEvent]:
        events: list[StreamEvent] = []
        while not self.idle:
            produced = self.step()
            events.extend(produced)
            # a step that only read the tokens in flight (the last request ended on one of them) ran
            # no batch and may emit nothing: that is the end of the work, not a lack of progress
            if not self._last_batch and not produced and not self.idle:
                raise RuntimeError("scheduler made no progress")
        return events

    def run(self, prompts: Sequence, sampling_params: SamplingParams | None = None) -> list[RequestView]:
        """Run the prompts to completion, admitting each as the request limit and the pages allow
        (a prompt that can never be admitted raises ``OverloadedError`` once nothing else is
        running), and return every request's last view, in the order of the prompts.  The requests
        are forgotten."""
        pending = deque(enumerate(prompts))
        ids: dict[int, str] = {}
        while pending or not self.idle:
            while pending:
                index, prompt = pending[0]
                try:
                    ids[index] = self.submit(prompt, sampling_params=sampling_params)
                except OverloadedError:
                    if self.idle:
                        raise
                    break
                pending.popleft()
            produced = self.step()
            if not self._last_batch and not produced and not self.idle:
                raise RuntimeError("scheduler made no progress")
        views = [self.request(ids[index]) for index in range(len(prompts))]
        for index in range(len(prompts)):
            self.forget(ids[index])
        return views

    def generate(self, prompts: Sequence, sampling_params: SamplingParams | None = None) -> list[list[int]]:
        """Run the prompts to completion (admitting them as room allows) and
        return each one's generated token ids."""
        views = self.run(prompts, sampling_params)
        for view in views:
            if view.status is RequestStatus.FAILED:
                raise RuntimeError(f"request {view.request_id} failed: {view.error}")
        return [list(view.output_token_ids) for view in views]

    # -------------------------------------------------------------- results
    def _consume(self, request: _Request, token: int) -> list[StreamEvent]:
        """Order of the reference (scheduler.py:472-519): count the token; end
        of sequence finishes with "stop" and is not emitted; else the token is
        emitted, a stop string finishes with "stop", the token limit with
        "length".  The last sampled token is never fed to the model."""
        request.status = RequestStatus.RUNNING
        request.sampled_tokens += 1
        fragments: list[str] = []
        emitted: tuple[int, ...] = ()
        reached_eos = token in request.eos_ids
        finish = reached_eos
        stopped = False
        if not reached_eos:
            request.outputs.append(token)
            emitted = (token,)
            if request.detokenizer is not None:
                fragment = request.detokenizer.push(token)
                if fragment:
                    fragments.append(fragment)
                stopped = request.detokenizer.stopped
            finish = stopped
        reached_limit = request.sampled_tokens >= request.params.max_new_tokens
        finish = finish or reached_limit
        if finish:
            if request.detokenizer is not None:
                tail = request.detokenizer.finish()
                if tail:
                    fragments.append(tail)
            request.status = RequestStatus.FINISHED
            request.finish_reason = "stop" if reached_eos or stopped else "length"
            self._cleanup(request)
        text = "".join(fragments)
        request.text += text
        if emitted or text or request.status.terminal:
            return [StreamEvent(request.request_id, text, request.status, emitted)]
        return []

    def _fail(self, requests: list[_Request], error: Exception) -> list[StreamEvent]:
        events = []
        for request in requests:
            request.status = RequestStatus.FAILED
            request.finish_reason = "error"
            request.error = f"{type(error).__name__}: {error}"
            self._cleanup(request)
            events.append(StreamEvent(request.request_id, "", request.status))
        return events

    def _fail_batch(self, requests: list[_Request], error: Exception) -> list[StreamEvent]:
        """A model call or a sampling call failed: every live request of its batch fails."""
        for request in requests:
            request.in_flight = False
        events = self._fail([r for r in requests if not r.status.terminal], error)
        self._drop_terminal()
        return events

    def _cleanup(self, request: _Request) -> None:
        """Pages, state slot and reservation go back exactly once."""
        if request.holds_cache:
            self._runner.end(request.request_id)
            request.holds_cache = False
        if not request.reservation_released:
            self._reserved = [taken - held for taken, held in zip(self._reserved, request.reserved_blocks)]
            request.reservation_released = True

    def _drop_terminal(self) -> None:
        self._order = deque(i for i in self._order if not self._requests[i].status.terminal)

    # ---------------------------------------------------------------- views
    def request(self, request_id: str) -> RequestView:
        r = self._request(request_id)
        return RequestView(r.request_id, r.status, len(r.prompt), r.sampled_tokens,
                           0 if r.reservation_released else max(r.reserved_blocks, default=0), r.finish_reason, r.error,
                           tuple(r.outputs), r.text)

    def forget(self, request_id: str) -> None:
        request = self._request(request_id)
        if not request.status.terminal:
            raise ValueError("cannot forget an active request")
        self._order = deque(i for i in self._order if i != request_id)
        del self._requests[request_id]

    def snapshot(self) -> SchedulerSnapshot:
        requests = list(self._requests.values())
        return SchedulerSnapshot(
            iteration=self._iteration,
            waiting=sum(r.status is RequestStatus.WAITING for r in requests),
            running=sum(r.status is RequestStatus.RUNNING for r in requests),
            terminal=sum(r.status.terminal for r in requests),
            reserved_blocks=max(self._reserved, default=0),
            allocated_blocks=self._runner.cache.allocated_pages,
            last_batch=self._last_batch,
            model_batches=(self._last_batch,) if self._last_batch else (),
            last_batch_tokens=self._last_tokens,
            preemptions=self._preemptions,
        )

    def _request(self, request_id: str) -> _Request:
        try:
            return self._requests[request_id]
        except KeyError:
            raise KeyError(f"unknown request_id: {request_id}") from None

    def _new_id(self) -> str:
        while True:
            candidate = f"req-{self._next_number}"
            self._next_number += 1
            if candidate not in self._requests:
                return candidate
