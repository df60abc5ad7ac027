"""The scheduler's decisions, on the CPU with the kernels' plain references
patched in: admission and reservation, round-robin order, portions under the
token budget, mixed batches, finishing, cancelling, failures, and both answers
to "the pages ran out"."""

from __future__ import annotations

import pytest
import torch

import kernel_refs
import plain_qwen3 as plain
from conftest import TINY
from forge_engine_amd.config import SchedulerConfig, load_model_config
from forge_engine_amd.engine import (ConcurrentGenerationEngine, GenerationEngine, IncrementalDetokenizer, ModelRunner,
                                     OverloadedError, RequestStatus, StepEntry, build_engine, load_model)
from forge_engine_amd.sampling import SamplingParams
from forge_engine_amd.sampling.sampler import Sampler
from forge_engine_amd.weights import write_random_model
from safetensors.torch import load_file


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    path = tmp_path_factory.mktemp("sched_model")
    write_random_model(load_model_config(TINY["A"]), 5, path)
    return path


@pytest.fixture()
def make(folder, monkeypatch):
    kernel_refs.install(monkeypatch)

    def build(**limits) -> ConcurrentGenerationEngine:
        _, model = load_model(folder, dtype="float32", device="cpu")
        eos = limits.pop("eos", ())
        config = SchedulerConfig(**{"block_size": 2, "block_capacity": 64, **limits})
        return build_engine(model, scheduler_config=config, eos_token_ids=eos)
    return build


def params(n=3, **kw):
    return SamplingParams(max_new_tokens=n, **kw)


def plain_greedy(folder, prompt, n):
    weights = {k: v.float() for k, v in load_file(str(folder / "model.safetensors")).items()}
    return plain.greedy_generate(weights, TINY["A"], prompt, n)


def test_reservation_is_worst_case_and_overload_comes_before_any_page(make):
    # 3 prompt tokens + 3 new tokens at block size 2 reserve 3 pages (reference tests/test_scheduler.py:125-143)
    engine = make(block_capacity=5)
    first = engine.submit([1, 2, 3], sampling_params=params(3))
    assert engine.request(first).reserved_blocks == 3
    with pytest.raises(OverloadedError, match="only 2 are unreserved"):
        engine.submit([4, 5, 6], sampling_params=params(3))
    assert engine.cache_pool.allocated_pages == 0 and len(engine.cache_pool.live_requests()) == 1
    with pytest.raises(OverloadedError, match="pool capacity"):
        engine.submit([1] * 20, sampling_params=params(3))
    engine.run_until_idle()
    assert engine.snapshot().reserved_blocks == 0 and engine.cache_pool.allocated_pages == 0
    assert engine.request(first).reserved_blocks == 0
    engine.submit([4, 5, 6], sampling_params=params(3))       # room again


def test_request_limit_duplicates_and_bad_prompts(make):
    engine = make(max_requests=1)
    engine.submit([1, 2], request_id="x", sampling_params=params(1))
    with pytest.raises(OverloadedError, match="request limit"):
        engine.submit([3], sampling_params=params(1))
    engine.run_until_idle()
    with pytest.raises(ValueError, match="duplicate"):
        engine.submit([3], request_id="x", sampling_params=params(1))
    with pytest.raises(ValueError, match="non-empty"):
        engine.submit([], sampling_params=params(1))
    with pytest.raises(ValueError, match="vocabulary"):
        engine.submit([256], sampling_params=params(1))
    with pytest.raises(ValueError, match="tokenizer"):
        engine.submit("text", sampling_params=params(1))


def test_round_robin_order(make):
    # a, b, c, then a again (reference tests/test_scheduler.py:235-250)
    engine = make(max_batch_size=1)
    for name in "abc":
        engine.submit([1, 2, 3], request_id=name, sampling_params=params(2))
    seen = []
    for _ in range(4):
        engine.step()
        seen.extend(engine.snapshot().last_batch)
    assert seen == ["a", "b", "c", "a"]


def test_late_joiner_shares_the_batch_with_a_decoding_request(make):
    engine = make()
    engine.submit([1, 2, 3], request_id="early", sampling_params=params(4))
    engine.step()
    assert engine.request("early").status is RequestStatus.RUNNING
    engine.submit([9, 8, 7, 6, 5], request_id="late", sampling_params=params(4))
    engine.step()
    snap = engine.snapshot()
    assert snap.last_batch == ("early", "late") and snap.last_batch_tokens == (1, 5)
    assert snap.model_batches == (("early", "late"),)          # one model call for the decode token and the prompt
    assert snap.running == 2 and snap.waiting == 0


def test_token_budget_cuts_prompts_into_portions(make):
    engine = make(token_budget=8, max_batch_size=4)
    engine.submit(list(range(1, 21)), request_id="long", sampling_params=params(2))
    engine.submit([5, 6, 7], request_id="short", sampling_params=params(2))
    engine.step()
    assert engine.snapshot().last_batch_tokens == (8,)         # the budget is spent on the first prompt
    assert engine.request("long").status is RequestStatus.WAITING
    engine.step()                                              # round-robin: short first, long gets the rest
    assert engine.snapshot().last_batch == ("short", "long") and engine.snapshot().last_batch_tokens == (3, 5)
    engine.step()                                              # short decodes (1) beside the last 7 of long
    assert engine.snapshot().last_batch_tokens == (1, 7)
    assert engine.request("long").status is RequestStatus.RUNNING and engine.request("long").sampled_tokens == 1
    engine.run_until_idle()
    assert engine.request("long").finish_reason == "length"


def test_prefill_chunk_bounds_each_portion(make):
    engine = make(prefill_chunk=4)
    engine.submit(list(range(1, 12)), request_id="p", sampling_params=params(1))
    sizes = []
    while not engine.idle:
        engine.step()
        sizes.extend(engine.snapshot().last_batch_tokens)
    assert sizes == [4, 4, 3]


def test_greedy_generation_equals_plain_under_any_cut(make, folder):
    prompts = {"a": [5, 17, 3, 200, 9], "b": list(range(30, 41)), "c": list(range(100, 117))}
    want = {k: plain_greedy(folder, p, 8) for k, p in prompts.items()}
    for limits in ({}, {"token_budget": 7, "block_size": 4}, {"prefill_chunk": 3, "max_batch_size": 2}):
        engine = make(**limits)
        for name, prompt in prompts.items():
            engine.submit(prompt, request_id=name, sampling_params=params(8))
        engine.run_until_idle()
        for name in prompts:
            view = engine.request(name)
            assert list(view.output_token_ids) == want[name], (limits, name)
            assert view.status is RequestStatus.FINISHED and view.finish_reason == "length"
        assert engine.cache_pool.allocated_pages == 0


def test_generate_admits_as_room_allows(make, folder):
    engine = make(block_capacity=8, max_requests=2)
    prompts = [[5, 17, 3], [9, 9, 9, 9], [1, 2], [7]]
    got = engine.generate(prompts, params(4))
    assert got == [plain_greedy(folder, p, 4) for p in prompts]
    assert engine.snapshot().reserved_blocks == 0


def test_end_of_sequence_is_not_emitted_and_finishes_with_stop(make, folder):
    sampled = params(12, temperature=1.0, seed=5)
    probe = make()
    probe.submit([5, 17, 3], request_id="e", sampling_params=sampled)
    probe.run_until_idle()
    tokens = list(probe.request("e").output_token_ids)
    at = next(i for i in range(1, 12) if tokens[i] not in tokens[:i])   # first token not seen before
    engine = make(eos=(tokens[at],))
    engine.submit([5, 17, 3], request_id="e", sampling_params=sampled)
    events = engine.run_until_idle()
    view = engine.request("e")
    assert view.finish_reason == "stop" and view.sampled_tokens == at + 1
    assert list(view.output_token_ids) == tokens[:at]
    assert [e.token_ids for e in events] == [(t,) for t in tokens[:at]] + [()]
    assert events[-1].status is RequestStatus.FINISHED


def test_the_last_sampled_token_is_never_fed(make):
    engine = make()
    engine.submit([1, 2, 3], request_id="x", sampling_params=params(3))
    engine.run_until_idle()
    assert engine._runner.steps_run == 3      # prefill + 2 decodes for 3 tokens


def test_cancel_and_forget(make):
    engine = make()
    engine.submit([1, 2, 3, 4, 5], request_id="c", sampling_params=params(5))
    engine.step()
    assert engine.cache_pool.allocated_pages > 0
    assert engine.cancel("c") is True and engine.cancel("c") is False
    assert engine.request("c").status is RequestStatus.CANCELLED
    assert engine.cache_pool.allocated_pages == 0 and engine.snapshot().reserved_blocks == 0
    engine.submit([1], request_id="live", sampling_params=params(2))
    with pytest.raises(ValueError, match="active"):
        engine.forget("live")
    engine.forget("c")
    with pytest.raises(KeyError):
        engine.request("c")
    assert engine.idle is False


def test_a_failing_model_call_fails_its_batch_and_frees_everything(make, monkeypatch):
    engine = make()
    engine.submit([1, 2, 3], request_id="a", sampling_params=params(4))
    engine.submit([4, 5], request_id="b", sampling_params=params(4))
    engine.step()
    calls = {"n": 0}
    real = engine._runner.model.forward

    def broken(batch, views):
        calls["n"] += 1
        raise RuntimeError("device lost")
    monkeypatch.setattr(engine._runner.model, "forward", broken)
    events = engine.step()
    assert {e.request_id for e in events} == {"a", "b"} and all(e.status is RequestStatus.FAILED for e in events)
    assert engine.request("a").error == "RuntimeError: device lost"
    assert engine.cache_pool.allocated_pages == 0 and engine.snapshot().reserved_blocks == 0 and engine.idle
    monkeypatch.setattr(engine._runner.model, "forward", real)
    engine.submit([7, 7], request_id="after", sampling_params=params(2))
    engine.run_until_idle()
    assert engine.request("after").status is RequestStatus.FINISHED


def test_preemption_when_pages_run_out(make, folder):
    prompts = {"old": list(range(1, 9)), "young": list(range(20, 28))}
    want = {k: plain_greedy(folder, p, 10) for k, p in prompts.items()}
    # each request ends with 18 tokens = 9 pages of 2; 12 pages cannot hold both
    engine = make(admission="preempt", block_capacity=12)
    for name, prompt in prompts.items():
        engine.submit(prompt, request_id=name, sampling_params=params(10))
    assert engine.snapshot().reserved_blocks == 0
    engine.run_until_idle()
    assert engine.snapshot().preemptions >= 1
    for name in prompts:
        assert list(engine.request(name).output_token_ids) == want[name]
        assert engine.request(name).status is RequestStatus.FINISHED
    assert engine.cache_pool.allocated_pages == 0
    # under reservation the second request is simply not admitted
    engine = make(block_capacity=12)
    engine.submit(prompts["old"], sampling_params=params(10))
    with pytest.raises(OverloadedError):
        engine.submit(prompts["young"], sampling_params=params(10))


def test_preempted_sampling_continues_the_same_random_stream(make):
    outputs = []
    for capacity in (64, 12):
        engine = make(admission="preempt", block_capacity=capacity)
        for name, prompt in (("old", list(range(1, 9))), ("young", list(range(20, 28)))):
            engine.submit(prompt, request_id=name, sampling_params=params(10, temperature=0.9, seed=77))
        engine.run_until_idle()
        outputs.append([engine.request(n).output_token_ids for n in ("old", "young")])
    assert outputs[0] == outputs[1]


def test_seeded_sampling_repeats_and_seeds_differ(make):
    def run(seed):
        engine = make()
        engine.submit([3, 1, 4, 1, 5], request_id="s", sampling_params=params(12, temperature=1.0, seed=seed))
        engine.run_until_idle()
        return engine.request("s").output_token_ids
    assert run(731) == run(731)
    assert run(731) != run(732)


def test_single_request_engine_streams_and_cleans_up(make, folder):
    engine = GenerationEngine(make())
    want = plain_greedy(folder, [5, 17, 3], 5)
    assert list(engine.stream([5, 17, 3], params(5))) == want
    assert engine.generate([5, 17, 3], params(5)) == want
    stream = engine.stream([5, 17, 3], params(5))
    next(stream)
    stream.close()                       # the consumer stops early: pages go back
    assert engine.engine.cache_pool.allocated_pages == 0 and engine.engine.idle


class DeviceFeedRunner:
    """The CPU runner with the two things that overlapped decoding asks of a runner: it says that
    it can feed a step of single tokens from a device tensor, and does so (here by reading it)."""

    def __init__(self, runner) -> None:
        self._runner = runner
        self.fail_next_step = None

    def __getattr__(self, name):
        return getattr(self._runner, name)

    def feeds_from_device(self, entries) -> bool:
        return all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries)

    def step(self, entries, device_tokens=None):
        if self.fail_next_step is not None:
            error, self.fail_next_step = self.fail_next_step, None
            raise error
        if device_tokens is not None:
            entries = [StepEntry(e.request_id, [int(device_tokens[i])], e.want) for i, e in enumerate(entries)]
        return self._runner.step(entries)


@pytest.fixture()
def make_overlapped(folder, monkeypatch):
    kernel_refs.install(monkeypatch)

    def build(**limits) -> ConcurrentGenerationEngine:
        _, model = load_model(folder, dtype="float32", device="cpu")
        eos = limits.pop("eos", ())
        config = SchedulerConfig(**{"block_size": 2, "block_capacity": 64, **limits})
        runner = DeviceFeedRunner(ModelRunner(model, block_size=config.block_size, block_capacity=config.block_capacity,
                                              num_state_slots=config.max_requests))
        return ConcurrentGenerationEngine(runner, Sampler(model.ctx.device), SamplingParams(), config, eos_token_ids=eos)
    return build


def test_overlapped_decoding_ends_cleanly_when_the_last_request_stops_on_its_end_token(make_overlapped, folder):
    # the request's end token is read a step late, while the request rides in a step already launched:
    # the step after that only reads that step's tokens, runs no batch and emits nothing, and is the end
    sampled = params(12, temperature=1.0, seed=5)
    probe = make_overlapped(overlap_decode=False)
    tokens = probe.generate([[5, 17, 3]], sampled)[0]
    at = next(i for i in range(2, 12) if tokens[i] not in tokens[:i])   # first token not seen before
    engine = make_overlapped(eos=(tokens[at],))
    engine.submit([5, 17, 3], request_id="e", sampling_params=sampled)
    events = engine.run_until_idle()
    view = engine.request("e")
    assert engine.overlapped_steps >= at - 1 and engine.idle
    assert view.status is RequestStatus.FINISHED and view.finish_reason == "stop"
    assert list(view.output_token_ids) == tokens[:at] and view.sampled_tokens == at + 1
    assert [e.token_ids for e in events] == [(t,) for t in tokens[:at]] + [()]
    assert engine.cache_pool.allocated_pages == 0 and engine.snapshot().reserved_blocks == 0
    assert engine.generate([[5, 17, 3]], sampled) == [tokens[:at]]     # and through generate


def test_overlapped_decoding_serves_requests_in_the_same_order(make_overlapped, make, folder):
    # more live requests than a step takes: a selection that could not be overlapped is made again
    # from the queue as it stood, so nobody loses a turn and the batches are those of the plain scheduler
    prompts = {name: [3 + i, 40 + i, 9] for i, name in enumerate("abcde")}
    batches = {}
    for overlap, build in ((True, make_overlapped), (False, make)):
        engine = build(max_batch_size=2, overlap_decode=overlap)
        for name, prompt in prompts.items():
            engine.submit(prompt, request_id=name, sampling_params=params(4))
        seen = []
        while not engine.idle:
            engine.step()
            seen.append(engine.snapshot().last_batch)
        batches[overlap] = [b for b in seen if b]
        for name, prompt in prompts.items():
            assert list(engine.request(name).output_token_ids) == plain_greedy(folder, prompt, 4)
    assert batches[True] == batches[False]


def test_a_failure_after_an_overlapped_step_has_run_fails_the_batch(make_overlapped, monkeypatch):
    # the step ran and moved the cache on; if sampling then fails, feeding the same tokens again would
    # put them one position late: the batch fails instead, and everything is given back
    engine = make_overlapped()
    engine.submit([1, 2, 3], request_id="a", sampling_params=params(8))
    engine.submit([4, 5], request_id="b", sampling_params=params(8))
    engine.step()
    engine.step()
    assert engine.overlapped_steps == 1

    def broken(*args, **kwargs):
        raise RuntimeError("sampling kernel failed")
    monkeypatch.setattr(engine._sampler, "sample_on_device", broken)
    events = engine.step()
    assert all(engine.request(n).status is RequestStatus.FAILED for n in "ab")
    assert engine.request("a").error == "RuntimeError: sampling kernel failed"
    assert [e.status for e in events if e.status is RequestStatus.FAILED] == [RequestStatus.FAILED] * 2
    assert engine.cache_pool.allocated_pages == 0 and engine.snapshot().reserved_blocks == 0 and engine.idle
    # a model call that fails is not retried on the plain path either
    engine = make_overlapped()
    engine.submit([1, 2, 3], request_id="a", sampling_params=params(8))
    engine.step()
    engine.step()
    engine._runner.fail_next_step = RuntimeError("device lost")
    engine.step()
    assert engine.request("a").error == "RuntimeError: device lost" and engine.idle
    assert engine._runner.steps_run == 2 and engine.cache_pool.allocated_pages == 0


class WordTokenizer:
    WORDS = {1: "one ", 2: "two ", 3: "STOP", 4: "�", 5: "é"}

    def decode(self, ids, skip_special_tokens=True):
        text = "".join(self.WORDS.get(i, f"<{i}>") for i in ids)
        return text.replace("�é", "è")


def test_detokenizer_holds_back_stop_prefixes_and_half_characters():
    # behaviour of the reference's detokenizer (tests/test_generation_core.py:139-174 there)
    d = IncrementalDetokenizer(WordTokenizer(), ("o STOP",))
    assert d.push(1) == "one "
    assert d.push(2) == "tw"               # the tail "o " could grow into "o STOP" and is held
    assert d.push(3) == "" and d.stopped   # "two STOP" completes the stop string
    assert d.finish() == ""
    with pytest.raises(RuntimeError):
        d.push(1)
    d = IncrementalDetokenizer(WordTokenizer())
    assert d.push(4) == ""                 # half a character waits
    assert d.push(5) == "è"
    d = IncrementalDetokenizer(WordTokenizer(), ("two STOP",))
    assert d.push(2) == "" and d.finish() == "two "   # a stop prefix is flushed when generation ends


def test_a_requests_token_inputs_follow_its_tokens():
    """Per-token inputs that came with a prompt are cut as the prompt is: a portion gets its rows; tokens
    past the prompt (sampled ones, fed again after a preemption or for the first time) bring their
    position on every axis, at the width of the prompt's rows."""
    from forge_engine_amd.engine.scheduler import _Request
    request = _Request("r", [5, 6, 7, 8], SamplingParams(max_new_tokens=4), 1, frozenset(), None, [0], 1,
                       inputs={"grid": [[9, 1], [9, 2], [9, 3], [9, 4]], "kind": [7, 7, 8, 8]})
    assert request.next_inputs(3) == {"grid": [[9, 1], [9, 2], [9, 3]], "kind": [7, 7, 8]}
    request.fed = 3
    request.outputs = [11, 12]
    assert request.next_tokens(3) == [8, 11, 12]
    assert request.next_inputs(3) == {"grid": [[9, 4], [4, 4], [5, 5]], "kind": [8, [4], [5]]}
    request.fed = 5
    assert request.next_inputs(1) == {"grid": [[5, 5]], "kind": [[5]]}
    request.inputs = None
    assert request.next_inputs(2) is None
