"""The engine on the GPU: generation through the entry points, long decoding
through captured graphs, the first tokens of a sequence, each part alone, and a
toy architecture (a mixer with state of its own, a windowed mixer, a layer run
twice, a layer reading another's cache) registered from here."""

from __future__ import annotations

import json
from dataclasses import dataclass
from typing import ClassVar

import pytest
import torch
from safetensors.torch import load_file

import plain_qwen3 as plain
import replay_util as ru
from conftest import BLOCK_SIZE, TINY
from forge_engine_amd.cache import CacheNeeds, FixedState
from forge_engine_amd.config import EngineConfig, SchedulerConfig, load_model_config
from forge_engine_amd.config.model import KeyReader, ModelConfig
from forge_engine_amd.engine import (GenerationEngine, ModelRunner, StepEntry, build_model,
                                     engine_from_folder, load_model)
from forge_engine_amd.engine.api import build_engine
from forge_engine_amd.parts import (BuildContext, LayerCall, LayerSpec, Mixer, ModelPlan, ParamSpec, PartSpec,
                                    Residual, build_part)
from forge_engine_amd.parts.base import Block, Embedding, FeedForward, Head, Norm
from forge_engine_amd.registry import register_architecture, register_part
from forge_engine_amd.sampling import SamplingParams
from forge_engine_amd.weights import fill_random_weights, write_random_model

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}
    for name in TINY:
        folder = tmp_path_factory.mktemp(f"engine_{name}")
        write_random_model(load_model_config(TINY[name]), 31, folder)
        made[name] = folder
    return made


def folder_weights(folder):
    return {k: v.float() for k, v in load_file(str(folder / "model.safetensors")).items()}


def check_choice(weights, config, prompt, tokens, dtype):
    """Each generated token must be the plain implementation's argmax, or (bfloat16)
    within the rounding bound of it."""
    ids = list(prompt)
    for token in tokens:
        logits = plain.forward(weights, config, ids)[-1]
        if dtype == "float32":
            assert token == int(logits.argmax()), f"token {token} after {len(ids)} ids"
        else:
            assert float(logits.max() - logits[token]) <= ru.BF16_FRACTION * float(logits.abs().max())
        ids.append(token)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_through_the_entry_point(name, dtype, folders):
    config, weights = TINY[name], folder_weights(folders[name])
    prompts = list(ru.make_requests(config, 8, (5, 11, 17)).values())
    scheduler = SchedulerConfig(block_size=BLOCK_SIZE[name], block_capacity=64, token_budget=16, max_batch_size=4)
    engine = engine_from_folder(folders[name], engine_config=EngineConfig(max_new_tokens=8),
                                scheduler_config=scheduler, dtype=dtype)
    outputs = engine.generate(prompts)
    assert engine.cache_pool.allocated_pages == 0
    for prompt, tokens in zip(prompts, outputs):
        assert len(tokens) == 8
        check_choice(weights, config, prompt, tokens, dtype)
    single = GenerationEngine(engine)
    assert single.generate(prompts[0]) == outputs[0]          # alone or batched: the same tokens
    assert list(single.stream(prompts[1])) == outputs[1]


@pytest.mark.parametrize("name", ["B", "C"])
def test_scheduler_under_page_pressure_on_the_gpu(name, folders):
    """Twelve requests of random lengths through the scheduler with too few pages for all of them
    (requests are preempted and recomputed), portions of prompts beside decoded tokens, decode and
    portion graphs: in float32 every request generates what it generates alone in the plain
    implementation, and every page comes back."""
    import random
    config, weights = TINY[name], folder_weights(folders[name])
    rng = random.Random(51)
    lengths = [rng.randrange(3, 40) for _ in range(12)]
    prompts = list(ru.make_requests(config, 52, lengths).values())
    new_tokens = [rng.randrange(4, 14) for _ in prompts]
    block = BLOCK_SIZE[name]
    capacity = 3 * (-(-(max(lengths) + 14) // block)) + 2        # room for about three requests
    scheduler = SchedulerConfig(block_size=block, block_capacity=capacity, token_budget=24, max_batch_size=6,
                                max_requests=16, prefill_chunk=16, admission="preempt")
    engine = engine_from_folder(folders[name], scheduler_config=scheduler, dtype="float32")
    ids = [engine.submit(p, sampling_params=SamplingParams(max_new_tokens=n)) for p, n in zip(prompts, new_tokens)]
    engine.run_until_idle()
    assert engine.snapshot().preemptions >= 1
    assert engine.cache_pool.allocated_pages == 0
    for request_id, prompt, n in zip(ids, prompts, new_tokens):
        got = list(engine.request(request_id).output_token_ids)
        assert got == plain.greedy_generate(weights, config, prompt, n), request_id


@pytest.mark.parametrize("sampled", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_overlapped_decode_steps_generate_the_same_tokens(dtype, sampled, folders):
    """Steady decode steps (greedy, or drawn with temperature, top-k and top-p from seeded
    generators) take their tokens on the device and the host reads a step late:
    the same tokens, finish reasons and freed pages as with every step read back at once; with
    requests that end on an end-of-sequence token (seen a step late), on their token limit (known
    in advance), a request cancelled while its token is in flight, and a late joiner."""
    def sampling(limit, seed):
        if sampled:
            return SamplingParams(temperature=0.9, top_k=20, top_p=0.95, seed=seed, max_new_tokens=limit)
        return SamplingParams(max_new_tokens=limit)
    name = "B"          # a head of its own: greedy tokens vary instead of falling into a loop at once
    config = TINY[name]
    prompts = list(ru.make_requests(config, 87, (12, 30, 7, 19, 25)).values())
    limits = [9, 40, 40, 23, 31]
    results = {}
    for overlap in (False, True):
        scheduler = SchedulerConfig(block_size=8, block_capacity=64, token_budget=64, max_batch_size=8,
                                    overlap_decode=overlap)
        engine = engine_from_folder(folders[name], scheduler_config=scheduler, dtype=dtype)
        if not overlap:
            # choose an end-of-sequence token that the second request really samples, a few tokens in
            probe = engine.generate([prompts[1]], sampling(24, 101))[0]
            at = next(j for j in range(3, len(probe)) if probe[j] not in probe[:j])    # first seen at place j >= 3
            results["eos"], results["stop_after"] = probe[at], at
        engine = engine_from_folder(folders[name], scheduler_config=scheduler, dtype=dtype, eos_token_ids=[results["eos"]])
        ids = [engine.submit(p, sampling_params=sampling(n, 100 + i)) for i, (p, n) in enumerate(zip(prompts[:4], limits[:4]))]
        steps = 0
        while not engine.idle:
            engine.step()
            steps += 1
            if steps == 6:
                ids.append(engine.submit(prompts[4], sampling_params=sampling(limits[4], 104)))   # joins late
            if steps == 12:
                engine.cancel(ids[2])
        views = [engine.request(i) for i in ids]
        results[overlap] = [(v.status.value, v.finish_reason, v.output_token_ids if i != 2 else None) for i, v in enumerate(views)]
        assert engine.cache_pool.allocated_pages == 0
        assert (engine.overlapped_steps > 8) == overlap
        assert views[1].finish_reason == "stop" and len(views[1].output_token_ids) == results["stop_after"]   # the end token is not emitted
        assert views[0].finish_reason == "length" and len(views[0].output_token_ids) == 9
        assert views[2].status.value == "cancelled"
    assert results[True] == results[False]


def test_command_line_generates(folders, capsys):
    from forge_engine_amd.cli import main
    prompt = [5, 17, 3, 200, 9]
    code = main(["generate", "--model", str(folders["A"]), "--dtype", "float32", "--prompt-ids",
                 ",".join(map(str, prompt)), "--prompt-ids", "7,7", "--max-new-tokens", "5", "--block-size", "4"])
    assert code == 0
    records = [json.loads(line) for line in capsys.readouterr().out.strip().splitlines()]
    assert [r["prompt"] for r in records] == [0, 1] and all(r["finish_reason"] == "length" for r in records)
    check_choice(folder_weights(folders["A"]), TINY["A"], prompt, records[0]["token_ids"], "float32")


def test_a_lone_request_that_ends_on_its_end_token_while_decoding_overlapped(folders, tmp_path, capsys):
    """The last running request samples its end-of-sequence token during overlapped decoding: it
    still rides in the step already launched, the step after that only reads that step's tokens,
    and the run ends there, through ``run_until_idle`` and through the command line (whose model
    folder names the end token in config.json; more prompts than ``--max-requests`` wait their turn)."""
    from forge_engine_amd.cli import main
    name = "B"
    prompt = ru.make_requests(TINY[name], 87, (12, 30))["r1"]
    scheduler = SchedulerConfig(block_size=8, block_capacity=64)
    probe = engine_from_folder(folders[name], scheduler_config=scheduler, dtype="float32", eos_token_ids=[])
    tokens = probe.generate([prompt], SamplingParams(max_new_tokens=24))[0]
    at = next(j for j in range(3, len(tokens)) if tokens[j] not in tokens[:j])
    engine = engine_from_folder(folders[name], scheduler_config=scheduler, dtype="float32", eos_token_ids=[tokens[at]])
    request_id = engine.submit(prompt, sampling_params=SamplingParams(max_new_tokens=24))
    engine.run_until_idle()
    view = engine.request(request_id)
    assert engine.overlapped_steps >= at - 1 and engine.idle and engine.cache_pool.allocated_pages == 0
    assert view.finish_reason == "stop" and list(view.output_token_ids) == tokens[:at]
    # the command line: a folder whose config.json names that end token, three prompts through two request places
    folder = tmp_path / "with_eos"
    folder.mkdir()
    (folder / "model.safetensors").symlink_to(folders[name] / "model.safetensors")
    (folder / "config.json").write_text(json.dumps({**TINY[name], "eos_token_id": tokens[at]}))
    ids = ",".join(map(str, prompt))
    code = main(["generate", "--model", str(folder), "--dtype", "float32", "--prompt-ids", ids, "--prompt-ids", "7,7,9",
                 "--prompt-ids", ids, "--max-new-tokens", "24", "--block-size", "8", "--max-requests", "2"])
    assert code == 0
    records = [json.loads(line) for line in capsys.readouterr().out.strip().splitlines()]
    assert [r["prompt"] for r in records] == [0, 1, 2]
    assert records[0]["finish_reason"] == "stop" and records[0]["token_ids"] == tokens[:at]
    assert records[2] == {**records[0], "prompt": 2}


def test_temperature_sampling_is_seeded_and_batch_independent(folders):
    scheduler = SchedulerConfig(block_size=8, block_capacity=64)
    engine = engine_from_folder(folders["B"], scheduler_config=scheduler, dtype="float32")
    params = SamplingParams(temperature=0.8, seed=1234, max_new_tokens=12)
    prompts = list(ru.make_requests(TINY["B"], 2, (1, 7, 23, 40)).values())
    together = engine.generate(prompts, params)
    alone = [engine.generate([p], params)[0] for p in prompts]
    assert together == alone
    assert engine.generate(prompts[:1], SamplingParams(temperature=0.8, seed=99, max_new_tokens=12))[0] != alone[0]
    filtered = SamplingParams(temperature=0.9, top_k=3, top_p=0.9, min_p=0.05, seed=5, max_new_tokens=6)
    top = engine.generate(prompts[:2], filtered)
    assert all(len(t) == 6 for t in top)
    assert engine.generate(prompts[:2], filtered) == top
    # every drawn token is one that the plain filters leave (sampling.py:83-140 of the reference)
    weights = folder_weights(folders["B"])
    kept_sizes = []
    for prompt, tokens in zip(prompts[:2], top):
        ids = list(prompt)
        for token in tokens:
            logits = plain.forward(weights, TINY["B"], ids)[-1]
            left = plain.filter_logits(logits[None], 0.9, top_k=3, top_p=0.9, min_p=0.05)[0]
            assert torch.isfinite(left[token]), f"token {token} after {len(ids)} ids was filtered out"
            kept_sizes.append(int(torch.isfinite(left).sum()))
            ids.append(token)
    assert max(kept_sizes) <= 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_graphs_matches_eager_and_plain(dtype, folders):
    """300 decode steps: replays of captured graphs, with eager steps of another
    request between them, against the eager engine and the plain implementation."""
    name = "C"
    config, weights = TINY[name], folder_weights(folders[name])
    tokens = ru.make_requests(config, 13, (340,))["r0"]
    other = ru.make_requests(config, 14, (90,))["r0"]
    _, model = load_model(folders[name], dtype=dtype, device=DEV)
    runs = {}
    for graphs in (True, False):
        runner = ModelRunner(model, block_size=16, block_capacity=40, num_state_slots=4, use_graphs=graphs)
        runner.begin("a")
        runner.begin("b")
        rows = [runner.step([StepEntry("a", tokens[:40], [39])])[0].clone()]
        fed_other = 0
        for i in range(40, 340):
            rows.append(runner.step([StepEntry("a", [tokens[i]], [0])])[0].clone())
            if i % 25 == 0 and fed_other < len(other):      # eager work between the replays
                runner.step([StepEntry("b", other[fed_other:fed_other + 9], [])])
                fed_other += 9
        runs[graphs] = torch.stack(rows).cpu()
        assert (runner.graph_replays > 250) == graphs
        # most replays take the short way (same request, room in its last page); a new page every 16
        # tokens and the other request's steps make the step look again
        assert (runner.steady_steps > 200) == graphs and (not graphs or runner.steady_steps < runner.graph_replays - 15)
        runner.end("a")
        runner.end("b")
        assert runner.cache.allocated_pages == 0
    want = plain.forward(weights, config, tokens)[39:]
    scale = float(want.abs().max())
    bound = 1e-4 * scale if dtype == "float32" else ru.BF16_FRACTION * scale
    assert float((runs[True] - want).abs().max()) <= bound
    assert float((runs[False] - want).abs().max()) <= bound
    assert torch.isfinite(runs[True]).all()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_tokens_fed_on_the_device_decode_like_tokens_from_the_host(dtype, folders):
    """Greedy decoding of three requests where every step takes its tokens from the arg-max of
    the step before without the host in between (it reads them a step late), across page edges
    and a change of the batch: the same tokens and logits as decoding with host tokens."""
    from forge_engine_amd.sampling.sampler import Sampler
    name = "C"
    config = TINY[name]
    prompts = ru.make_requests(config, 83, (21, 9, 30))
    _, model = load_model(folders[name], dtype=dtype, device=DEV)
    sampler = Sampler(DEV)
    outputs = {}
    for mode in ("host", "device"):
        runner = ModelRunner(model, block_size=16, block_capacity=24, num_state_slots=4)
        last = {}
        for k, tokens in prompts.items():
            runner.begin(k)
            last[k] = int(runner.step([StepEntry(k, tokens, [len(tokens) - 1])])[0].argmax())
        names = list(prompts)
        generated = {k: [last[k]] for k in names}
        rows = []
        if mode == "host":
            for step in range(40):
                if step == 25:
                    names = names[:2]                      # one request leaves: another graph, other table rows
                logits = runner.step([StepEntry(k, [generated[k][-1]], [0]) for k in names])
                rows.append(logits.clone())
                for k, t in zip(names, sampler.sample(logits, [SamplingParams()] * len(names), [0] * len(names), [0] * len(names))):
                    generated[k].append(t)
        else:
            feed = torch.tensor([last[k] for k in names], dtype=torch.int32, device=DEV)
            unread = []
            for step in range(40):
                if step == 25:
                    names = names[:2]
                    feed = feed[:2].contiguous()
                entries = [StepEntry(k, [0], [0]) for k in names]
                assert runner.feeds_from_device(entries)
                logits = runner.step(entries, device_tokens=feed)
                rows.append(logits.clone())
                both = sampler.sample_greedy_on_device(logits)
                unread.append((list(names), both))
                feed = both[0]
                if len(unread) > 1:                        # the host reads a step late
                    ks, late = unread.pop(0)
                    for k, t in zip(ks, sampler.read(late)):
                        generated[k].append(t)
            for ks, both in unread:
                for k, t in zip(ks, sampler.read(both)):
                    generated[k].append(t)
            assert runner.graph_replays == 40
            with pytest.raises(ValueError, match="single tokens"):
                runner.step([StepEntry(names[0], [1, 2], [1])], device_tokens=feed)
        outputs[mode] = (generated, torch.cat([r.flatten() for r in rows]).cpu())
        for k in prompts:
            runner.end(k)
    assert outputs["host"][0] == outputs["device"][0]
    assert torch.equal(outputs["host"][1], outputs["device"][1])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_steps_with_portions_replay_captured_graphs(name, dtype, folders):
    """A scheduler that fills its token budget repeats few step shapes; such steps (prompt portions
    beside decoded tokens) are captured on their second sighting and replayed.  Requests come and go
    (pages and sequence slots of the captured shape are reused, padded sequences stay empty), every
    position's logits are wanted and compared with the plain implementation, with and without graphs."""
    config = TINY[name]
    block = BLOCK_SIZE[name]
    requests = ru.make_requests(config, 41, (37, 52, 23, 44, 31, 18))
    want = ru.plain_logits(folders[name], requests)
    _, model = load_model(folders[name], dtype=dtype, device=DEV)
    for graphs in (True, False):
        runner = ModelRunner(model, block_size=block, block_capacity=3 * (60 // block + 2), num_state_slots=3,
                             use_graphs=graphs)
        waiting = list(requests)
        live, at, got = [], {}, {}
        while waiting or live:
            while waiting and len(live) < 3:          # at most three live: pages are used again
                k = waiting.pop(0)
                runner.begin(k)
                live.append(k)
                at[k] = 0
            entries = []
            for k in live:
                tokens = requests[k]
                # portions of 6 tokens; the last 5 tokens of a request come one by one beside them
                size = 6 if at[k] + 6 <= len(tokens) - 5 else (len(tokens) - 5 - at[k] if at[k] < len(tokens) - 5 else 1)
                entries.append(StepEntry(k, tokens[at[k]:at[k] + size], list(range(size))))
            logits = runner.step(entries).cpu()
            row = 0
            for e in entries:
                for i in range(len(e.tokens)):
                    got[(e.request_id, at[e.request_id] + i)] = logits[row + i].clone()
                row += len(e.tokens)
                at[e.request_id] += len(e.tokens)
            for k in [k for k in live if at[k] == len(requests[k])]:
                runner.end(k)
                live.remove(k)
        assert runner.cache.allocated_pages == 0
        runner.cache.check_invariants()
        assert (runner.portion_graph_replays >= 5) == graphs
        ru.compare(got, want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_of_a_hundred_requests_with_portions_replay_captured_graphs(dtype, folders):
    """Steps of more than 64 requests that hold prompt portions beside decoded tokens are captured
    too: 90 requests, ten of which bring portions of 5 tokens in every step while the others bring
    one token each; the same shape comes six times.  The attention kernels then find their work
    among more sequences than a wave has lanes."""
    name = "C"
    config, weights = TINY[name], folder_weights(folders[name])
    count = 90
    lengths = tuple(31 + (3 * i) % 11 if i < 10 else 12 + (7 * i) % 9 for i in range(count))
    requests = ru.make_requests(config, 43, lengths)
    names = list(requests)
    want = {k: plain.forward(weights, config, v) for k, v in requests.items()}
    _, model = load_model(folders[name], dtype=dtype, device=DEV)
    runner = ModelRunner(model, block_size=16, block_capacity=3 * count + 8, num_state_slots=count)
    at = {}
    for first in range(0, count, 45):
        chunk = names[first:first + 45]
        for k in chunk:
            runner.begin(k)
        # everything but the part that the six steps below bring
        runner.step([StepEntry(k, requests[k][:len(requests[k]) - (30 if names.index(k) < 10 else 6)], []) for k in chunk])
        for k in chunk:
            at[k] = len(requests[k]) - (30 if names.index(k) < 10 else 6)
    worst = 0.0
    scale = max(float(w.abs().max()) for w in want.values())
    bound = 1e-4 * scale + 1e-5 if dtype == "float32" else ru.BF16_FRACTION * scale
    for step in range(6):
        entries = []
        for i, k in enumerate(names):
            size = 5 if i < 10 else 1
            entries.append(StepEntry(k, requests[k][at[k]:at[k] + size], list(range(size))))
        logits = runner.step(entries).cpu()
        row = 0
        for e in entries:
            for j in range(len(e.tokens)):
                worst = max(worst, float((logits[row + j] - want[e.request_id][at[e.request_id] + j]).abs().max()))
            row += len(e.tokens)
            at[e.request_id] += len(e.tokens)
    assert runner.portion_graph_replays >= 3
    assert worst <= bound, f"{worst:.3e} > {bound:.3e}"
    for k in names:
        runner.end(k)
    assert runner.cache.allocated_pages == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_first_tokens_of_a_sequence(name, dtype, folders):
    """Position 0 alone, then 1, 2, 3: the shortest contexts, one page, first slots."""
    config = TINY[name]
    requests = ru.make_requests(config, 17, (1, 2, 4))
    trace = ru.TraceBuilder()
    trace.step([(k, v[:1]) for k, v in requests.items()])
    trace.step([(k, v[1:2]) for k, v in requests.items() if len(v) > 1], end=["r0"])
    trace.step([("r2", requests["r2"][2:4])], end=["r1", "r2"])
    import tempfile
    with tempfile.TemporaryDirectory() as out:
        got = ru.run_trace(folders[name], dtype, trace, out, block_size=BLOCK_SIZE[name])
    ru.compare(got, ru.plain_logits(folders[name], requests), dtype)


# ---------------------------------------------------------------- parts alone

def ctx(dtype=torch.float32):
    return BuildContext(DEV, dtype)


def randn(*shape, scale=1.0, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def test_norm_part_alone():
    part = build_part("norm", PartSpec("rms_norm", {"size": 72, "eps": 1e-5}, "n"), ctx())
    assert list(part.param_specs()) == ["n.weight"]
    w = 1 + randn(72, scale=0.1)
    part.set_param("n.weight", w.to(DEV))
    h, update = randn(5, 72, seed=1), randn(5, 72, seed=2)
    residual = Residual(h.to(DEV).clone())
    residual.add(update.to(DEV))
    got = part.forward(residual)
    torch.testing.assert_close(got.cpu(), plain.rms_norm(h + update, w, 1e-5), atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(residual.h.cpu(), h + update)        # the add happened in the stream
    assert residual.pending is None
    rows = torch.tensor([4, 0], dtype=torch.int32, device=DEV)
    torch.testing.assert_close(part.forward(residual, rows=rows).cpu(), plain.rms_norm((h + update)[[4, 0]], w, 1e-5),
                               atol=1e-5, rtol=1e-5)


def test_position_part_alone():
    part = build_part("position", PartSpec("rotary", {"head_dim": 48, "theta": 1e6}), ctx())
    inv_freq, rotary_dim = part.rotary()
    assert rotary_dim == 48
    want = 1.0 / (1e6 ** (torch.arange(0, 48, 2, dtype=torch.float32) / 48))
    assert torch.equal(inv_freq.cpu(), want)                         # bit-equal to the reference's expression
    partial = build_part("position", PartSpec("rotary", {"head_dim": 48, "theta": 1e4, "rotary_dim": 16}), ctx())
    assert partial.rotary()[0].shape == (8,) and partial.rotary()[1] == 16
    assert build_part("position", PartSpec("none"), ctx()).rotary() is None


def test_feed_forward_part_alone():
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        part = build_part("feed_forward", PartSpec("swiglu", {"hidden_size": 40, "intermediate_size": 104}, "m"), ctx(dtype))
        weights = {"m.gate_proj.weight": randn(104, 40, scale=0.2, seed=3), "m.up_proj.weight": randn(104, 40, scale=0.2, seed=4),
                   "m.down_proj.weight": randn(40, 104, scale=0.2, seed=5)}
        weights = {k: v.to(dtype) for k, v in weights.items()}
        for k, v in weights.items():
            part.set_param(k, v.to(DEV))
        x = randn(70, 40, seed=6).to(dtype)          # more than 64 rows: the library product; fewer: the streaming one
        want = plain.swiglu_mlp(x.float(), {k: v.float() for k, v in weights.items()}, "m")
        bound = tol * float(want.abs().max())     # the activation between the two products is rounded to bfloat16
        for rows in (70, 9):
            got = part.forward(x[:rows].to(DEV)).cpu()
            assert got.dtype == torch.float32
            assert float((got - want[:rows]).abs().max()) <= bound


def test_embedding_and_head_parts_alone():
    embedding = build_part("embedding", PartSpec("token_embedding", {"vocab_size": 50, "hidden_size": 24}, "e"), ctx())
    table = randn(50, 24, seed=7)
    embedding.set_param("e.weight", table.to(DEV))
    tied = build_part("head", PartSpec("lm_head", {"vocab_size": 50, "hidden_size": 24, "tied": True}, "h"), ctx())
    tied.tie(embedding)
    assert tied.param_specs() == {}
    z = randn(3, 24, seed=8)
    torch.testing.assert_close(tied.forward(z.to(DEV)).cpu(), z @ table.T, atol=1e-5, rtol=1e-5)
    untied = build_part("head", PartSpec("lm_head", {"vocab_size": 50, "hidden_size": 24}, "h"), ctx())
    matrix = randn(50, 24, seed=9)
    untied.set_param("h.weight", matrix.to(DEV))
    torch.testing.assert_close(untied.forward(z.to(DEV)).cpu(), z @ matrix.T, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_mixer_and_block_alone(dtype):
    """One pre-norm block built from specs, stepped over a paged cache in two portions and a
    decode token, against the plain layer on the whole sequence."""
    hidden, heads, kv_heads, head_dim, inter, eps, theta = 48, 3, 1, 16, 80, 1e-5, 1e4
    plan_config = {"num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": head_dim,
                   "rms_norm_eps": eps, "rope_theta": theta}
    spec = LayerSpec(
        "pre_norm",
        PartSpec("gqa_attention", {"hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": head_dim,
                                   "qk_norm_eps": eps, "position": PartSpec("rotary", {"head_dim": head_dim, "theta": theta})},
                 "model.layers.0.self_attn"),
        PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": inter}, "model.layers.0.mlp"),
        {"input": PartSpec("rms_norm", {"size": hidden, "eps": eps}, "model.layers.0.input_layernorm"),
         "post_mixer": PartSpec("rms_norm", {"size": hidden, "eps": eps}, "model.layers.0.post_attention_layernorm")})
    plan = ModelPlan(hidden, 30, PartSpec("token_embedding", {"vocab_size": 30, "hidden_size": hidden}, "model.embed_tokens"),
                     (spec,), (LayerCall(0),), PartSpec("rms_norm", {"size": hidden, "eps": eps}, "model.norm"),
                     PartSpec("lm_head", {"vocab_size": 30, "hidden_size": hidden, "tied": True}, "lm_head"))
    from forge_engine_amd.models import DecoderModel
    model = DecoderModel(plan, ctx(dtype))
    fill_random_weights(model, 3, device=DEV, dtype=dtype)
    block = model.layers[0]
    weights = {}
    for module, part in block.mixer.split_qkv_weight().items():
        weights[f"model.layers.0.self_attn.{module}.weight"] = part.float().cpu()
    weights["model.layers.0.self_attn.o_proj.weight"] = block.mixer.o_weight.float().cpu()
    weights["model.layers.0.self_attn.q_norm.weight"] = block.mixer.q_norm.cpu()
    weights["model.layers.0.self_attn.k_norm.weight"] = block.mixer.k_norm.cpu()
    weights["model.layers.0.mlp.gate_proj.weight"] = block.feed_forward.gate_up_weight[:inter].float().cpu()
    weights["model.layers.0.mlp.up_proj.weight"] = block.feed_forward.gate_up_weight[inter:].float().cpu()
    weights["model.layers.0.mlp.down_proj.weight"] = block.feed_forward.down_weight.float().cpu()
    weights["model.layers.0.input_layernorm.weight"] = block.norms["input"].weight.cpu()
    weights["model.layers.0.post_attention_layernorm.weight"] = block.norms["post_mixer"].weight.cpu()
    h = randn(12, hidden, seed=11)
    want = plain.decoder_layer(h, weights, 0, plan_config, torch.arange(12))
    runner = ModelRunner(model, block_size=4, block_capacity=8, num_state_slots=1, use_graphs=False)
    runner.begin("s")
    got = []
    for start, stop in ((0, 7), (7, 11), (11, 12)):
        batch = runner.prepare([StepEntry("s", [0] * (stop - start), [])])
        residual = Residual(h[start:stop].to(DEV).clone())
        block.forward(residual, batch, runner.cache_views(batch)[0])
        got.append(residual.flush().cpu())
        runner.cache.commit("s", stop)
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    torch.testing.assert_close(torch.cat(got), want, atol=tol, rtol=tol)


# ------------------------------------------------- a toy architecture, defined here

class EmaMixer(Mixer):
    """A toy mixer with two states of its own, of different shape and precision: a float32
    s_t = decay * s_{t-1} + x_t (per request, zero before its first token) and a bfloat16 pair
    (n_t, -n_t) that counts the request's tokens (small integers: exact in bfloat16);
    update = W s_t + (n_t / 8) W[:, 0].  Plain torch ops: it is test code, not a kernel."""

    graph_safe = False      # it loops over the step's requests on the host

    def __init__(self, ctx, prefix, *, hidden_size: int, decay: float) -> None:
        super().__init__(ctx, prefix)
        self.hidden_size, self.decay = hidden_size, decay
        self.weight = None

    def param_specs(self):
        return {self.name("mix.weight"): ParamSpec((self.hidden_size, self.hidden_size))}

    def set_param(self, name, tensor):
        self.weight = tensor

    def cache_needs(self):
        return CacheNeeds(state={"ema": FixedState((self.hidden_size,), torch.float32),
                                 "seen": FixedState((2,), torch.bfloat16)})

    def forward(self, x, batch, cache, writes_cache=True):
        assert cache.states["ema"].dtype == torch.float32 and cache.states["seen"].dtype == torch.bfloat16
        out = torch.empty((x.shape[0], self.hidden_size), dtype=torch.float32, device=x.device)
        slots = batch.state_slots_host
        weight = self.weight.float()
        at = 0
        for i, count in enumerate(batch.q_lens):
            # both states are zero when a request begins, also in a slot that another request used: the runner clears them
            state, seen = cache.states["ema"][slots[i]], cache.states["seen"][slots[i]]
            for t in range(at, at + count):
                state.mul_(self.decay).add_(x[t].float())
                seen += torch.tensor([1.0, -1.0], dtype=seen.dtype, device=seen.device)
                assert float(seen[0]) == batch.ctx_before_host[i] + t - at + 1 and float(seen[1]) == -float(seen[0])
                out[t] = weight @ state + seen[0].float() / 8.0 * weight[:, 0]
            at += count
        return out


class DeviceEmaMixer(EmaMixer):
    """The same mixer with nothing decided on the host: it reads the step's layout from the
    device tensors of the batch (``cu_q``, ``token_seq``, ``state_slots``), so its steps may be
    captured and replayed.  Within a step, token t of a sequence that starts at token a gets
    s_t = decay^(t-a+1) * s_before + sum_{a <= u <= t} decay^(t-u) x_u; the state after the
    sequence's last token goes back to its slot, and an empty sequence leaves its slot alone; the
    count of tokens seen goes on from the slot's likewise.  The slot starts at zero because the
    runner clears it when the request begins."""

    graph_safe = True

    def forward(self, x, batch, cache, writes_cache=True):
        tokens = x.shape[0]
        xf = x.float()
        cu, seq, slots = batch.cu_q.long(), batch.token_seq.long(), batch.state_slots.long()
        t = torch.arange(tokens, device=x.device)
        start = cu.index_select(0, seq)
        distance = t[:, None] - t[None, :]
        visible = (seq[:, None] == seq[None, :]) & (distance >= 0)
        mix = torch.where(visible, torch.pow(self.decay, distance.clamp(min=0).float()), torch.zeros((), device=x.device))
        ema, seen = cache.states["ema"], cache.states["seen"]
        before = ema.index_select(0, slots)
        carried = torch.pow(self.decay, (t - start + 1).float())[:, None] * before.index_select(0, seq)
        states = mix @ xf + carried
        lengths = cu[1:] - cu[:-1]
        last = (cu[1:] - 1).clamp(min=0)
        after = torch.where((lengths > 0)[:, None], states.index_select(0, last), before)
        ema.index_copy_(0, slots, after)
        seen_before = seen.index_select(0, slots).float()                       # [sequences, 2]: (n, -n)
        count = seen_before[:, 0].index_select(0, seq) + (t - start + 1).float()
        seen.index_copy_(0, slots, (seen_before + torch.stack((lengths, -lengths), dim=1).float()).to(seen.dtype))
        weight = self.weight.float()
        return states @ weight.T + (count / 8.0)[:, None] * weight[:, 0][None, :]


@dataclass(frozen=True)
class ToyConfig(ModelConfig):
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    window: int
    decay: float
    rms_norm_eps: float
    rope_theta: float
    architecture: ClassVar[str] = "ToyMixedLM"

    @classmethod
    def from_dict(cls, raw):
        read = KeyReader(raw)
        return cls(*(read.integer(k) for k in ("vocab_size", "hidden_size", "intermediate_size", "num_attention_heads",
                                              "num_key_value_heads", "head_dim", "window")),
                   read.number("decay"), read.number("rms_norm_eps"), read.number("rope_theta"))


def toy_plan(config: ToyConfig) -> ModelPlan:
    def norm(prefix):
        return PartSpec("rms_norm", {"size": config.hidden_size, "eps": config.rms_norm_eps}, prefix)

    def attention(prefix, window):
        return PartSpec("gqa_attention", {
            "hidden_size": config.hidden_size, "num_heads": config.num_attention_heads,
            "num_kv_heads": config.num_key_value_heads, "head_dim": config.head_dim, "qk_norm_eps": config.rms_norm_eps,
            "window": window, "position": PartSpec("rotary", {"head_dim": config.head_dim, "theta": config.rope_theta})}, prefix)

    def layer(index, mixer):
        prefix = f"model.layers.{index}"
        return LayerSpec("pre_norm", mixer,
                         PartSpec("swiglu", {"hidden_size": config.hidden_size, "intermediate_size": config.intermediate_size}, f"{prefix}.mlp"),
                         {"input": norm(f"{prefix}.input_layernorm"), "post_mixer": norm(f"{prefix}.post_attention_layernorm")})

    layers = (layer(0, attention("model.layers.0.self_attn", None)),
              layer(1, PartSpec("toy_ema", {"hidden_size": config.hidden_size, "decay": config.decay}, "model.layers.1.ema")),
              layer(2, attention("model.layers.2.self_attn", config.window)))
    # layer 0 runs twice (two caches of its own); the last call runs layer 0's weights
    # over the cache that the first call wrote, writing nothing
    schedule = (LayerCall(0), LayerCall(1), LayerCall(2), LayerCall(0), LayerCall(1), LayerCall(0, cache=0, writes_cache=False))
    sizes = {"vocab_size": config.vocab_size, "hidden_size": config.hidden_size}
    return ModelPlan(config.hidden_size, config.vocab_size, PartSpec("token_embedding", dict(sizes), "model.embed_tokens"),
                     layers, schedule, norm("model.norm"), PartSpec("lm_head", dict(sizes, tied=True), "lm_head"))


def toy_plain_forward(weights, config: ToyConfig, tokens):
    """The toy model on one whole sequence with the plain implementation's functions."""
    positions = torch.arange(len(tokens))
    h = weights["model.embed_tokens.weight"][torch.tensor(tokens)]
    eps = config.rms_norm_eps
    kept = {}

    def attention(x, prefix, window, reuse_kv=None):
        heads, kv_heads, d = config.num_attention_heads, config.num_key_value_heads, config.head_dim
        q = (x @ weights[f"{prefix}.q_proj.weight"].T).view(-1, heads, d)
        q = plain.rms_norm(q, weights[f"{prefix}.q_norm.weight"], eps).transpose(0, 1)
        cos, sin = plain.rotary_tables(positions, d, config.rope_theta)
        q = plain.apply_rotary(q, cos, sin)
        if reuse_kv is None:
            k = (x @ weights[f"{prefix}.k_proj.weight"].T).view(-1, kv_heads, d)
            k = plain.apply_rotary(plain.rms_norm(k, weights[f"{prefix}.k_norm.weight"], eps).transpose(0, 1), cos, sin)
            v = (x @ weights[f"{prefix}.v_proj.weight"].T).view(-1, kv_heads, d).transpose(0, 1)
        else:
            k, v = reuse_kv
        out = plain.causal_attention(q, k, v, d ** -0.5, window=window)
        return out.transpose(0, 1).reshape(len(tokens), heads * d) @ weights[f"{prefix}.o_proj.weight"].T, (k, v)

    def ema(x, prefix):
        state = torch.zeros(config.hidden_size)
        rows = []
        for t in range(len(tokens)):
            state = config.decay * state + x[t]
            rows.append(weights[f"{prefix}.mix.weight"] @ state + (t + 1) / 8.0 * weights[f"{prefix}.mix.weight"][:, 0])
        return torch.stack(rows)

    for call, (index, mode) in enumerate([(0, "own"), (1, "ema"), (2, "window"), (0, "own"), (1, "ema"), (0, "shared")]):
        prefix = f"model.layers.{index}"
        x = plain.rms_norm(h, weights[f"{prefix}.input_layernorm.weight"], eps)
        if mode == "ema":
            update = ema(x, f"{prefix}.ema")
        elif mode == "shared":
            update, _ = attention(x, f"{prefix}.self_attn", None, reuse_kv=kept[0])
        else:
            update, kv = attention(x, f"{prefix}.self_attn", config.window if mode == "window" else None)
            kept.setdefault(call, kv)
        h, y = plain.add_rms_norm(h, update, weights[f"{prefix}.post_attention_layernorm.weight"], eps)
        h = h + plain.swiglu_mlp(y, weights, f"{prefix}.mlp")
    return plain.rms_norm(h, weights["model.norm.weight"], eps) @ weights["model.embed_tokens.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("ema", [EmaMixer, DeviceEmaMixer])
def test_toy_architecture_registered_from_a_test(dtype, ema):
    """``ema``: the stateful mixer decides on the host (its steps run eagerly), or reads only
    device tensors (its steps are captured and replayed; a captured step must update the state
    once, not once more for the run that precedes the capture)."""
    register_part("mixer", "toy_ema", ema, replace=True)
    register_architecture("ToyMixedLM", ToyConfig, toy_plan, replace=True)
    raw = {"architectures": ["ToyMixedLM"], "vocab_size": 90, "hidden_size": 40, "intermediate_size": 72,
           "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16, "window": 6, "decay": 0.5,
           "rms_norm_eps": 1e-5, "rope_theta": 1e4}
    config = load_model_config(raw)
    assert isinstance(config, ToyConfig)
    model = build_model(config, dtype=dtype, device=DEV)
    fill_random_weights(model, 7, device=DEV, dtype=model.ctx.dtype)
    # the windowed group has a smaller pool: two requests hold at most its window's keys and a step's (4 pages each)
    runner = ModelRunner(model, block_size=4, block_capacity=[24, 8], num_state_slots=2)
    groups = runner.cache.groups
    assert [(g.window or 0, len(g.slots)) for g in groups] == [(0, 2), (6, 1)]   # windowed pages apart from full ones
    assert [p.shape[1] for p in runner.key_pages] == [24, 8] and [pool.capacity for pool in runner.cache.pools] == [24, 8]
    assert {name: (tuple(t.shape[1:]), t.dtype) for name, t in runner.states[1].items()} == {
        "ema": ((40,), torch.float32), "seen": ((2,), torch.bfloat16)}
    weights = {}
    for name in model.param_specs():
        owner = model._owners[name]
        if hasattr(owner, "split_qkv_weight") and name.rsplit(".", 2)[-2] in ("q_proj", "k_proj", "v_proj"):
            weights[name] = owner.split_qkv_weight()[name.rsplit(".", 2)[-2]].float().cpu()
    for index in (0, 1, 2):
        block = model.layers[index]
        p = f"model.layers.{index}"
        weights[f"{p}.input_layernorm.weight"] = block.norms["input"].weight.cpu()
        weights[f"{p}.post_attention_layernorm.weight"] = block.norms["post_mixer"].weight.cpu()
        inter = config.intermediate_size
        weights[f"{p}.mlp.gate_proj.weight"] = block.feed_forward.gate_up_weight[:inter].float().cpu()
        weights[f"{p}.mlp.up_proj.weight"] = block.feed_forward.gate_up_weight[inter:].float().cpu()
        weights[f"{p}.mlp.down_proj.weight"] = block.feed_forward.down_weight.float().cpu()
        if index == 1:
            weights[f"{p}.ema.mix.weight"] = block.mixer.weight.float().cpu()
        else:
            weights[f"{p}.self_attn.o_proj.weight"] = block.mixer.o_weight.float().cpu()
            weights[f"{p}.self_attn.q_norm.weight"] = block.mixer.q_norm.cpu()
            weights[f"{p}.self_attn.k_norm.weight"] = block.mixer.k_norm.cpu()
    weights["model.embed_tokens.weight"] = model.embedding.weight.float().cpu()
    weights["model.norm.weight"] = model.final_norm.weight.cpu()

    requests = ru.make_requests(raw, 3, (23, 9, 31, 14))
    want = {k: toy_plain_forward(weights, config, v) for k, v in requests.items()}
    # two requests at a time in two state slots: portions, then single tokens; the third and
    # fourth request reuse the slots and pages of the first two
    got = {k: [] for k in requests}
    for pair in (("r0", "r1"), ("r2", "r3")):
        at = {k: 0 for k in pair}
        for k in pair:
            runner.begin(k)
        step = 0
        while any(at[k] < len(requests[k]) for k in pair):
            entries = []
            for k in pair:
                if at[k] >= len(requests[k]):
                    continue
                size = (5, 2, 3, 1, 1, 4)[(step + len(k)) % 6] if at[k] < len(requests[k]) - 6 else 1
                size = min(size, len(requests[k]) - at[k])
                entries.append(StepEntry(k, requests[k][at[k]:at[k] + size], list(range(size))))
                at[k] += size
            logits = runner.step(entries).cpu()
            row = 0
            for e in entries:
                got[e.request_id].append(logits[row:row + len(e.tokens)])
                row += len(e.tokens)
            step += 1
        for k in pair:
            runner.end(k)
        assert runner.cache.allocated_pages == 0
        runner.cache.check_invariants()
    # the mixer that reads only device tensors went through captured steps, single tokens and portions
    assert (runner.graph_replays > 10) == (ema is DeviceEmaMixer)
    assert (runner.portion_graph_replays > 0) == (ema is DeviceEmaMixer)
    for k in requests:
        rows = torch.cat(got[k])
        scale = float(want[k].abs().max())
        bound = 1e-4 * scale + 1e-5 if dtype == "float32" else ru.BF16_FRACTION * scale
        assert float((rows - want[k]).abs().max()) <= bound, k


# ------------------- a second toy: learned absolute positions, a feed-forward with routing

class PositionedEmbedding(Embedding):
    """Another position encoding: h0 = E[token] + P[position], a learned table (plain torch ops:
    test code).  The attention layers of this toy rotate nothing."""

    def __init__(self, ctx, prefix, *, vocab_size: int, hidden_size: int, max_positions: int) -> None:
        super().__init__(ctx, prefix)
        self.vocab_size, self.hidden_size, self.max_positions = vocab_size, hidden_size, max_positions
        self.weight = self.positions = None

    def param_specs(self):
        return {self.name("weight"): ParamSpec((self.vocab_size, self.hidden_size)),
                self.name("positions"): ParamSpec((self.max_positions, self.hidden_size))}

    def set_param(self, name, tensor):
        if name == self.name("weight"):
            self.weight = tensor
        else:
            self.positions = tensor

    def forward(self, batch) -> Residual:
        h = self.weight[batch.token_ids.long()].float() + self.positions[batch.positions.long()].float()
        return Residual(h.contiguous())


class RoutedFeedForward(FeedForward):
    """A feed-forward with routing: router logits in float32, the best expert of each token
    (lowest index among equals) weighted by its softmax probability.  Every expert runs on every
    token and a mask keeps the chosen one: nothing is decided on the host, so decode steps with
    this part replay from captured graphs."""

    def __init__(self, ctx, prefix, *, hidden_size: int, intermediate_size: int, experts: int) -> None:
        super().__init__(ctx, prefix)
        self.hidden_size, self.intermediate_size, self.experts = hidden_size, intermediate_size, experts
        self.router = None
        self.gate_up = [None] * experts
        self.down = [None] * experts

    def param_specs(self):
        specs = {self.name("router.weight"): ParamSpec((self.experts, self.hidden_size))}
        for e in range(self.experts):
            specs[self.name(f"experts.{e}.gate_up.weight")] = ParamSpec((2 * self.intermediate_size, self.hidden_size))
            specs[self.name(f"experts.{e}.down.weight")] = ParamSpec((self.hidden_size, self.intermediate_size))
        return specs

    def set_param(self, name, tensor):
        local = name[len(self.prefix) + 1:]
        if local == "router.weight":
            self.router = tensor
        else:
            _, index, which, _ = local.split(".")
            (self.gate_up if which == "gate_up" else self.down)[int(index)] = tensor

    def forward(self, x, batch=None):
        from forge_engine_amd.kernels import ops
        logits = x.float() @ self.router.float().T
        probs = torch.softmax(logits, dim=-1)
        chosen = logits.argmax(dim=-1, keepdim=True)
        update = torch.zeros((x.shape[0], self.hidden_size), dtype=torch.float32, device=x.device)
        for e in range(self.experts):
            out = ops.linear(ops.linear_swiglu(x, self.gate_up[e]), self.down[e], out_dtype=torch.float32)
            update += out * (probs[:, e:e + 1] * (chosen == e))
        return update


@dataclass(frozen=True)
class RoutedConfig(ModelConfig):
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    experts: int
    max_positions: int
    rms_norm_eps: float
    architecture: ClassVar[str] = "ToyRoutedLM"

    @classmethod
    def from_dict(cls, raw):
        read = KeyReader(raw)
        return cls(*(read.integer(k) for k in ("vocab_size", "hidden_size", "intermediate_size", "num_attention_heads",
                                              "num_key_value_heads", "head_dim", "experts", "max_positions")),
                   read.number("rms_norm_eps"))


def routed_plan(config: RoutedConfig) -> ModelPlan:
    def norm(prefix):
        return PartSpec("rms_norm", {"size": config.hidden_size, "eps": config.rms_norm_eps}, prefix)

    def layer(index, feed_forward):
        prefix = f"model.layers.{index}"
        attention = PartSpec("gqa_attention", {
            "hidden_size": config.hidden_size, "num_heads": config.num_attention_heads,
            "num_kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
            "position": PartSpec("none", {})}, f"{prefix}.self_attn")
        return LayerSpec("pre_norm", attention, feed_forward,
                         {"input": norm(f"{prefix}.input_layernorm"), "post_mixer": norm(f"{prefix}.post_attention_layernorm")})

    sizes = {"hidden_size": config.hidden_size, "intermediate_size": config.intermediate_size}
    layers = (layer(0, PartSpec("toy_routed", dict(sizes, experts=config.experts), "model.layers.0.moe")),
              layer(1, PartSpec("swiglu", dict(sizes), "model.layers.1.mlp")))
    table = {"vocab_size": config.vocab_size, "hidden_size": config.hidden_size}
    return ModelPlan(config.hidden_size, config.vocab_size,
                     PartSpec("toy_positioned", dict(table, max_positions=config.max_positions), "model.embed_tokens"),
                     layers, (LayerCall(0), LayerCall(1)), norm("model.norm"), PartSpec("lm_head", dict(table, tied=False), "lm_head"))


def routed_plain_forward(w, config: RoutedConfig, tokens):
    t = len(tokens)
    eps = config.rms_norm_eps
    heads, kv_heads, d = config.num_attention_heads, config.num_key_value_heads, config.head_dim
    h = w["model.embed_tokens.weight"][torch.tensor(tokens)] + w["model.embed_tokens.positions"][:t]
    for index in (0, 1):
        p = f"model.layers.{index}"
        x = plain.rms_norm(h, w[f"{p}.input_layernorm.weight"], eps)
        q = (x @ w[f"{p}.self_attn.q_proj.weight"].T).view(t, heads, d).transpose(0, 1)
        k = (x @ w[f"{p}.self_attn.k_proj.weight"].T).view(t, kv_heads, d).transpose(0, 1)
        v = (x @ w[f"{p}.self_attn.v_proj.weight"].T).view(t, kv_heads, d).transpose(0, 1)
        attn = plain.causal_attention(q, k, v, d ** -0.5).transpose(0, 1).reshape(t, heads * d)
        h, y = plain.add_rms_norm(h, attn @ w[f"{p}.self_attn.o_proj.weight"].T, w[f"{p}.post_attention_layernorm.weight"], eps)
        if index == 1:
            h = h + plain.swiglu_mlp(y, w, f"{p}.mlp")
            continue
        logits = y @ w[f"{p}.moe.router.weight"].T
        probs = torch.softmax(logits, dim=-1)
        rows = []
        for i in range(t):
            e = int(logits[i].argmax())
            gate_up = w[f"{p}.moe.experts.{e}.gate_up.weight"]
            inter = config.intermediate_size
            act = torch.nn.functional.silu(y[i] @ gate_up[:inter].T) * (y[i] @ gate_up[inter:].T)
            rows.append(probs[i, e] * (act @ w[f"{p}.moe.experts.{e}.down.weight"].T))
        h = h + torch.stack(rows)
    return plain.rms_norm(h, w["model.norm.weight"], eps) @ w["lm_head.weight"].T


def test_routed_feed_forward_and_learned_positions_registered_from_a_test(tmp_path):
    """Parts of other kinds than Qwen3's (an embedding that adds learned positions, attention
    without rotation, a feed-forward with routing in one layer and a dense one in the other) are
    registered here, built from a model folder and stepped: portions, then decoding through
    captured graphs, against a plain whole-sequence implementation."""
    register_part("embedding", "toy_positioned", PositionedEmbedding, replace=True)
    register_part("feed_forward", "toy_routed", RoutedFeedForward, replace=True)
    register_architecture("ToyRoutedLM", RoutedConfig, routed_plan, replace=True)
    raw = {"architectures": ["ToyRoutedLM"], "vocab_size": 77, "hidden_size": 48, "intermediate_size": 40,
           "num_attention_heads": 3, "num_key_value_heads": 3, "head_dim": 16, "experts": 3, "max_positions": 64,
           "rms_norm_eps": 1e-6}
    config = load_model_config(raw)
    folder = write_random_model(config, 11, tmp_path, dtype=torch.float32)
    assert json.loads((folder / "config.json").read_text())["experts"] == 3
    w = {k: v.float() for k, v in load_file(str(folder / "model.safetensors")).items()}
    w["model.embed_tokens.positions"] *= 20.0     # positions that matter, and routing that is not uniform
    w["model.layers.0.moe.router.weight"] *= 200.0
    from safetensors.torch import save_file
    save_file({k: v.contiguous() for k, v in w.items()}, str(folder / "model.safetensors"))
    _, model = load_model(folder, dtype="float32", device=DEV)
    assert model.graph_safe
    requests = ru.make_requests(raw, 5, (29, 40, 17))
    want = {k: routed_plain_forward(w, config, v) for k, v in requests.items()}
    runner = ModelRunner(model, block_size=4, block_capacity=30, num_state_slots=3)
    got = {k: [] for k in requests}
    for k in requests:
        runner.begin(k)
    cut = {k: len(v) - 8 for k, v in requests.items()}
    at = {k: 0 for k in requests}
    step = 0
    while any(at[k] < cut[k] for k in requests):          # prompts in portions of changing size, side by side
        entries = []
        for k in requests:
            size = min((7, 2, 5, 3)[(step + len(requests[k])) % 4], cut[k] - at[k])
            if size > 0:
                entries.append(StepEntry(k, requests[k][at[k]:at[k] + size], list(range(size))))
                at[k] += size
        logits = runner.step(entries).cpu()
        row = 0
        for e in entries:
            got[e.request_id].append(logits[row:row + len(e.tokens)])
            row += len(e.tokens)
        step += 1
    for i in range(8):                                     # then single tokens: captured graphs
        entries = [StepEntry(k, [requests[k][cut[k] + i]], [0]) for k in requests]
        logits = runner.step(entries).cpu()
        for row, e in enumerate(entries):
            got[e.request_id].append(logits[row:row + 1])
    assert runner.graph_replays >= 6
    for k in requests:
        rows = torch.cat(got[k])
        scale = float(want[k].abs().max())
        assert float((rows - want[k]).abs().max()) <= 1e-4 * scale + 1e-5, k
    # the routing really spreads: every expert is some token's choice
    y = plain.rms_norm(w["model.embed_tokens.weight"], w["model.norm.weight"], 1e-6)
    assert len(set((y @ w["model.layers.0.moe.router.weight"].T).argmax(-1).tolist())) == 3


# ------------------- a third toy: a position encoding with two axes a token (per-token inputs of a step)

class GridEmbedding(Embedding):
    """h0 = E[token] + R[row] + C[column]: a learned position encoding over two axes, which a step's
    entries bring per token (an image's patches have a row and a column; text has its position on
    both).  The part asks for them by name; the framework carries them beside the positions."""

    def __init__(self, ctx, prefix, *, vocab_size: int, hidden_size: int, max_positions: int) -> None:
        super().__init__(ctx, prefix)
        self.vocab_size, self.hidden_size, self.max_positions = vocab_size, hidden_size, max_positions
        self.tables = {}

    def token_inputs(self):
        return {"grid": 2}

    def param_specs(self):
        return {self.name("weight"): ParamSpec((self.vocab_size, self.hidden_size)),
                self.name("rows"): ParamSpec((self.max_positions, self.hidden_size)),
                self.name("columns"): ParamSpec((self.max_positions, self.hidden_size))}

    def set_param(self, name, tensor):
        self.tables[name[len(self.prefix) + 1:]] = tensor

    def forward(self, batch) -> Residual:
        grid = batch.inputs["grid"].long()
        h = (self.tables["weight"][batch.token_ids.long()].float() + self.tables["rows"][grid[:, 0]].float()
             + self.tables["columns"][grid[:, 1]].float())
        return Residual(h.contiguous())


@dataclass(frozen=True)
class GridConfig(ModelConfig):
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_positions: int
    rms_norm_eps: float
    architecture: ClassVar[str] = "ToyGridLM"

    @classmethod
    def from_dict(cls, raw):
        read = KeyReader(raw)
        return cls(*(read.integer(k) for k in ("vocab_size", "hidden_size", "intermediate_size", "num_attention_heads",
                                              "num_key_value_heads", "head_dim", "max_positions")),
                   read.number("rms_norm_eps"))


def grid_plan(config: GridConfig) -> ModelPlan:
    def norm(prefix):
        return PartSpec("rms_norm", {"size": config.hidden_size, "eps": config.rms_norm_eps}, prefix)

    prefix = "model.layers.0"
    attention = PartSpec("gqa_attention", {
        "hidden_size": config.hidden_size, "num_heads": config.num_attention_heads,
        "num_kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
        "position": PartSpec("none", {})}, f"{prefix}.self_attn")
    mlp = PartSpec("swiglu", {"hidden_size": config.hidden_size, "intermediate_size": config.intermediate_size}, f"{prefix}.mlp")
    layer = LayerSpec("pre_norm", attention, mlp,
                      {"input": norm(f"{prefix}.input_layernorm"), "post_mixer": norm(f"{prefix}.post_attention_layernorm")})
    table = {"vocab_size": config.vocab_size, "hidden_size": config.hidden_size}
    return ModelPlan(config.hidden_size, config.vocab_size,
                     PartSpec("toy_grid", dict(table, max_positions=config.max_positions), "model.embed_tokens"),
                     (layer,), (LayerCall(0),), norm("model.norm"), PartSpec("lm_head", dict(table, tied=False), "lm_head"))


def grid_plain_forward(w, config: GridConfig, tokens, grid):
    t = len(tokens)
    eps = config.rms_norm_eps
    heads, kv_heads, d = config.num_attention_heads, config.num_key_value_heads, config.head_dim
    grid = torch.tensor(grid)
    h = (w["model.embed_tokens.weight"][torch.tensor(tokens)] + w["model.embed_tokens.rows"][grid[:, 0]]
         + w["model.embed_tokens.columns"][grid[:, 1]])
    p = "model.layers.0"
    x = plain.rms_norm(h, w[f"{p}.input_layernorm.weight"], eps)
    q = (x @ w[f"{p}.self_attn.q_proj.weight"].T).view(t, heads, d).transpose(0, 1)
    k = (x @ w[f"{p}.self_attn.k_proj.weight"].T).view(t, kv_heads, d).transpose(0, 1)
    v = (x @ w[f"{p}.self_attn.v_proj.weight"].T).view(t, kv_heads, d).transpose(0, 1)
    attn = plain.causal_attention(q, k, v, d ** -0.5).transpose(0, 1).reshape(t, heads * d)
    h, y = plain.add_rms_norm(h, attn @ w[f"{p}.self_attn.o_proj.weight"].T, w[f"{p}.post_attention_layernorm.weight"], eps)
    h = h + plain.swiglu_mlp(y, w, f"{p}.mlp")
    return plain.rms_norm(h, w["model.norm.weight"], eps) @ w["lm_head.weight"].T


def test_a_position_encoding_with_two_axes_registered_from_a_test(tmp_path):
    """A part may ask for integers per token beside the positions (`token_inputs`); a step's entries
    bring them, the batch carries them, eager and in captured graphs.  Here: rows and columns of a
    learned two-axis position encoding.  Prompt tokens lie on a grid of their own (six to a row), the
    tokens after the prompt bring nothing and get their position on both axes, except one request whose
    decode steps bring explicit rows.  Against a plain whole-sequence implementation; then the same
    through the scheduler, greedy."""
    register_part("embedding", "toy_grid", GridEmbedding, replace=True)
    register_architecture("ToyGridLM", GridConfig, grid_plan, replace=True)
    raw = {"architectures": ["ToyGridLM"], "vocab_size": 61, "hidden_size": 48, "intermediate_size": 40,
           "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 16, "max_positions": 80, "rms_norm_eps": 1e-6}
    config = load_model_config(raw)
    folder = write_random_model(config, 13, tmp_path, dtype=torch.float32)
    w = {k: v.float() for k, v in load_file(str(folder / "model.safetensors")).items()}
    for name in ("rows", "columns"):
        w[f"model.embed_tokens.{name}"] *= 20.0           # positions that matter
    from safetensors.torch import save_file
    save_file({k: v.contiguous() for k, v in w.items()}, str(folder / "model.safetensors"))
    _, model = load_model(folder, dtype="float32", device=DEV)
    assert model.token_inputs() == {"grid": 2} and model.graph_safe
    requests = ru.make_requests(raw, 6, (29, 40, 17))
    tail = 8                                               # tokens fed one by one at the end
    explicit = "r1"                                        # this request's single tokens bring rows of their own
    assert explicit in requests

    def grid_of(name, length):
        prompt = length - tail
        rows = [[i // 6, i % 6 + 7] for i in range(prompt)]
        if name == explicit:
            rows += [[70 - j, 3 * j] for j in range(tail)]
        else:
            rows += [[i, i] for i in range(prompt, length)]
        return rows

    grids = {k: grid_of(k, len(v)) for k, v in requests.items()}
    want = {k: grid_plain_forward(w, config, v, grids[k]) for k, v in requests.items()}
    # the encoding matters: with every token's position on both axes the logits differ
    plain_positions = grid_plain_forward(w, config, requests["r0"], [[i, i] for i in range(len(requests["r0"]))])
    assert float((plain_positions - want["r0"]).abs().max()) > 0.1 * float(want["r0"].abs().max())

    runner = ModelRunner(model, block_size=4, block_capacity=30, num_state_slots=3, eager_sightings=1)
    got = {k: [] for k in requests}
    for k in requests:
        runner.begin(k)
    cut = {k: len(v) - tail for k, v in requests.items()}
    at = {k: 0 for k in requests}
    step = 0
    while any(at[k] < cut[k] for k in requests):          # prompts in portions of changing size, side by side
        entries = []
        for k in requests:
            size = min((7, 2, 5, 3)[(step + len(requests[k])) % 4], cut[k] - at[k])
            if size > 0:
                entries.append(StepEntry(k, requests[k][at[k]:at[k] + size], list(range(size)),
                                         {"grid": grids[k][at[k]:at[k] + size]}))
                at[k] += size
        logits = runner.step(entries).cpu()
        row = 0
        for e in entries:
            got[e.request_id].append(logits[row:row + len(e.tokens)])
            row += len(e.tokens)
        step += 1
    assert runner.portion_graph_replays >= 1
    for i in range(tail):                                  # then single tokens: captured graphs, steady steps
        entries = [StepEntry(k, [requests[k][cut[k] + i]], [0],
                             {"grid": [grids[k][cut[k] + i]]} if k == explicit else None) for k in requests]
        logits = runner.step(entries).cpu()
        for row, e in enumerate(entries):
            got[e.request_id].append(logits[row:row + 1])
    assert runner.graph_replays >= tail - 2 and runner.steady_steps >= 1
    for k in requests:
        rows = torch.cat(got[k])
        scale = float(want[k].abs().max())
        assert float((rows - want[k]).abs().max()) <= 1e-4 * scale + 1e-5, k
    with pytest.raises(ValueError, match="rows of 2 integers"):
        runner.step([StepEntry("r0", [1, 2], [], {"grid": [[1, 2]]})])
    with pytest.raises(ValueError, match="no part of the model"):
        runner.step([StepEntry("r0", [1, 2], [], {"axes": [[1], [2]]})])

    # through the scheduler: the prompt's rows come with the request, sampled tokens get their position
    scheduler = SchedulerConfig(block_size=4, block_capacity=40, token_budget=11, max_batch_size=4, max_requests=4,
                                prefill_chunk=6)
    engine = build_engine(model, scheduler_config=scheduler)
    prompts = {k: v[:cut[k]] for k, v in requests.items()}
    ids = {k: engine.submit(prompts[k], sampling_params=SamplingParams(max_new_tokens=5),
                            inputs={"grid": grids[k][:cut[k]]}) for k in requests}
    engine.run_until_idle()
    for k, request_id in ids.items():
        tokens, grid = list(prompts[k]), list(grids[k][:cut[k]])
        for _ in range(5):
            tokens.append(int(grid_plain_forward(w, config, tokens, grid)[-1].argmax()))
            grid.append([len(grid), len(grid)])           # a sampled token: its position on both axes
        assert list(engine.request(request_id).output_token_ids) == tokens[cut[k]:], k
    with pytest.raises(ValueError, match="asks for no token input"):
        engine.submit([1, 2, 3], inputs={"axes": [[0], [1], [2]]})


class ParallelBlock(Block):
    """``h += mixer(norm(h)) + ffn(norm(h))``: one norm, both parts read the same rows."""

    def forward(self, residual: Residual, batch, cache, writes_cache: bool = True) -> None:
        x = self.norms["input"].forward(residual)
        residual.add(self.mixer.forward(x, batch, cache, writes_cache))
        residual.add(self.feed_forward.forward(x, batch))


class SandwichBlock(Block):
    """``h += norm_a(mixer(norm_in(h))); h += norm_b(ffn(norm_post(h)))``: a norm on what each part
    returns as well as on what it reads."""

    def normalised(self, update, norm, like):
        inner = Residual(torch.zeros_like(like))      # an update may come as partial sums: added up here
        inner.add(update)
        return norm.forward(inner).float()

    def forward(self, residual: Residual, batch, cache, writes_cache: bool = True) -> None:
        x = self.norms["input"].forward(residual)
        residual.add(self.normalised(self.mixer.forward(x, batch, cache, writes_cache), self.norms["after_mixer"], residual.h))
        y = self.norms["post_mixer"].forward(residual)
        residual.add(self.normalised(self.feed_forward.forward(y, batch), self.norms["after_ffn"], residual.h))


ARRANGEMENTS = ("pre_norm", "toy_parallel", "toy_sandwich", "toy_parallel")
ARRANGED_NORMS = {"pre_norm": ("input_layernorm", "post_attention_layernorm"), "toy_parallel": ("input_layernorm",),
                  "toy_sandwich": ("input_layernorm", "after_mixer_norm", "post_attention_layernorm", "after_ffn_norm")}
NORM_ROLES = {"input_layernorm": "input", "post_attention_layernorm": "post_mixer", "after_mixer_norm": "after_mixer",
              "after_ffn_norm": "after_ffn"}


@dataclass(frozen=True)
class ArrangedConfig(ModelConfig):
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    architecture: ClassVar[str] = "ToyArrangedLM"

    @classmethod
    def from_dict(cls, raw):
        read = KeyReader(raw)
        return cls(*(read.integer(k) for k in ("vocab_size", "hidden_size", "intermediate_size", "num_attention_heads",
                                              "num_key_value_heads", "head_dim")),
                   read.number("rms_norm_eps"), read.number("rope_theta"))


def arranged_plan(config: ArrangedConfig) -> ModelPlan:
    def norm(prefix):
        return PartSpec("rms_norm", {"size": config.hidden_size, "eps": config.rms_norm_eps}, prefix)

    def layer(index, arrangement):
        prefix = f"model.layers.{index}"
        attention = PartSpec("gqa_attention", {
            "hidden_size": config.hidden_size, "num_heads": config.num_attention_heads,
            "num_kv_heads": config.num_key_value_heads, "head_dim": config.head_dim, "qk_norm_eps": config.rms_norm_eps,
            "position": PartSpec("rotary", {"head_dim": config.head_dim, "theta": config.rope_theta})}, f"{prefix}.self_attn")
        mlp = PartSpec("swiglu", {"hidden_size": config.hidden_size, "intermediate_size": config.intermediate_size}, f"{prefix}.mlp")
        return LayerSpec(arrangement, attention, mlp,
                         {NORM_ROLES[name]: norm(f"{prefix}.{name}") for name in ARRANGED_NORMS[arrangement]})

    layers = tuple(layer(i, a) for i, a in enumerate(ARRANGEMENTS))
    table = {"vocab_size": config.vocab_size, "hidden_size": config.hidden_size}
    return ModelPlan(config.hidden_size, config.vocab_size, PartSpec("token_embedding", dict(table), "model.embed_tokens"),
                     layers, tuple(LayerCall(i) for i in range(len(layers))), norm("model.norm"),
                     PartSpec("lm_head", dict(table, tied=False), "lm_head"))


def arranged_plain_forward(w, config: ArrangedConfig, tokens):
    t = len(tokens)
    eps = config.rms_norm_eps
    heads, kv_heads, d = config.num_attention_heads, config.num_key_value_heads, config.head_dim
    cos, sin = plain.rotary_tables(torch.arange(t), d, config.rope_theta)

    def attention(x, p):
        q = plain.rms_norm((x @ w[f"{p}.q_proj.weight"].T).view(t, heads, d), w[f"{p}.q_norm.weight"], eps).transpose(0, 1)
        k = plain.rms_norm((x @ w[f"{p}.k_proj.weight"].T).view(t, kv_heads, d), w[f"{p}.k_norm.weight"], eps).transpose(0, 1)
        v = (x @ w[f"{p}.v_proj.weight"].T).view(t, kv_heads, d).transpose(0, 1)
        out = plain.causal_attention(plain.apply_rotary(q, cos, sin), plain.apply_rotary(k, cos, sin), v, d ** -0.5)
        return out.transpose(0, 1).reshape(t, heads * d) @ w[f"{p}.o_proj.weight"].T

    h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    for index, arrangement in enumerate(ARRANGEMENTS):
        p = f"model.layers.{index}"
        x = plain.rms_norm(h, w[f"{p}.input_layernorm.weight"], eps)
        update = attention(x, f"{p}.self_attn")
        if arrangement == "pre_norm":
            h, y = plain.add_rms_norm(h, update, w[f"{p}.post_attention_layernorm.weight"], eps)
            h = h + plain.swiglu_mlp(y, w, f"{p}.mlp")
        elif arrangement == "toy_parallel":
            h = h + update + plain.swiglu_mlp(x, w, f"{p}.mlp")
        else:
            h = h + plain.rms_norm(update, w[f"{p}.after_mixer_norm.weight"], eps)
            y = plain.rms_norm(h, w[f"{p}.post_attention_layernorm.weight"], eps)
            h = h + plain.rms_norm(plain.swiglu_mlp(y, w, f"{p}.mlp"), w[f"{p}.after_ffn_norm.weight"], eps)
    return plain.rms_norm(h, w["model.norm.weight"], eps) @ w["lm_head.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_block_arrangements_registered_from_a_test(dtype, tmp_path):
    """How a layer's parts and norms are arranged is a part like the others: a model whose layers
    are the framework's arrangement, one with a single norm whose parts run side by side, and one
    with norms behind its parts too, each chosen by name layer by layer.  Portions of changing
    size, then single tokens through captured graphs, against a plain whole-sequence implementation."""
    register_part("block", "toy_parallel", ParallelBlock, replace=True)
    register_part("block", "toy_sandwich", SandwichBlock, replace=True)
    register_architecture("ToyArrangedLM", ArrangedConfig, arranged_plan, replace=True)
    raw = {"architectures": ["ToyArrangedLM"], "vocab_size": 83, "hidden_size": 48, "intermediate_size": 56,
           "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 16, "rms_norm_eps": 1e-5, "rope_theta": 1e4}
    config = load_model_config(raw)
    folder = write_random_model(config, 19, tmp_path)
    w = {k: v.float() for k, v in load_file(str(folder / "model.safetensors")).items()}
    assert "model.layers.2.after_ffn_norm.weight" in w and "model.layers.1.post_attention_layernorm.weight" not in w
    _, model = load_model(folder, dtype=dtype, device=DEV)
    requests = ru.make_requests(raw, 8, (37, 22, 30))
    want = {k: arranged_plain_forward(w, config, v) for k, v in requests.items()}
    runner = ModelRunner(model, block_size=4, block_capacity=30, num_state_slots=3, eager_sightings=1)
    got = {k: [] for k in requests}
    for k in requests:
        runner.begin(k)
    tail = 9
    cut = {k: len(v) - tail for k, v in requests.items()}
    at = {k: 0 for k in requests}
    step = 0
    while any(at[k] < cut[k] for k in requests):
        entries = []
        for k in requests:
            size = min((6, 2, 5, 3)[(step + len(requests[k])) % 4], cut[k] - at[k])
            if size > 0:
                entries.append(StepEntry(k, requests[k][at[k]:at[k] + size], list(range(size))))
                at[k] += size
        logits = runner.step(entries).float().cpu()
        row = 0
        for e in entries:
            got[e.request_id].append(logits[row:row + len(e.tokens)])
            row += len(e.tokens)
        step += 1
    for i in range(tail):
        entries = [StepEntry(k, [requests[k][cut[k] + i]], [0]) for k in requests]
        logits = runner.step(entries).float().cpu()
        for row, e in enumerate(entries):
            got[e.request_id].append(logits[row:row + 1])
    assert runner.graph_replays >= tail - 2
    for k in requests:
        rows = torch.cat(got[k])
        scale = float(want[k].abs().max())
        bound = 1e-4 * scale + 1e-5 if dtype == "float32" else ru.BF16_FRACTION * scale
        assert float((rows - want[k]).abs().max()) <= bound, k


class CentredNorm(Norm):
    """``y = (s - mean(s)) / sqrt(var(s) + eps) * w + b`` with ``s`` the stream plus what is pending:
    a norm that subtracts the mean and has a bias, in plain tensor operations."""

    def __init__(self, ctx, prefix, *, size: int, eps: float) -> None:
        super().__init__(ctx, prefix)
        self.size, self.eps = size, float(eps)
        self.tensors = {}

    def param_specs(self):
        return {self.name("weight"): ParamSpec((self.size,), kind="vector", init="norm"),
                self.name("bias"): ParamSpec((self.size,), kind="vector", init="norm")}

    def set_param(self, name, tensor):
        self.tensors[name[len(self.prefix) + 1:]] = tensor

    def forward(self, residual: Residual, rows=None):
        if rows is None:
            s = residual.flush()
        else:                       # the chosen rows; the stream and what is pending stay as they are
            s = residual.h[rows.long()]
            if residual.pending is not None:
                pending = residual.pending if residual.pending.dim() == 2 else residual.pending.sum(0)
                s = s + pending[rows.long()]
        centred = s - s.mean(-1, keepdim=True)
        y = centred * torch.rsqrt(centred.square().mean(-1, keepdim=True) + self.eps)
        return (y * self.tensors["weight"] + self.tensors["bias"]).to(self.ctx.dtype)


class CappedHead(Head):
    """``logits = cap * tanh((z W^T) / cap)``: a head with a matrix of its own that bounds its logits."""

    def __init__(self, ctx, prefix, *, vocab_size: int, hidden_size: int, cap: float) -> None:
        super().__init__(ctx, prefix)
        self.vocab_size, self.hidden_size, self.cap = vocab_size, hidden_size, float(cap)
        self.weight = None

    def param_specs(self):
        return {self.name("weight"): ParamSpec((self.vocab_size, self.hidden_size))}

    def set_param(self, name, tensor):
        self.weight = tensor

    def forward(self, z):
        return self.cap * torch.tanh(z.float() @ self.weight.float().T / self.cap)


@dataclass(frozen=True)
class CentredConfig(ModelConfig):
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    norm_eps: float
    rope_theta: float
    logit_cap: float
    architecture: ClassVar[str] = "ToyCentredLM"

    @classmethod
    def from_dict(cls, raw):
        read = KeyReader(raw)
        return cls(*(read.integer(k) for k in ("vocab_size", "hidden_size", "intermediate_size", "num_attention_heads",
                                              "num_key_value_heads", "head_dim")),
                   read.number("norm_eps"), read.number("rope_theta"), read.number("logit_cap"))


def centred_plan(config: CentredConfig) -> ModelPlan:
    def norm(prefix):
        return PartSpec("toy_centred", {"size": config.hidden_size, "eps": config.norm_eps}, prefix)

    def layer(index):
        prefix = f"model.layers.{index}"
        attention = PartSpec("gqa_attention", {
            "hidden_size": config.hidden_size, "num_heads": config.num_attention_heads,
            "num_kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
            "position": PartSpec("rotary", {"head_dim": config.head_dim, "theta": config.rope_theta})}, f"{prefix}.self_attn")
        mlp = PartSpec("swiglu", {"hidden_size": config.hidden_size, "intermediate_size": config.intermediate_size}, f"{prefix}.mlp")
        return LayerSpec("pre_norm", attention, mlp,
                         {"input": norm(f"{prefix}.input_layernorm"), "post_mixer": norm(f"{prefix}.post_attention_layernorm")})

    table = {"vocab_size": config.vocab_size, "hidden_size": config.hidden_size}
    return ModelPlan(config.hidden_size, config.vocab_size, PartSpec("token_embedding", dict(table), "model.embed_tokens"),
                     (layer(0), layer(1)), (LayerCall(0), LayerCall(1)), norm("model.norm"),
                     PartSpec("toy_capped", dict(table, cap=config.logit_cap), "lm_head"))


def centred_plain_forward(w, config: CentredConfig, tokens):
    t = len(tokens)
    heads, kv_heads, d = config.num_attention_heads, config.num_key_value_heads, config.head_dim
    cos, sin = plain.rotary_tables(torch.arange(t), d, config.rope_theta)

    def norm(x, prefix):
        return torch.nn.functional.layer_norm(x, (config.hidden_size,), w[f"{prefix}.weight"], w[f"{prefix}.bias"], config.norm_eps)

    h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    for index in range(2):
        p = f"model.layers.{index}"
        x = norm(h, f"{p}.input_layernorm")
        q = (x @ w[f"{p}.self_attn.q_proj.weight"].T).view(t, heads, d).transpose(0, 1)
        k = (x @ w[f"{p}.self_attn.k_proj.weight"].T).view(t, kv_heads, d).transpose(0, 1)
        v = (x @ w[f"{p}.self_attn.v_proj.weight"].T).view(t, kv_heads, d).transpose(0, 1)
        out = plain.causal_attention(plain.apply_rotary(q, cos, sin), plain.apply_rotary(k, cos, sin), v, d ** -0.5)
        h = h + out.transpose(0, 1).reshape(t, heads * d) @ w[f"{p}.self_attn.o_proj.weight"].T
        h = h + plain.swiglu_mlp(norm(h, f"{p}.post_attention_layernorm"), w, f"{p}.mlp")
    return config.logit_cap * torch.tanh(norm(h, "model.norm") @ w["lm_head.weight"].T / config.logit_cap)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_norm_and_a_head_registered_from_a_test(dtype, tmp_path):
    """The two roles that the other toys leave to the framework's own parts: a norm that subtracts
    the mean and adds a bias (against the library's layer norm), and a head that bounds its logits.
    The norm meets every way the stream reaches it: an update pending whole or in partial sums,
    nothing pending, and the wanted rows only before the head."""
    register_part("norm", "toy_centred", CentredNorm, replace=True)
    register_part("head", "toy_capped", CappedHead, replace=True)
    register_architecture("ToyCentredLM", CentredConfig, centred_plan, replace=True)
    raw = {"architectures": ["ToyCentredLM"], "vocab_size": 77, "hidden_size": 64, "intermediate_size": 48,
           "num_attention_heads": 2, "num_key_value_heads": 2, "head_dim": 32, "norm_eps": 1e-3, "rope_theta": 1e3,
           "logit_cap": 0.4}
    config = load_model_config(raw)
    folder = write_random_model(config, 23, tmp_path)
    w = {k: v.float() for k, v in load_file(str(folder / "model.safetensors")).items()}
    assert float(w["model.norm.bias"].abs().min()) > 0.5           # a bias that is left out would show
    _, model = load_model(folder, dtype=dtype, device=DEV)
    requests = ru.make_requests(raw, 10, (33, 18))
    want = {k: centred_plain_forward(w, config, v) for k, v in requests.items()}
    assert float(want["r0"].abs().max()) > 0.5 * config.logit_cap     # the cap bends the logits
    runner = ModelRunner(model, block_size=4, block_capacity=20, num_state_slots=2, eager_sightings=1)
    got = {k: [] for k in requests}
    for k in requests:
        runner.begin(k)
    tail = 7
    cut = {k: len(v) - tail for k, v in requests.items()}
    at = {k: 0 for k in requests}
    step = 0
    while any(at[k] < cut[k] for k in requests):
        entries = []
        for k in requests:
            size = min((4, 7, 2)[(step + len(requests[k])) % 3], cut[k] - at[k])
            if size > 0:
                entries.append(StepEntry(k, requests[k][at[k]:at[k] + size], list(range(size))))
                at[k] += size
        logits = runner.step(entries).float().cpu()
        row = 0
        for e in entries:
            got[e.request_id].append(logits[row:row + len(e.tokens)])
            row += len(e.tokens)
        step += 1
    for i in range(tail):
        entries = [StepEntry(k, [requests[k][cut[k] + i]], [0]) for k in requests]
        logits = runner.step(entries).float().cpu()
        for row, e in enumerate(entries):
            got[e.request_id].append(logits[row:row + 1])
    assert runner.graph_replays >= tail - 2
    for k in requests:
        rows = torch.cat(got[k])
        scale = float(want[k].abs().max())
        bound = 1e-4 * scale + 1e-5 if dtype == "float32" else ru.BF16_FRACTION * scale
        assert float((rows - want[k]).abs().max()) <= bound, k


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batched_decode_through_graphs_matches_eager(dtype, folders):
    """Twenty requests decode together (more than 16 rows: the matrix library's products sit
    inside the captured graph); every replay is compared with the eager step, with eager
    prompt portions of a late request between the replays."""
    name = "C"
    config = TINY[name]
    requests = ru.make_requests(config, 23, tuple(range(17, 57, 2)))        # 20 requests of 17..55 tokens
    late = ru.make_requests(config, 24, (50,))["r0"]
    _, model = load_model(folders[name], dtype=dtype, device=DEV)
    rows = {}
    for graphs in (True, False):
        runner = ModelRunner(model, block_size=16, block_capacity=120, num_state_slots=24, use_graphs=graphs)
        for k, tokens in requests.items():
            runner.begin(k)
            runner.step([StepEntry(k, tokens[:-14], [])])
        runner.begin("late")
        collected = []
        for step in range(14):
            entries = [StepEntry(k, [tokens[len(tokens) - 14 + step]], [0]) for k, tokens in requests.items()]
            collected.append(runner.step(entries).clone())
            if step % 3 == 0:
                runner.step([StepEntry("late", late[step * 3:step * 3 + 9], [0])])
        rows[graphs] = torch.stack(collected).cpu()
        assert (runner.graph_replays == 14) == graphs
        for k in list(requests) + ["late"]:
            runner.end(k)
    want = torch.stack([plain.forward(folder_weights(folders[name]), config, tokens)[-14:] for tokens in requests.values()], dim=1)
    scale = float(want.abs().max())
    bound = 1e-4 * scale if dtype == "float32" else ru.BF16_FRACTION * scale
    assert float((rows[True] - rows[False]).abs().max()) <= bound * 0.5
    assert float((rows[True] - want).abs().max()) <= bound


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("count", [65, 130, 256])
def test_decode_steps_of_many_requests_replay_graphs(count, dtype, folders):
    """Decode steps of 65 to 256 requests are captured and replayed like smaller ones: every
    request's last six tokens one by one, all requests in one step, against the plain
    implementation; a 257th request makes the step run eagerly."""
    name = "C"
    config, weights = TINY[name], folder_weights(folders[name])
    lengths = tuple(7 + (5 * i) % 23 for i in range(count))
    requests = ru.make_requests(config, 41, lengths)
    _, model = load_model(folders[name], dtype=dtype, device=DEV)
    runner = ModelRunner(model, block_size=16, block_capacity=2 * count + 8, num_state_slots=count + 1)
    names = list(requests)
    for at in range(0, count, 40):                                  # prompts, forty requests a step
        for k in names[at:at + 40]:
            runner.begin(k)
        runner.step([StepEntry(k, requests[k][:-6], []) for k in names[at:at + 40]])
    collected = []
    for step in range(6):
        entries = [StepEntry(k, [requests[k][len(requests[k]) - 6 + step]], [0]) for k in names]
        collected.append(runner.step(entries).clone())
    assert runner.graph_replays == 6
    got = torch.stack(collected).cpu()
    want = torch.stack([plain.forward(weights, config, tokens)[-6:] for tokens in requests.values()], dim=1)
    scale = float(want.abs().max())
    bound = 1e-4 * scale + 1e-5 if dtype == "float32" else ru.BF16_FRACTION * scale
    assert float((got - want).abs().max()) <= bound
    if count == 256:
        extra = ru.make_requests(config, 42, (9,))["r0"]
        runner.begin("one more")
        runner.step([StepEntry("one more", extra[:-1], [])])
        replays = runner.graph_replays
        entries = [StepEntry(k, [3], [0]) for k in names] + [StepEntry("one more", extra[-1:], [0])]
        logits = runner.step(entries)
        assert runner.graph_replays == replays and logits.shape[0] == 257
        expect = plain.forward(weights, config, extra)[-1]
        assert float((logits[-1].cpu() - expect).abs().max()) <= bound


def test_steps_of_single_tokens_prepare_queries_and_keys_inside_attention(folders, monkeypatch):
    """A step in which every request brings one token runs norm, rotation, cache write and
    attention as one launch per layer; a mixed step runs them as two.  The same tokens fed
    both ways (the others' single tokens beside a two-token portion of one request, then the
    same single tokens alone) give the same cache and logits within rounding."""
    from forge_engine_amd.kernels import ops
    name = "C"          # head size 128, five query heads a kv head: sizes the fast kernels serve
    config = TINY[name]
    requests = ru.make_requests(config, 29, (40, 33, 21))
    _, model = load_model(folders[name], dtype="bfloat16", device=DEV)
    calls = {"one": 0, "two": 0}
    one, two = ops.decode_attention_prepare, ops.qk_norm_rope_write

    def count_one(*args, **kwargs):
        calls["one"] += 1
        return one(*args, **kwargs)

    def count_two(*args, **kwargs):
        calls["two"] += 1
        return two(*args, **kwargs)

    monkeypatch.setattr(ops, "decode_attention_prepare", count_one)
    monkeypatch.setattr(ops, "qk_norm_rope_write", count_two)
    layers = config["num_hidden_layers"]
    got = {}
    for mode in ("alone", "beside a portion"):
        runner = ModelRunner(model, block_size=16, block_capacity=40, num_state_slots=6, use_graphs=False)
        for k, tokens in requests.items():
            runner.begin(k)
            runner.step([StepEntry(k, tokens[:-6], [])])
        runner.begin("other")
        calls["one"] = calls["two"] = 0
        rows = []
        for step in range(6):
            entries = [StepEntry(k, [tokens[len(tokens) - 6 + step]], [0]) for k, tokens in requests.items()]
            if mode == "beside a portion":
                entries.append(StepEntry("other", [3 + step, 5 + step], []))
            rows.append(runner.step(entries).clone())
        got[mode] = torch.stack(rows).cpu()
        assert (calls["one"], calls["two"]) == ((6 * layers, 0) if mode == "alone" else (0, 6 * layers))
    want = torch.stack([plain.forward(folder_weights(folders[name]), config, tokens)[-6:] for tokens in requests.values()], dim=1)
    bound = ru.BF16_FRACTION * float(want.abs().max())
    assert float((got["alone"] - want).abs().max()) <= bound
    assert float((got["beside a portion"] - want).abs().max()) <= bound
    assert float((got["alone"] - got["beside a portion"]).abs().max()) <= bound * 0.5


@pytest.fixture(scope="module")
def wide_folder(tmp_path_factory):
    """Two layers with the widths, head counts and vocabulary of Qwen3-4B."""
    config = dict(TINY["C"], vocab_size=151936, hidden_size=2560, intermediate_size=9728, num_hidden_layers=2,
                  num_attention_heads=32, num_key_value_heads=8, head_dim=128, max_position_embeddings=4096,
                  rms_norm_eps=1e-6, rope_theta=5000000.0, tie_word_embeddings=True)
    folder = tmp_path_factory.mktemp("engine_wide")
    write_random_model(load_model_config(config), 37, folder)
    weights = folder_weights(folder)
    return folder, config, weights


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_of_the_large_model_against_the_plain_implementation(dtype, wide_folder):
    """The kernels at the sizes they are tuned for (weight-streaming products with resident
    blocks and K in parts, a vocabulary that is no power of two, four query heads a kv head):
    a prompt whole, another with its last tokens one by one, and eight requests decoding
    together through a captured graph, all against the plain implementation."""
    folder, config, weights = wide_folder
    _, model = load_model(folder, dtype=dtype, device=DEV)
    requests = ru.make_requests(config, 41, (150, 97, 40, 43, 46, 49, 52, 55, 58, 61))
    runner = ModelRunner(model, block_size=16, block_capacity=80, num_state_slots=20)
    got, want = {}, {}

    def keep(request_id, positions, logits):
        for row, position in zip(logits.cpu(), positions):
            got[(request_id, position)] = row.clone()

    # whole: the last 8 places of one step
    runner.begin("r0")
    keep("r0", range(142, 150), runner.step([StepEntry("r0", requests["r0"], list(range(142, 150)))]))
    runner.end("r0")
    # most of it in one step, the last 12 one by one
    runner.begin("r1")
    tokens = requests["r1"]
    keep("r1", [84], runner.step([StepEntry("r1", tokens[:85], [84])]))
    for position in range(85, 97):
        keep("r1", [position], runner.step([StepEntry("r1", [tokens[position]], [0])]))
    runner.end("r1")
    # eight together: prompts one after the other, then five steps of eight single tokens
    group = [f"r{i}" for i in range(2, 10)]
    for k in group:
        runner.begin(k)
        runner.step([StepEntry(k, requests[k][:-5], [])])
    for step in range(5):
        logits = runner.step([StepEntry(k, [requests[k][len(requests[k]) - 5 + step]], [0]) for k in group])
        for row, k in zip(logits.cpu(), group):
            got[(k, len(requests[k]) - 5 + step)] = row.clone()
    assert runner.graph_replays >= 5 + 12
    for k in group:
        runner.end(k)
    # eighteen together (more than 16 rows: the products for 17 to 64 rows), three steps
    many = ru.make_requests(config, 43, tuple(range(8, 26)))
    many = {f"m{i}": tokens for i, tokens in enumerate(many.values())}
    requests = {**requests, **many}
    for k, tokens in many.items():
        runner.begin(k)
        runner.step([StepEntry(k, tokens[:-3], [])])
    for step in range(3):
        logits = runner.step([StepEntry(k, [tokens[len(tokens) - 3 + step]], [0]) for k, tokens in many.items()])
        for row, (k, tokens) in zip(logits.cpu(), many.items()):
            got[(k, len(tokens) - 3 + step)] = row.clone()
    for k in many:
        runner.end(k)
    for request_id, tokens in requests.items():
        logits = plain.forward(weights, config, tokens)
        for (rid, position) in got:
            if rid == request_id:
                want[(rid, position)] = logits[position]
    ru.compare(got, want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["portions", "mixed"])
def test_schedules_at_the_large_widths(mode, dtype, wide_folder, tmp_path):
    """Replay at the widths of the large model, where the products that split K over blocks, keep
    their activations resident and serve 17 to 64 rows engage (the tiny models never reach them):
    portions of changing size, and up to four live requests with portions of some beside decoded
    tokens of others in a pool so small that pages are used again.  Logits at the last token of
    every entry of every step."""
    folder, config, weights = wide_folder
    requests = ru.make_requests(config, 71, (40, 70, 33, 90, 25, 50, 61))
    if mode == "portions":
        trace = ru.trace_portions(requests, sizes=(16, 7, 33, 3, 2, 64, 9, 2, 20), want_all=False)
    else:
        trace = ru.trace_mixed(requests, 11, max_live=4, want_all=False, portion_sizes=(2, 3, 5, 8, 13, 21))
        assert sum(ru.round64(len(t)) for t in requests.values()) > trace.peak_tokens     # pages are used again
    rows = {key for keys in trace.rows.values() for key in keys}
    got = ru.run_trace(folder, dtype, trace, tmp_path, block_size=16)
    want = {}
    for request_id, tokens in requests.items():
        positions = sorted(position for rid, position in rows if rid == request_id)
        for row, position in zip(plain.forward(weights, config, tokens, rows=positions), positions):
            want[(request_id, position)] = row
    ru.compare(got, want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_portions_at_the_large_widths(dtype, wide_folder, tmp_path):
    """Portions of 65 to 400 tokens at the widths of the large model: the row counts at which the
    products for portions of prompts run (parts of K in row tiles of 128, the stored q/k/v product in
    tiles of 64 and 128, blocks of eight waves for the long K) and, beyond them, the matrix library
    that adds into the stream as it stores; a step of two portions beside each other; the second and
    later portions read what the first left in the cache.  Logits at each portion's last token."""
    folder, config, weights = wide_folder
    requests = ru.make_requests(config, 73, (700, 330, 129))
    trace = ru.TraceBuilder(False)
    a, b, c = (requests[key] for key in sorted(requests))
    ida, idb, idc = sorted(requests)
    trace.step([(ida, a[:130])])                         # 130 rows
    trace.step([(ida, a[130:330]), (idb, b[:65])])       # 265 rows in one step, two requests
    trace.step([(ida, a[330:700])], end=[ida])           # 370 rows
    trace.step([(idb, b[65:330])], end=[idb])            # 265 rows
    trace.step([(idc, c[:100])])                         # 100 rows
    trace.step([(idc, c[100:129])], end=[idc])
    rows = {key for keys in trace.rows.values() for key in keys}
    got = ru.run_trace(folder, dtype, trace, tmp_path, block_size=16)
    want = {}
    for request_id, tokens in requests.items():
        positions = sorted(position for rid, position in rows if rid == request_id)
        for row, position in zip(plain.forward(weights, config, tokens, rows=positions), positions):
            want[(request_id, position)] = row
    assert len(want) == 7
    ru.compare(got, want, dtype)


def test_a_portion_of_two_thousand_tokens_at_the_large_widths(wide_folder, tmp_path):
    """A prompt of 2,300 tokens fed as 2,100 + 200 at the widths of the large model, bfloat16: the row
    count at which the gate/up product runs in the kernel that keeps tiles of x in LDS (wide tiles for
    whole rounds, narrow ones for the rest, a last row tile that is partly empty), the prefill attention
    walks 33 key tiles, and the second portion reads 2,100 cached keys.  Logits at four positions."""
    folder, config, weights = wide_folder
    tokens = ru.make_requests(config, 75, (2300,))["r0"]
    trace = ru.TraceBuilder(False)
    trace.step([("r0", tokens[:2100])], want_all=False)
    trace.step([("r0", tokens[2100:])], end=["r0"], want_all=False)
    got = ru.run_trace(folder, "bfloat16", trace, tmp_path, block_size=16)
    positions = [2099, 2299]
    want = {("r0", p): row for p, row in zip(positions, plain.forward(weights, config, tokens, rows=positions))}
    assert set(got) == set(want)
    ru.compare(got, want, "bfloat16")


def test_a_portion_of_three_thousand_tokens_at_the_large_widths(wide_folder, tmp_path):
    """A prompt of 3,300 tokens fed as 3,100 + 200 at the widths of the large model, bfloat16: with 32
    query heads the first step is the size from which the prefill attention launch chooses blocks of 128
    query rows (two sets of rows a wave, two LDS buffers) by itself, its last block a partly filled one;
    the gate/up product runs 13 row tiles in the kernel that keeps tiles of x in LDS; the second portion
    reads 3,100 cached keys through a table of 207 pages.  Logits at two positions."""
    folder, config, weights = wide_folder
    tokens = ru.make_requests(config, 76, (3300,))["r0"]
    trace = ru.TraceBuilder(False)
    trace.step([("r0", tokens[:3100])], want_all=False)
    trace.step([("r0", tokens[3100:])], end=["r0"], want_all=False)
    got = ru.run_trace(folder, "bfloat16", trace, tmp_path, block_size=16)
    positions = [3099, 3299]
    want = {("r0", p): row for p, row in zip(positions, plain.forward(weights, config, tokens, rows=positions))}
    assert set(got) == set(want)
    ru.compare(got, want, "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_scheduler_with_sixty_four_rows_at_the_large_widths(dtype, wide_folder):
    """Forty requests through the scheduler at its largest batch (64 requests a step, 256 tokens):
    prompts are cut into portions beside decoded tokens, and decode steps of 17 to 40 rows replay
    graphs of the products for that many rows.  Every generated token must be the plain
    implementation's choice at its place (teacher-forced: one plain pass over prompt and output)."""
    import random
    folder, config, weights = wide_folder
    rng = random.Random(91)
    lengths = [rng.randrange(3, 60) for _ in range(40)]
    prompts = list(ru.make_requests(config, 92, lengths).values())
    new_tokens = [rng.randrange(3, 9) for _ in prompts]
    scheduler = SchedulerConfig(block_size=16, block_capacity=40 * 5, token_budget=256, max_batch_size=64,
                                max_requests=64)
    engine = engine_from_folder(folder, scheduler_config=scheduler, dtype=dtype)
    ids = [engine.submit(p, sampling_params=SamplingParams(max_new_tokens=n)) for p, n in zip(prompts, new_tokens)]
    widest = 0
    while not engine.idle:
        engine.step()
        widest = max(widest, len(engine.snapshot().last_batch))
    assert widest > 32 and engine.cache_pool.allocated_pages == 0
    for request_id, prompt, n in zip(ids, prompts, new_tokens):
        got = list(engine.request(request_id).output_token_ids)
        assert len(got) == n
        places = list(range(len(prompt) - 1, len(prompt) - 1 + n))
        logits = plain.forward(weights, config, prompt + got[:-1], rows=places)
        for row, token in zip(logits, got):
            if dtype == "float32":
                # among 151,936 logits two can lie closer than float32 sums in another order resolve
                # (seen: 4.53608 twice); anything further from the top than that is a wrong token
                assert token == int(row.argmax()) or float(row.max() - row[token]) <= 2 * ru.F32_ATOL, request_id
            else:
                assert float(row.max() - row[token]) <= ru.BF16_FRACTION * float(row.abs().max()), request_id


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_beyond_the_reach_of_32_bit_offsets(dtype, wide_folder):
    """A pool of a layer with more than 2**32 elements, and a request whose pages lie at its
    far end: an offset into the pool that a kernel computed in 32 bits, signed or not, would
    wrap and read or write another page.  The same steps in a small pool give the same logits."""
    folder, config, _ = wide_folder
    _, model = load_model(folder, dtype=dtype, device=DEV)
    tokens = ru.make_requests(config, 67, (150, 40))
    page_elements = config["num_key_value_heads"] * 16 * config["head_dim"]
    low_pages = 2 ** 32 // page_elements + 64

    def run(capacity, held):
        runner = ModelRunner(model, block_size=16, block_capacity=capacity, num_state_slots=4)
        taken = runner.cache.pools[0].allocate(held) if held else []
        rows = []
        runner.begin("a")
        runner.begin("b")
        rows.append(runner.step([StepEntry("a", tokens["r0"][:140], [138, 139])]))                  # a prompt whole
        rows.append(runner.step([StepEntry("a", tokens["r0"][140:146], [5]),                        # portions together
                                 StepEntry("b", tokens["r1"][:37], [36])]))
        for i in range(3):                                                                          # single tokens
            rows.append(runner.step([StepEntry("a", [tokens["r0"][146 + i]], [0]),
                                     StepEntry("b", [tokens["r1"][37 + i]], [0])]))
        pages = [page for name in "ab" for table in runner.cache.request(name).tables for page in table]
        runner.end("a")
        runner.end("b")
        if taken:
            runner.cache.pools[0].release(taken)
        runner.cache.check_invariants()
        return torch.cat([r.float().cpu() for r in rows]), pages

    want, near = run(40, 0)
    torch.cuda.empty_cache()
    got, far = run(low_pages + 40, low_pages)
    torch.cuda.empty_cache()
    assert max(near) < 40 and min(far) >= low_pages and min(far) * page_elements >= 2 ** 32
    scale = float(want.abs().max())
    assert float((got - want).abs().max()) <= (1e-5 if dtype == "float32" else 1e-3) * scale


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_name_used_again_decodes_from_its_new_pages(dtype, folders):
    """A request ends and another begins under the same name with a table of the same length
    but other pages (a third request took the old ones meanwhile): the captured decode step
    must read the new table, not the row it kept for the name."""
    name = "C"
    config, weights = TINY[name], folder_weights(folders[name])
    requests = ru.make_requests(config, 61, (20, 20, 21))
    first, other, second = requests["r0"], requests["r1"], requests["r2"]
    _, model = load_model(folders[name], dtype=dtype, device=DEV)
    runner = ModelRunner(model, block_size=16, block_capacity=12, num_state_slots=4)

    def decode(request_id, tokens, start):
        rows = []
        for position in range(start, len(tokens)):
            rows.append(runner.step([StepEntry(request_id, [tokens[position]], [0])])[0].cpu().clone())
        return torch.stack(rows)

    runner.begin("a")
    runner.step([StepEntry("a", first[:17], [])])
    got_first = decode("a", first, 17)                  # captured here, with the table of the first lease
    pages_before = [list(t) for t in runner.cache.request("a").tables]
    runner.end("a")
    runner.begin("other")
    runner.step([StepEntry("other", other, [])])        # takes the pages that were given back
    runner.begin("a")
    runner.step([StepEntry("a", second[:17], [])])
    assert [list(t) for t in runner.cache.request("a").tables] != pages_before
    replays = runner.graph_replays
    got_second = decode("a", second, 17)
    assert runner.graph_replays == replays + len(second) - 17
    for got, tokens in ((got_first, first), (got_second, second)):
        want = plain.forward(weights, config, tokens)[17:]
        scale = float(want.abs().max())
        bound = 1e-4 * scale if dtype == "float32" else ru.BF16_FRACTION * scale
        assert float((got - want).abs().max()) <= bound
