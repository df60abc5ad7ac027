"""Trace replay on the GPU against the plain implementation, in float32 and in
bfloat16: each request alone and whole; most of it in one step and the last 32
tokens one by one; in portions of changing size down to two tokens; and mixed,
up to four live requests with so few pages that they are used again."""

from __future__ import annotations

import json
import os
import subprocess
import sys
from pathlib import Path

import pytest

import replay_util as ru
from conftest import BLOCK_SIZE, ROOT, TINY
from forge_engine_amd.config import load_model_config
from forge_engine_amd.weights import write_random_model

pytestmark = pytest.mark.gpu

LENGTHS = {"A": (5, 11, 17, 40, 97), "B": (1, 7, 23, 40, 66, 150), "C": (3, 40, 129, 70, 200)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}
    for name in TINY:
        folder = tmp_path_factory.mktemp(f"tiny_{name}")
        write_random_model(load_model_config(TINY[name]), 21, folder)
        made[name] = folder
    return made


@pytest.fixture(scope="module")
def plain_cache():
    return {}


def expected(name, folders, cache, requests):
    key = (name, tuple(sorted((k, tuple(v)) for k, v in requests.items())))
    if key not in cache:
        cache[key] = ru.plain_logits(folders[name], requests)
    return cache[key]


TRACES = {
    "whole": ru.trace_whole,
    "tail": lambda r: ru.trace_tail(r, 32),
    "portions": ru.trace_portions,
    "mixed": lambda r: ru.trace_mixed(r, 5, max_live=4),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", list(TRACES))
def test_replay_matches_plain(name, mode, dtype, folders, plain_cache, tmp_path):
    requests = ru.make_requests(TINY[name], 3, LENGTHS[name])
    trace = TRACES[mode](requests)
    print(f"replay {name} {mode} {dtype}: {len(trace.steps)} steps, pool for {trace.peak_tokens} tokens", flush=True)
    got = ru.run_trace(folders[name], dtype, trace, tmp_path, block_size=BLOCK_SIZE[name])
    worst = ru.compare(got, expected(name, folders, plain_cache, requests), dtype)
    print(f"  worst difference {worst:.3e}", flush=True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_of_long_requests_whose_block_tables_cross_64_and_128_pages(dtype, folders, tmp_path):
    """The lengths at which benchmarks run and no tiny trace arrives: a request of 2,608 tokens fed
    as 2,048 + 500 and then token by token, beside one of 1,100 tokens fed as 1,000 and then token by
    token.  The block tables pass 64 pages (the second of the captured decode steps' table widths),
    128 and 160; the decode attention takes 16 key splits and then 24 (the merge in one round, and
    the merge in a loop); the prefill attention walks 32 key tiles.  Every position's logits are
    compared with the plain implementation."""
    name = "C"
    requests = ru.make_requests(TINY[name], 17, (2608, 1100))
    long, grow = requests["r0"], requests["r1"]
    trace = ru.TraceBuilder()
    trace.step([("r0", long[:2048])])
    trace.step([("r1", grow[:1000])])
    trace.step([("r0", long[2048:2548])])
    for i in range(100):                       # both decode; the shorter one ends after 100 tokens, the longer after 60
        parts = [("r1", grow[1000 + i:1001 + i])]
        if i < 60:
            parts.append(("r0", long[2548 + i:2549 + i]))
        trace.step(parts, end=[r for r, last in (("r0", 59), ("r1", 99)) if i == last])
    print(f"long replay {dtype}: {len(trace.steps)} steps, pool for {trace.peak_tokens} tokens", flush=True)
    got = ru.run_trace(folders[name], dtype, trace, tmp_path, block_size=BLOCK_SIZE[name])
    tables = [json.loads((tmp_path / f"{i}.json").read_text())["tables"] for i in range(len(trace.steps))]
    assert len(tables[3]["r1"]["pages"][0]) == 63 and len(tables[30]["r1"]["pages"][0]) == 65     # crosses 64 pages while decoding
    assert len(tables[3]["r0"]["pages"][0]) == 160 and len(tables[62]["r0"]["pages"][0]) == 163
    worst = ru.compare(got, ru.plain_logits(folders[name], requests), dtype)
    print(f"  worst difference {worst:.3e}", flush=True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", list(TRACES))
def test_replay_of_the_reference_tiny_configuration(mode, dtype, tmp_path):
    """The configuration of the reference's own model tests: two query heads of four elements over
    one kv head, a width of eight (every product and head size below the kernels' vector widths)."""
    from conftest import TINY_R
    folder = tmp_path / "model"
    write_random_model(load_model_config(TINY_R), 77, folder)
    requests = ru.make_requests(TINY_R, 5, (3, 7, 30, 61, 12))
    got = ru.run_trace(folder, dtype, TRACES[mode](requests), tmp_path / "out", block_size=2)
    ru.compare(got, ru.plain_logits(folder, requests), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_replay_reuses_pages(dtype, folders, plain_cache, tmp_path):
    requests = ru.make_requests(TINY["B"], 4, (30, 50, 20, 64, 33, 12, 41, 90, 5))
    trace = ru.trace_mixed(requests, 9, max_live=4)
    assert sum(ru.round64(len(t)) for t in requests.values()) > trace.peak_tokens
    got = ru.run_trace(folders["B"], dtype, trace, tmp_path, block_size=8)
    ru.compare(got, expected("B", folders, plain_cache, requests), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_swapped_pages_of_one_layer_are_seen_in_both_dtypes(name, dtype, folders, plain_cache):
    """The control of the comparisons above: two requests are fed all but their last eight tokens,
    then one page of one layer changes places with a page of the other request (as a wrong entry
    in that layer's block table would have it), and the last tokens are decoded.  The comparison
    with the plain implementation must fail, in bfloat16 at its own bound too; without the swap
    the same steps pass."""
    import torch
    from forge_engine_amd.engine import ModelRunner, StepEntry, load_model

    requests = ru.make_requests(TINY[name], 3, (70, 90))
    want = expected(name, folders, plain_cache, requests)
    _, model = load_model(folders[name], dtype=dtype, device="cuda:0")
    for layer in (None, 0, len(model.schedule) - 1):
        runner = ModelRunner(model, block_size=BLOCK_SIZE[name], block_capacity=64, num_state_slots=4)
        for request_id, tokens in requests.items():
            runner.begin(request_id)
            runner.step([StepEntry(request_id, tokens[:-8], [])])
        if layer is not None:
            mine = runner.cache.request("r0").tables[0][1]
            theirs = runner.cache.request("r1").tables[0][2]
            for pages in (runner.key_pages[0][layer], runner.value_pages[0][layer]):
                kept = pages[mine].clone()
                pages[mine].copy_(pages[theirs])
                pages[theirs].copy_(kept)
        got = {}
        for i in range(8):
            entries = [StepEntry(r, [t[len(t) - 8 + i]], [0]) for r, t in requests.items()]
            logits = runner.step(entries).cpu()
            for row, (request_id, tokens) in zip(logits, requests.items()):
                got[(request_id, len(tokens) - 8 + i)] = row.clone()
        torch.cuda.synchronize()
        tail = {key: want[key] for key in got}
        if layer is None:
            ru.compare(got, tail, dtype)
        else:
            with pytest.raises(AssertionError, match="logits differ"):
                ru.compare(got, tail, dtype)


def test_trace_run_program(folders, tmp_path):
    """The program itself, as a child process: protocol, files, exit code."""
    requests = ru.make_requests(TINY["A"], 6, (9, 30))
    trace = ru.trace_mixed(requests, 2, max_live=2)
    lines = "".join(json.dumps(step) + "\n" for step in trace.steps)
    out = tmp_path / "out"
    done = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folders["A"]), "--dtype", "float32",
         "--out", str(out), "--max-tokens", str(trace.peak_tokens)],
        input=lines, capture_output=True, text=True, timeout=300, env=dict(os.environ))
    assert done.returncode == 0, done.stderr[-2000:]
    assert done.stdout.split() == [w for s in trace.steps for w in ("done", str(s["step"]))]
    got = ru.collect(trace, out, TINY["A"]["vocab_size"])
    ru.compare(got, ru.plain_logits(folders["A"], requests), "float32")


def _drawn_configuration(seed: int):
    """A small configuration whose every size is drawn: head sizes from 16 to 256, any group
    size, widths and vocabularies that are no power of two, bias or not, tied or not."""
    import random
    rng = random.Random(1000 + seed)
    kv = rng.choice([1, 2, 3, 4])
    groups = rng.choice([1, 2, 3, 4, 5, 7, 8, 9])
    config = {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_act": "silu",
        "vocab_size": rng.choice([97, 256, 300, 1003, 2049]), "hidden_size": rng.choice([40, 64, 72, 136, 200, 264]),
        "intermediate_size": rng.choice([48, 128, 136, 328, 520]), "num_hidden_layers": rng.choice([1, 2, 3]),
        "num_attention_heads": kv * groups, "num_key_value_heads": kv,
        "head_dim": rng.choice([16, 32, 48, 64, 64, 80, 96, 128, 128, 160, 256]) if seed < 100 else rng.choice([2, 4, 6, 10, 12, 20, 36, 100]),
        "max_position_embeddings": 512, "rms_norm_eps": rng.choice([1e-6, 1e-5, 1e-3]),
        "rope_theta": rng.choice([10000.0, 1e6, 5e6]), "tie_word_embeddings": rng.choice([True, False]),
        "attention_bias": rng.choice([False, False, True]), "eos_token_id": None,
    }
    block_size = rng.choice([4, 8, 16, 16, 32, 64])
    lengths = tuple(rng.choice([1, 2, 3, 17, 33, 40, 64, 65, 100, 150]) for _ in range(rng.randrange(3, 6)))
    return config, block_size, lengths


@pytest.mark.parametrize("seed", [1, 6, 12, 13, 24, 47, 74, 101, 102, 103])      # from 100 on: head sizes that are no multiple of 16
def test_replay_of_drawn_configurations(seed, tmp_path):
    """Configurations nobody chose by hand, every way of cutting, both dtypes."""
    config, block_size, lengths = _drawn_configuration(seed)
    folder = tmp_path / "model"
    write_random_model(load_model_config(config), 50 + seed, folder)
    requests = ru.make_requests(config, seed, lengths)
    want = ru.plain_logits(folder, requests)
    for dtype in ("float32", "bfloat16"):
        for mode, make in TRACES.items():
            got = ru.run_trace(folder, dtype, make(requests), tmp_path / f"{dtype}_{mode}", block_size=block_size)
            ru.compare(got, want, dtype)
