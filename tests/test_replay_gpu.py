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
def test_mixed_replay_reuses_pages(dtype, folders, plain_cache, tmp_path):
    requests = ru.make_requests(TINY["B"], 4, (30, 50, 20, 64, 33, 12, 41, 90, 5))
    trace = ru.trace_mixed(requests, 9, max_live=4)
    assert sum(ru.round64(len(t)) for t in requests.values()) > trace.peak_tokens
    got = ru.run_trace(folders["B"], dtype, trace, tmp_path, block_size=8)
    ru.compare(got, expected("B", folders, plain_cache, requests), dtype)


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
