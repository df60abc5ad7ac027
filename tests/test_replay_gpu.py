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
        "head_dim": rng.choice([16, 32, 48, 64, 64, 80, 96, 128, 128, 160, 256]),
        "max_position_embeddings": 512, "rms_norm_eps": rng.choice([1e-6, 1e-5, 1e-3]),
        "rope_theta": rng.choice([10000.0, 1e6, 5e6]), "tie_word_embeddings": rng.choice([True, False]),
        "attention_bias": rng.choice([False, False, True]), "eos_token_id": None,
    }
    block_size = rng.choice([4, 8, 16, 16, 32, 64])
    lengths = tuple(rng.choice([1, 2, 3, 17, 33, 40, 64, 65, 100, 150]) for _ in range(rng.randrange(3, 6)))
    return config, block_size, lengths


@pytest.mark.parametrize("seed", [1, 6, 12, 13, 24, 47, 74])
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
