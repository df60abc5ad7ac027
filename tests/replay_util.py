"""Helpers of the replay tests: traces that cut the same requests in different
ways, a runner for them, and the comparison with the plain implementation."""

from __future__ import annotations

import io
import json
import random
from argparse import Namespace
from pathlib import Path

import numpy as np
import torch
from safetensors.torch import load_file

import plain_qwen3 as plain


def make_requests(config: dict, seed: int, lengths) -> dict[str, list[int]]:
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(config["vocab_size"]) for _ in range(n)]
            for i, n in enumerate(lengths)}


def round64(n: int) -> int:
    return (n + 63) // 64 * 64


class TraceBuilder:
    """Collects steps; remembers which (request, position) each output row is."""

    def __init__(self, want_all: bool = True) -> None:
        self.want_all = want_all          # logits at every token of a step, or only at each entry's last
        self.steps: list[dict] = []
        self.rows: dict[int, list[tuple[str, int]]] = {}
        self.fed: dict[str, int] = {}
        self.peak_tokens = 0

    def step(self, parts: list[tuple[str, list[int]]], end=(), want_all: bool | None = None) -> None:
        want_all = self.want_all if want_all is None else want_all
        index = len(self.steps)
        entries, rows = [], []
        for request_id, tokens in parts:
            start = self.fed.get(request_id, 0)
            want = list(range(len(tokens))) if want_all else [len(tokens) - 1]
            entries.append({"id": request_id, "tokens": tokens, "want": want})
            rows.extend((request_id, start + w) for w in want)
            self.fed[request_id] = start + len(tokens)
        self.peak_tokens = max(self.peak_tokens, sum(round64(n) for n in self.fed.values()))
        for request_id in end:
            del self.fed[request_id]
        self.steps.append({"step": index, "entries": entries, "end": list(end)})
        self.rows[index] = rows


def trace_whole(requests) -> TraceBuilder:
    """Each request alone, whole, in one step."""
    trace = TraceBuilder()
    for request_id, tokens in requests.items():
        trace.step([(request_id, tokens)], end=[request_id])
    return trace


def trace_tail(requests, tail: int = 32) -> TraceBuilder:
    """Most of a request in one step, its last ``tail`` tokens one by one."""
    trace = TraceBuilder()
    for request_id, tokens in requests.items():
        head = max(1, len(tokens) - tail)
        trace.step([(request_id, tokens[:head])], end=[request_id] if head == len(tokens) else [])
        for i in range(head, len(tokens)):
            trace.step([(request_id, tokens[i:i + 1])], end=[request_id] if i == len(tokens) - 1 else [])
    return trace


def trace_portions(requests, sizes=(16, 7, 5, 3, 2, 2, 9, 2, 4), want_all: bool = True) -> TraceBuilder:
    """Portions of changing size, down to two tokens."""
    trace = TraceBuilder(want_all)
    for n, (request_id, tokens) in enumerate(requests.items()):
        at, k = 0, n  # each request starts elsewhere in the size cycle
        while at < len(tokens):
            size = min(sizes[k % len(sizes)], len(tokens) - at)
            k += 1
            last = at + size >= len(tokens)
            trace.step([(request_id, tokens[at:at + size])], end=[request_id] if last else [])
            at += size
    return trace


def trace_mixed(requests, seed: int, max_live: int = 4, prompt_fraction: float = 0.6,
                want_all: bool = True, portion_sizes=(2, 3, 5, 8, 13)) -> TraceBuilder:
    """Up to ``max_live`` requests at a time: portions of the prompts of some
    beside single decoded tokens of others; a request may sit a step out; when
    one ends the next is admitted, so its pages are used again."""
    rng = random.Random(seed)
    trace = TraceBuilder(want_all)
    waiting = list(requests.items())
    live: dict[str, dict] = {}
    while waiting or live:
        while waiting and len(live) < max_live:
            request_id, tokens = waiting.pop(0)
            live[request_id] = {"tokens": tokens, "at": 0,
                                "prompt": max(1, int(len(tokens) * prompt_fraction))}
        parts, ended = [], []
        chosen = [r for r in live if rng.random() < 0.8] or [next(iter(live))]
        for request_id in chosen:
            state = live[request_id]
            tokens, at = state["tokens"], state["at"]
            if at < state["prompt"]:
                size = min(rng.choice(portion_sizes), state["prompt"] - at)
            else:
                size = 1
            parts.append((request_id, tokens[at:at + size]))
            state["at"] = at + size
            if state["at"] >= len(tokens):
                ended.append(request_id)
        trace.step(parts, end=ended)
        for request_id in ended:
            del live[request_id]
    return trace


def run_trace(model_dir, dtype: str, trace: TraceBuilder, out_dir, *, block_size: int,
              max_tokens: int | None = None, device: str = "cuda:0", on_cpu: bool = False):
    """Replay in-process through the replay module; returns
    {(request, position): logits row}.  ``on_cpu``: the caller has patched the kernels' plain
    references in and the model runs on the CPU."""
    from forge_engine_amd import replay

    out_dir = Path(out_dir)
    stdin = io.StringIO("".join(json.dumps(step) + "\n" for step in trace.steps))
    stdout = io.StringIO()
    args = Namespace(model=str(model_dir), dtype=dtype, out=str(out_dir), block_size=block_size,
                     max_tokens=trace.peak_tokens if max_tokens is None else max_tokens, device=device)
    assert replay.run(args, stdin=stdin, stdout=stdout, device="cpu" if on_cpu else None) == 0
    assert stdout.getvalue().split() == [w for s in trace.steps for w in ("done", str(s["step"]))]
    return collect(trace, out_dir, json.loads((Path(model_dir) / "config.json").read_text())["vocab_size"])


def collect(trace: TraceBuilder, out_dir, vocab: int):
    got = {}
    for index, rows in trace.rows.items():
        if not rows:
            continue
        data = np.fromfile(str(Path(out_dir) / f"{index}.f32"), dtype="<f4").reshape(len(rows), vocab)
        layout = json.loads((Path(out_dir) / f"{index}.json").read_text())
        assert [tuple(row) for row in layout["rows"]] == rows, "the step's own account of its rows differs"
        for row, key in zip(data, rows):
            got[key] = torch.from_numpy(row.copy())
    return got


def plain_logits(model_dir, requests, only=None) -> dict[tuple[str, int], torch.Tensor]:
    """The plain implementation on the folder's own tensors (widened to float32).  ``only``: the
    (request, position) pairs that are wanted (default: every position)."""
    config = json.loads((Path(model_dir) / "config.json").read_text())
    weights = {k: v.float() for k, v in load_file(str(Path(model_dir) / "model.safetensors")).items()}
    want = {}
    for request_id, tokens in requests.items():
        if only is None:
            positions = list(range(len(tokens)))
        else:
            positions = sorted(position for rid, position in only if rid == request_id)
        logits = plain.forward(weights, config, tokens, rows=positions)
        for row, position in zip(logits, positions):
            want[(request_id, position)] = row
    return want


# Tolerances.  float32: the engine and the plain implementation differ only in
# the order of float32 sums (1e-5, the reference's own bound for cached against
# uncached logits, tests/test_generation_core.py:77-82).  bfloat16: activations
# between kernels are rounded to 8 mantissa bits (2^-9 relative, half a dozen
# roundings a layer, adding up like a random walk); the bound is a fraction of
# the largest logit of the comparison.  The worst difference seen over every
# test of the suite is 0.5 % of that; one page of one layer swapped between two
# requests moves the logits by 3 % to 50 %
# (test_swapped_pages_of_one_layer_are_seen_in_both_dtypes), so the bound sits
# between the two, three times above the first.
F32_ATOL, F32_RTOL = 1e-5, 1e-4
BF16_FRACTION = 0.015


def compare(got: dict, want: dict, dtype: str) -> float:
    assert set(got) == set(want), "replay did not return every wanted row"
    worst = 0.0
    scale = max(float(v.abs().max()) for v in want.values())
    for key in sorted(want):
        g, w = got[key], want[key]
        assert torch.isfinite(g).all(), f"non-finite logits at {key}"
        diff = float((g - w).abs().max())
        if dtype == "float32":
            bound = F32_ATOL + F32_RTOL * float(w.abs().max())
        else:
            bound = BF16_FRACTION * scale
        assert diff <= bound, f"{dtype} logits differ at {key}: {diff:.3e} > {bound:.3e}"
        worst = max(worst, diff)
    return worst
