"""The step function, the cache manager and trace replay with the kernels'
plain references patched in: checks on the CPU that logits do not depend on how
requests are cut into steps, batched, or placed in pages.  The kernels
themselves are covered by the GPU tests."""

from __future__ import annotations

import pytest

import kernel_refs
import replay_util as ru
from conftest import BLOCK_SIZE, TINY
from forge_engine_amd.config import load_model_config
from forge_engine_amd.weights import write_random_model

LENGTHS = {"A": (5, 11, 17, 40), "B": (1, 7, 23, 40, 66)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}
    for name in ("A", "B"):
        folder = tmp_path_factory.mktemp(f"tiny_{name}")
        write_random_model(load_model_config(TINY[name]), 11, folder)
        made[name] = folder
    return made


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_replay_matches_plain(name, mode, folders, tmp_path, monkeypatch):
    kernel_refs.install(monkeypatch)
    requests = ru.make_requests(TINY[name], 3, LENGTHS[name])
    trace = {"whole": ru.trace_whole, "tail": lambda r: ru.trace_tail(r, 8),
             "portions": ru.trace_portions, "mixed": lambda r: ru.trace_mixed(r, 5, max_live=3)}[mode](requests)
    got = ru.run_trace(folders[name], "float32", trace, tmp_path, block_size=BLOCK_SIZE[name],
                       device="cpu", on_cpu=True)
    ru.compare(got, ru.plain_logits(folders[name], requests), "float32")


def test_mixed_trace_reuses_pages(folders, tmp_path, monkeypatch):
    kernel_refs.install(monkeypatch)
    requests = ru.make_requests(TINY["A"], 4, (30, 50, 20, 64, 33, 12, 41))
    trace = ru.trace_mixed(requests, 9, max_live=4)
    assert sum(ru.round64(len(t)) for t in requests.values()) > trace.peak_tokens  # pool smaller than the total
    got = ru.run_trace(folders["A"], "float32", trace, tmp_path, block_size=4, device="cpu", on_cpu=True)
    ru.compare(got, ru.plain_logits(folders["A"], requests), "float32")


def test_replay_writes_each_steps_block_tables(folders, tmp_path, monkeypatch):
    import json
    kernel_refs.install(monkeypatch)
    requests = ru.make_requests(TINY["A"], 6, (9, 6))
    trace = ru.TraceBuilder()
    trace.step([("r0", requests["r0"][:5])])
    trace.step([("r0", requests["r0"][5:]), ("r1", requests["r1"])], end=["r0"])
    trace.step([("r1", [7])], end=["r1"])
    ru.run_trace(folders["A"], "float32", trace, tmp_path, block_size=4, max_tokens=128, device="cpu", on_cpu=True)
    steps = [json.loads((tmp_path / f"{i}.json").read_text()) for i in range(3)]
    assert steps[0]["tables"] == {"r0": {"length": 5, "pages": [[0, 1]]}}
    assert steps[1]["tables"] == {"r0": {"length": 9, "pages": [[0, 1, 2]]}, "r1": {"length": 6, "pages": [[3, 4]]}}
    assert steps[2]["tables"] == {"r1": {"length": 7, "pages": [[3, 4]]}}     # r0's pages went back after step 1
    assert steps[1]["rows"] == [["r0", p] for p in range(5, 9)] + [["r1", p] for p in range(6)]
