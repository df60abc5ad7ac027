"""Sampling parameters and the sampler's routing (CPU); the filters' thresholds against the plain filters.  The draw kernels are
covered by the GPU tests."""

from __future__ import annotations

import pytest
import torch

import kernel_refs
import plain_qwen3 as plain
from forge_engine_amd.config import EngineConfig
from forge_engine_amd.sampling import SamplingParams
from forge_engine_amd.sampling.sampler import Sampler


@pytest.mark.parametrize("kwargs", [
    {"temperature": -0.1}, {"temperature": float("nan")}, {"temperature": float("inf")}, {"top_k": 0},
    {"top_p": 0.0}, {"top_p": 1.5}, {"min_p": -0.1}, {"min_p": 1.1}, {"max_new_tokens": 0},
    {"stop_strings": ("",)}, {"stop_strings": ("a", "a")},
])
def test_invalid_parameters(kwargs):
    with pytest.raises(ValueError):
        SamplingParams(**kwargs)
    with pytest.raises(ValueError):
        EngineConfig(**kwargs)


def test_defaults_follow_the_reference():
    p = SamplingParams()
    assert (p.temperature, p.top_k, p.top_p, p.min_p, p.max_new_tokens, p.stop_strings, p.seed) == (0.0, None, 1.0, 0.0, 256, (), None)
    assert p.greedy and not SamplingParams(temperature=0.5).greedy
    assert EngineConfig(temperature=0.7, seed=3).sampling_params() == SamplingParams(temperature=0.7, seed=3)


def kept(x):
    return torch.isfinite(x).nonzero()[:, 1].tolist()


@pytest.mark.parametrize("seed", range(5))
def test_the_kernel_reference_keeps_what_the_plain_filters_keep(seed):
    """The thresholds that the sampling kernel is tested against (kernel_refs.kept_after_filters)
    against the filters written from the reference's text, on rows without equal logits."""
    g = torch.Generator().manual_seed(100 + seed)
    logits = torch.randn(6, 300, generator=g) * 3
    for t, k, p, m in ((0.7, 5, 1.0, 0.0), (1.3, None, 0.6, 0.0), (0.9, None, 1.0, 0.1), (0.5, 20, 0.8, 0.05), (1.0, 1, 1.0, 0.0),
                       (1.1, 200, 0.95, 0.0), (2.0, 50, 0.3, 0.0)):
        want = torch.isfinite(plain.filter_logits(logits, t, k, p, m))
        for r in range(logits.shape[0]):
            _, kept = kernel_refs.kept_after_filters(logits[r], t, k or 0, p, m)
            assert torch.equal(kept, want[r]), (t, k, p, m, r)


def test_sample_parameters_are_packed_as_the_kernel_reads_them():
    from forge_engine_amd.kernels import ops
    packed = ops.pack_sample_params([(0.5, None, 1.0, 0.0, 2**64 - 1, 5), (0.0, 40, 0.9, 0.05, 7, 2**40 + 3)])
    assert packed.shape == (2, ops.SAMPLE_PARAM_WORDS) and packed.dtype == torch.int32
    rows = kernel_refs.unpack_sample_params(packed)
    assert rows[0] == (0.5, 0, 1.0, 0.0, 2**64 - 1, 5)
    assert rows[1][0] == 0.0 and rows[1][1] == 40 and abs(rows[1][2] - 0.9) < 1e-6 and rows[1][4:] == (7, 2**40 + 3)


def test_sampler_routes_rows_and_raises_on_bad_logits(monkeypatch):
    kernel_refs.install(monkeypatch)
    sampler = Sampler(torch.device("cpu"))
    logits = torch.tensor([[1.0, 3.0, 2.0], [7.0, -1.0, 4.0], [0.0, 0.0, 9.0]])
    greedy = SamplingParams()
    assert sampler.sample(logits[:2], [greedy, greedy], [0, 0], [0, 0]) == [1, 0]    # reference tests/test_sampling.py:40-45
    only_top = SamplingParams(temperature=1.0, top_k=1)
    assert sampler.sample(logits, [greedy, only_top, SamplingParams(temperature=1e-3)], [1, 2, 3], [0, 0, 0]) == [1, 0, 2]
    for bad, match in (([[0.0, float("nan")]], "NaN"), ([[float("-inf")] * 2], "finite"), ([[0.0, float("inf")]], "positive infinity")):
        with pytest.raises(ValueError, match=match):
            sampler.sample(torch.tensor(bad), [greedy], [0], [0])
        with pytest.raises(ValueError, match=match):
            sampler.sample(torch.tensor(bad), [only_top], [0], [0])


def test_uniform_logits_give_uniform_draws(monkeypatch):
    kernel_refs.install(monkeypatch)
    sampler = Sampler(torch.device("cpu"))
    p = SamplingParams(temperature=1.0)
    draws = [sampler.sample(torch.zeros(1, 8), [p], [731], [i])[0] for i in range(400)]
    counts = torch.bincount(torch.tensor(draws), minlength=8)
    assert counts.min() > 25 and counts.max() < 80
    assert draws == [sampler.sample(torch.zeros(1, 8), [p], [731], [i])[0] for i in range(400)]
