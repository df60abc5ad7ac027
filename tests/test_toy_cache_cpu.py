"""What a mixer may ask of the cache beyond keys and values of one width, shown with a toy mixer
defined here (plain torch ops on the CPU, with the kernels' references patched in for the built-in
parts): a mixer that keeps keys only gets no value pages, one whose values are wider than its keys
gets value pages of that width, and the two form cache groups of their own.  And the scheduler's
admission with a page capacity per cache group."""

from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar

import pytest
import torch

import kernel_refs
import plain_qwen3 as plain
from forge_engine_amd.cache import CacheGroup, CacheManager, CacheNeeds, FixedState, PagedKV
from forge_engine_amd.config import SchedulerConfig, load_model_config
from forge_engine_amd.config.model import KeyReader, ModelConfig
from forge_engine_amd.engine import ConcurrentGenerationEngine, ModelRunner, OverloadedError, StepEntry, build_model
from forge_engine_amd.parts import LayerCall, LayerSpec, Mixer, ModelPlan, ParamSpec, PartSpec
from forge_engine_amd.registry import register_architecture, register_part
from forge_engine_amd.sampling import SamplingParams
from forge_engine_amd.weights import fill_random_weights


class RunningMeanMixer(Mixer):
    """update_t = W_o [mean_{j <= t} k_j ; mean_{j <= t} v_j] with k = W_k x (``key_dim`` wide per
    head) and, if ``value_dim`` > 0, v = W_v x (``value_dim`` wide per head).  Keys and values live
    in the pages that the cache manager leases, and every step reads them back through the block
    table, so any cut of a request into steps gives the same result."""

    graph_safe = False

    def __init__(self, ctx, prefix, *, hidden_size: int, heads: int, key_dim: int, value_dim: int) -> None:
        super().__init__(ctx, prefix)
        self.hidden_size, self.heads, self.key_dim, self.value_dim = hidden_size, heads, key_dim, value_dim
        self.weights = {}

    def param_specs(self):
        specs = {self.name("k.weight"): ParamSpec((self.heads * self.key_dim, self.hidden_size)),
                 self.name("o.weight"): ParamSpec((self.hidden_size, self.heads * (self.key_dim + self.value_dim)))}
        if self.value_dim:
            specs[self.name("v.weight")] = ParamSpec((self.heads * self.value_dim, self.hidden_size))
        return specs

    def set_param(self, name, tensor):
        self.weights[name[len(self.prefix) + 1:]] = tensor.float()

    def cache_needs(self):
        return CacheNeeds(paged=PagedKV(self.heads, self.key_dim, value_dim=self.value_dim))

    def forward(self, x, batch, cache, writes_cache=True):
        assert (cache.value_pages is None) == (self.value_dim == 0)
        xf = x.float()
        keys = (xf @ self.weights["k.weight"].T).view(-1, self.heads, self.key_dim)
        values = (xf @ self.weights["v.weight"].T).view(-1, self.heads, self.value_dim) if self.value_dim else None
        size = cache.block_size
        out = torch.empty((x.shape[0], self.hidden_size), dtype=torch.float32)
        at = 0
        for i, count in enumerate(batch.q_lens):
            table = cache.block_table[i].tolist()
            for t in range(count):
                position = batch.ctx_before_host[i] + t
                page, slot = table[position // size], position % size
                cache.key_pages[page, :, slot] = keys[at + t].to(cache.key_pages.dtype)
                if values is not None:
                    cache.value_pages[page, :, :, slot] = values[at + t].to(cache.value_pages.dtype)   # values lie transposed
                held = position + 1
                pages = torch.tensor(table[:-(-held // size)])
                mean = cache.key_pages[pages].float().transpose(0, 1).reshape(self.heads, -1, self.key_dim)[:, :held].mean(1)
                parts = [mean.reshape(-1)]
                if values is not None:
                    seen = cache.value_pages[pages].float().permute(1, 2, 0, 3).reshape(self.heads, self.value_dim, -1)[:, :, :held]
                    parts.append(seen.mean(2).reshape(-1))
                out[at + t] = self.weights["o.weight"] @ torch.cat(parts)
            at += count
        return out


@dataclass(frozen=True)
class MeanConfig(ModelConfig):
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    heads: int
    key_dim: int
    value_dim: int
    rms_norm_eps: float
    architecture: ClassVar[str] = "ToyRunningMeanLM"

    @classmethod
    def from_dict(cls, raw):
        read = KeyReader(raw)
        return cls(*(read.integer(k) for k in ("vocab_size", "hidden_size", "intermediate_size", "heads", "key_dim", "value_dim")),
                   read.number("rms_norm_eps"))


def mean_plan(config: MeanConfig) -> ModelPlan:
    def norm(prefix):
        return PartSpec("rms_norm", {"size": config.hidden_size, "eps": config.rms_norm_eps}, prefix)

    def layer(index, value_dim):
        prefix = f"model.layers.{index}"
        mixer = PartSpec("toy_running_mean", {"hidden_size": config.hidden_size, "heads": config.heads,
                                              "key_dim": config.key_dim, "value_dim": value_dim}, f"{prefix}.mean")
        return LayerSpec("pre_norm", mixer,
                         PartSpec("swiglu", {"hidden_size": config.hidden_size, "intermediate_size": config.intermediate_size}, f"{prefix}.mlp"),
                         {"input": norm(f"{prefix}.input_layernorm"), "post_mixer": norm(f"{prefix}.post_attention_layernorm")})

    sizes = {"vocab_size": config.vocab_size, "hidden_size": config.hidden_size}
    # keys only; keys and wider values; keys only again (the same group as the first)
    layers = (layer(0, 0), layer(1, config.value_dim), layer(2, 0))
    return ModelPlan(config.hidden_size, config.vocab_size, PartSpec("token_embedding", dict(sizes), "model.embed_tokens"),
                     layers, tuple(LayerCall(i) for i in range(3)), norm("model.norm"),
                     PartSpec("lm_head", dict(sizes, tied=True), "lm_head"))


def mean_plain_forward(w, config: MeanConfig, tokens):
    h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    counts = torch.arange(1, len(tokens) + 1, dtype=torch.float32)[:, None]
    for index, value_dim in enumerate((0, config.value_dim, 0)):
        p = f"model.layers.{index}"
        x = plain.rms_norm(h, w[f"{p}.input_layernorm.weight"], config.rms_norm_eps)
        means = [((x @ w[f"{p}.mean.k.weight"].T).cumsum(0) / counts)]
        if value_dim:
            means.append((x @ w[f"{p}.mean.v.weight"].T).cumsum(0) / counts)
        update = torch.cat(means, dim=1) @ w[f"{p}.mean.o.weight"].T
        h, y = plain.add_rms_norm(h, update, w[f"{p}.post_attention_layernorm.weight"], config.rms_norm_eps)
        h = h + plain.swiglu_mlp(y, w, f"{p}.mlp")
    return plain.rms_norm(h, w["model.norm.weight"], config.rms_norm_eps) @ w["model.embed_tokens.weight"].T


RAW = {"architectures": ["ToyRunningMeanLM"], "vocab_size": 50, "hidden_size": 24, "intermediate_size": 40,
       "heads": 2, "key_dim": 8, "value_dim": 12, "rms_norm_eps": 1e-5}


def test_a_mixer_may_keep_keys_only_or_values_of_another_width(monkeypatch):
    kernel_refs.install(monkeypatch)
    register_part("mixer", "toy_running_mean", RunningMeanMixer, replace=True)
    register_architecture("ToyRunningMeanLM", MeanConfig, mean_plan, replace=True)
    config = load_model_config(RAW)
    model = build_model(config, dtype="float32", device="cpu")
    fill_random_weights(model, 3, device=torch.device("cpu"), dtype=torch.float32)
    runner = ModelRunner(model, block_size=4, block_capacity=[12, 8], num_state_slots=2)
    groups = runner.cache.groups
    assert [(g.value_width, g.slots) for g in groups] == [(0, (0, 2)), (12, (1,))]
    assert runner.value_pages[0] is None and runner.key_pages[0].shape == (2, 12, 2, 4, 8)
    assert runner.value_pages[1].shape == (1, 8, 2, 12, 4) and runner.key_pages[1].shape == (1, 8, 2, 4, 8)
    w = {}
    for index in range(3):
        block, p = model.layers[index], f"model.layers.{index}"
        w[f"{p}.input_layernorm.weight"] = block.norms["input"].weight
        w[f"{p}.post_attention_layernorm.weight"] = block.norms["post_mixer"].weight
        w[f"{p}.mlp.gate_proj.weight"] = block.feed_forward.gate_up_weight[:config.intermediate_size]
        w[f"{p}.mlp.up_proj.weight"] = block.feed_forward.gate_up_weight[config.intermediate_size:]
        w[f"{p}.mlp.down_proj.weight"] = block.feed_forward.down_weight
        for name, tensor in block.mixer.weights.items():
            w[f"{p}.mean.{name}"] = tensor
    w["model.embed_tokens.weight"] = model.embedding.weight
    w["model.norm.weight"] = model.final_norm.weight
    g = torch.Generator().manual_seed(4)
    requests = {name: torch.randint(0, 50, (n,), generator=g).tolist() for name, n in (("a", 19), ("b", 7), ("c", 22))}
    got = {name: [] for name in requests}
    for live in (("a", "b"), ("c",)):                 # the third request takes the pages that the first two gave back
        at = {name: 0 for name in live}
        for name in live:
            runner.begin(name)
        step = 0
        while any(at[n] < len(requests[n]) for n in live):
            entries = []
            for name in live:
                left = len(requests[name]) - at[name]
                if left <= 0:
                    continue
                size = min(left, (5, 1, 3, 1, 2)[(step + len(name)) % 5] if left > 4 else 1)
                entries.append(StepEntry(name, requests[name][at[name]:at[name] + size], list(range(size))))
                at[name] += size
            logits = runner.step(entries)
            row = 0
            for entry in entries:
                got[entry.request_id].append(logits[row:row + len(entry.tokens)])
                row += len(entry.tokens)
            step += 1
        for name in live:
            runner.end(name)
        runner.cache.check_invariants()
        assert runner.cache.allocated_pages == 0
    for name, tokens in requests.items():
        torch.testing.assert_close(torch.cat(got[name]), mean_plain_forward(w, config, tokens), atol=1e-5, rtol=1e-4)


def test_states_by_name_and_groups_by_value_width():
    one = CacheNeeds(state=FixedState((3,)))
    assert list(one.states()) == ["state"] and CacheNeeds().states() == {}
    two = CacheNeeds(state={"recurrent": FixedState((4, 4), torch.float32), "tail": FixedState((3, 8), torch.bfloat16)})
    assert {k: (v.shape, v.dtype) for k, v in two.states().items()} == {
        "recurrent": ((4, 4), torch.float32), "tail": ((3, 8), torch.bfloat16)}
    assert PagedKV(2, 8).value_width == 8 and PagedKV(2, 8, value_dim=0).value_width == 0


class PagesOnlyRunner:
    """What the scheduler asks of a runner, over a real cache manager and no model: a step leases
    and commits pages and returns logits that make every request sample token 1."""

    class _Plan:
        vocab_size = 16
        eos_token_ids = frozenset()

    class _Model:
        pass

    def __init__(self, cache: CacheManager) -> None:
        self.cache = cache
        self.model = self._Model()
        self.model.plan = self._Plan()

    def begin(self, request_id):
        self.cache.begin(request_id)

    def end(self, request_id):
        self.cache.end(request_id)

    def step(self, entries):
        lengths = {e.request_id: self.cache.length(e.request_id) + len(e.tokens) for e in entries}
        self.cache.reserve(lengths)
        for name, length in lengths.items():
            self.cache.commit(name, length)
        logits = torch.zeros(sum(len(e.want) for e in entries), 16)
        logits[:, 1] = 1.0
        return logits


class ArgmaxSampler:
    def sample(self, logits, params, seeds, draws):
        return logits.argmax(-1).tolist()


def test_admission_reserves_in_every_cache_group_against_that_groups_capacity():
    # group 0 keeps every key, group 1 only a window of 6: a request of 40 tokens holds 10 pages of 4 in
    # the first and at most blocks(6 - 1 + 8) + 1 = 5 in the second, whose pool can therefore be small
    groups = [CacheGroup(0, 1, 8, None, (0,)), CacheGroup(1, 1, 8, 6, (1,))]
    config = SchedulerConfig(block_size=4, block_capacity=(20, 10), token_budget=8, max_batch_size=4, overlap_decode=False)
    cache = CacheManager(groups, block_size=4, block_capacity=[20, 10], num_state_slots=16)
    engine = ConcurrentGenerationEngine(PagesOnlyRunner(cache), ArgmaxSampler(), SamplingParams(), config)
    first = engine.submit([1] * 30, sampling_params=SamplingParams(max_new_tokens=10))
    assert engine.request(first).reserved_blocks == 10 and engine._reserved == [10, 5]
    second = engine.submit([2] * 36, sampling_params=SamplingParams(max_new_tokens=4))
    assert engine._reserved == [20, 10]
    with pytest.raises(OverloadedError, match="only 0 are unreserved"):
        engine.submit([3], sampling_params=SamplingParams(max_new_tokens=1))
    engine.run_until_idle()
    assert engine._reserved == [0, 0] and cache.allocated_pages == 0
    cache.check_invariants()
    assert len(engine.request(first).output_token_ids) == 10 and len(engine.request(second).output_token_ids) == 4
    # the windowed group alone can refuse: three short requests fill its pool while the other has room
    for _ in range(3):
        engine.submit([1] * 9, sampling_params=SamplingParams(max_new_tokens=3))       # 3 pages in each group
    assert engine._reserved == [9, 9]
    with pytest.raises(OverloadedError, match="only 1 are unreserved"):
        engine.submit([1] * 9, sampling_params=SamplingParams(max_new_tokens=3))
    # a scheduler configuration must name the pools as they are
    with pytest.raises(ValueError, match="does not match"):
        ConcurrentGenerationEngine(PagesOnlyRunner(cache), ArgmaxSampler(), SamplingParams(),
                                   SchedulerConfig(block_size=4, block_capacity=20))
    with pytest.raises(ValueError, match="cache groups"):
        SchedulerConfig(block_size=4, block_capacity=(20, 10, 5)).capacities(2)


def test_per_token_inputs_lie_behind_the_block_tables():
    """What a model's parts ask for per token (`token_inputs`) is carried in the step's one buffer,
    name after name: rows that an entry brings, or the token's position on every axis; a captured
    step's buffer has the same places."""
    from forge_engine_amd.engine.batch import BatchLayout, StepEntry, build_batch, static_batch
    entries = [StepEntry("a", [5, 6, 7], [2], {"grid": [[1, 2], [3, 4], [5, 6]]}),
               StepEntry("b", [8], [0]),
               StepEntry("c", [9, 10], [], {"kind": [7, 8]})]
    asked = {"kind": 1, "grid": 2}
    batch = build_batch(entries, [10, 4, 0], [0, 1, 2], [[[3, 4, 5, 6], [1, 2], [0]]], torch.device("cpu"), token_inputs=asked)
    assert batch.inputs["grid"].tolist() == [[1, 2], [3, 4], [5, 6], [4, 4], [0, 0], [1, 1]]
    assert batch.inputs["kind"].tolist() == [[10], [11], [12], [4], [7], [8]]
    assert batch.positions.tolist() == [10, 11, 12, 4, 0, 1]
    assert batch.block_tables[0].tolist() == [[3, 4, 5, 6], [1, 2, -1, -1], [0, -1, -1, -1]]
    layout, bare = BatchLayout.of(6, 3, 2, [4], asked), BatchLayout.of(6, 3, 2, [4])
    assert layout.size == bare.size + 6 * 3 and bare.size == 3 * 6 + 4 * 3 + 1 + 2 + 3 * 4
    assert layout.span(("table", 0)) == bare.span(("table", 0)) == slice(bare.size - 12, bare.size)
    assert layout.span(("input", "grid")) == slice(bare.size, bare.size + 12)       # name after name, in the names' order
    assert layout.span(("input", "kind")) == slice(bare.size + 12, bare.size + 18)
    flat = torch.arange(layout.size, dtype=torch.int32)
    fixed = static_batch(flat, layout, max_q_len=6, max_ctx=16)
    assert fixed.inputs["grid"].shape == (6, 2) and int(fixed.inputs["grid"][0, 0]) == bare.size
    assert fixed.inputs["kind"].shape == (6, 1) and int(fixed.inputs["kind"][5, 0]) == layout.size - 1
    assert fixed.cu_q.tolist() == list(range(18, 22)) and fixed.block_tables[0].shape == (3, 4)
    # a step packed by build_batch lies exactly as the layout says
    packed = BatchLayout.of(6, 3, 1, [4], asked)
    assert packed.size == batch.inputs["kind"].numel() + batch.inputs["grid"].numel() + 3 * 6 + 4 * 3 + 1 + 1 + 12
    with pytest.raises(ValueError, match="3 rows of 2 integers"):
        build_batch([StepEntry("a", [5, 6, 7], [], {"grid": [[1, 2], [3, 4]]})], [0], [0], [[[0]]], torch.device("cpu"), token_inputs=asked)
    assert build_batch(entries[:2], [0, 0], [0, 1], [[[0], [1]]], torch.device("cpu")).inputs == {}
