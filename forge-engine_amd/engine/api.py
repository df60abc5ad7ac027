"""Python entry points: build an engine from a model folder or from a
configuration and a seed, then generate.

``GenerationEngine`` serves one request at a time (the reference's
``GenerationEngine.stream``, src/forge_engine/engine.py:365-451);
``ConcurrentGenerationEngine`` (scheduler.py) serves many.  Both sit on the same
step function; prompts are token ids (text if the model folder holds a
``tokenizer.json``).
"""

from __future__ import annotations

from pathlib import Path
from typing import Iterator

from ..config.engine import EngineConfig, SchedulerConfig
from ..config.model import ModelConfig
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .loading import load_model, random_model, require_gpu
from .runner import ModelRunner
from .scheduler import ConcurrentGenerationEngine, RequestStatus, StreamEvent


class FolderTokenizer:
    """``tokenizer.json`` of a model folder through the ``tokenizers`` package."""

    def __init__(self, path: Path) -> None:
        from tokenizers import Tokenizer

        self._tokenizer = Tokenizer.from_file(str(path))

    def encode(self, text: str) -> list[int]:
        return self._tokenizer.encode(text).ids

    def decode(self, ids, skip_special_tokens: bool = True) -> str:
        return self._tokenizer.decode(list(ids), skip_special_tokens=skip_special_tokens)


def load_tokenizer(folder: str | Path):
    path = Path(folder) / "tokenizer.json"
    return FolderTokenizer(path) if path.exists() else None


def build_engine(model, *, engine_config: EngineConfig | None = None,
                 scheduler_config: SchedulerConfig | None = None, tokenizer=None,
                 eos_token_ids=None) -> ConcurrentGenerationEngine:
    """A concurrent engine over ``model`` with a cache pool of the scheduler
    configuration's size."""
    scheduler_config = scheduler_config or SchedulerConfig()
    runner = ModelRunner(
        model, block_size=scheduler_config.block_size, block_capacity=scheduler_config.block_capacity,
        num_state_slots=scheduler_config.num_state_slots or scheduler_config.max_requests)
    params = (engine_config or EngineConfig()).sampling_params()
    return ConcurrentGenerationEngine(runner, Sampler(model.ctx.device), params, scheduler_config,
                                      tokenizer=tokenizer, eos_token_ids=eos_token_ids)


def engine_from_folder(folder: str | Path, *, engine_config: EngineConfig | None = None,
                       scheduler_config: SchedulerConfig | None = None, dtype="bfloat16",
                       device="cuda:0", eos_token_ids=None) -> ConcurrentGenerationEngine:
    """config.json picks the model class, the safetensors files fill it.  ``eos_token_ids``
    overrides the end-of-sequence tokens that config.json names."""
    device = require_gpu(device)
    _, model = load_model(folder, dtype=dtype, device=device)
    return build_engine(model, engine_config=engine_config, scheduler_config=scheduler_config,
                        tokenizer=load_tokenizer(folder), eos_token_ids=eos_token_ids)


def engine_from_random(config: ModelConfig, seed: int, *, engine_config: EngineConfig | None = None,
                       scheduler_config: SchedulerConfig | None = None, dtype="bfloat16",
                       device="cuda:0") -> ConcurrentGenerationEngine:
    """Random weights drawn on the device from ``seed``."""
    device = require_gpu(device)
    model = random_model(config, seed, dtype=dtype, device=device)
    return build_engine(model, engine_config=engine_config, scheduler_config=scheduler_config)


ConcurrentGenerationEngine.from_folder = staticmethod(engine_from_folder)
ConcurrentGenerationEngine.from_random = staticmethod(engine_from_random)


class GenerationEngine:
    """One request at a time: ``stream`` yields each generated token (its text
    if there is a tokenizer) as it is sampled; ``generate`` returns them all."""

    def __init__(self, engine: ConcurrentGenerationEngine) -> None:
        self._engine = engine

    @classmethod
    def from_folder(cls, folder, engine_config: EngineConfig | None = None, **options) -> "GenerationEngine":
        return cls(engine_from_folder(folder, engine_config=engine_config, **options))

    @classmethod
    def from_random(cls, config: ModelConfig, seed: int, engine_config: EngineConfig | None = None,
                    **options) -> "GenerationEngine":
        return cls(engine_from_random(config, seed, engine_config=engine_config, **options))

    @property
    def engine(self) -> ConcurrentGenerationEngine:
        return self._engine

    def events(self, prompt, sampling_params: SamplingParams | None = None) -> Iterator[StreamEvent]:
        request_id = self._engine.submit(prompt, sampling_params=sampling_params)
        try:
            while not self._engine.request(request_id).status.terminal:
                for event in self._engine.step():
                    if event.request_id == request_id:
                        yield event
            view = self._engine.request(request_id)
            if view.status is RequestStatus.FAILED:
                raise RuntimeError(f"generation failed: {view.error}")
        finally:
            self._engine.cancel(request_id)   # frees pages if the consumer stopped early
            self._engine.forget(request_id)

    def stream(self, prompt, sampling_params: SamplingParams | None = None) -> Iterator:
        """Token ids, or text fragments when the engine has a tokenizer."""
        text = self._engine._tokenizer is not None
        for event in self.events(prompt, sampling_params):
            if text:
                if event.text:
                    yield event.text
            else:
                yield from event.token_ids

    def generate(self, prompt, sampling_params: SamplingParams | None = None) -> list[int]:
        tokens: list[int] = []
        for event in self.events(prompt, sampling_params):
            tokens.extend(event.token_ids)
        return tokens
