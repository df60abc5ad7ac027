"""forge-engine for MI355X: a one-GPU inference engine for Qwen3 dense, built
from parameterised parts over hand-written HIP kernels for gfx950."""

__version__ = "0.1.0"

from .config import EngineConfig, Qwen3Config, SchedulerConfig, load_model_config  # noqa: E402
from .sampling import SamplingParams  # noqa: E402


def __getattr__(name):
    # the engine classes import torch; load them on first use
    if name in ("ConcurrentGenerationEngine", "GenerationEngine", "ModelRunner", "StepEntry",
                "OverloadedError", "RequestStatus", "engine_from_folder", "engine_from_random"):
        from . import engine

        return getattr(engine, name)
    raise AttributeError(name)


__all__ = ["ConcurrentGenerationEngine", "EngineConfig", "GenerationEngine", "ModelRunner",
           "Qwen3Config", "SamplingParams", "SchedulerConfig", "StepEntry", "load_model_config",
           "__version__"]
