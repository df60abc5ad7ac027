"""Typed configurations: the model's (read from config.json) and the engine's."""

from .engine import EngineConfig, SchedulerConfig
from .model import ConfigError, ModelConfig, load_model_config
from .qwen3 import Qwen3Config

__all__ = ["ConfigError", "EngineConfig", "ModelConfig", "Qwen3Config", "SchedulerConfig",
           "load_model_config"]
