"""The step function, the scheduler above it and the Python entry points."""

from .api import (GenerationEngine, build_engine, engine_from_folder, engine_from_random,
                  load_tokenizer)
from .batch import StepBatch, StepEntry
from .detokenizer import IncrementalDetokenizer
from .loading import build_model, load_model, parse_dtype, random_model
from .runner import ModelRunner
from .scheduler import (ConcurrentGenerationEngine, OverloadedError, RequestStatus, RequestView,
                        SchedulerSnapshot, StreamEvent)

__all__ = ["ConcurrentGenerationEngine", "GenerationEngine", "IncrementalDetokenizer", "ModelRunner",
           "OverloadedError", "RequestStatus", "RequestView", "SchedulerSnapshot", "StepBatch",
           "StepEntry", "StreamEvent", "build_engine", "build_model", "engine_from_folder",
           "engine_from_random", "load_model", "load_tokenizer", "parse_dtype", "random_model"]
