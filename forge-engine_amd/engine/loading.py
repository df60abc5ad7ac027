"""From a model folder, or a configuration and a seed, to a built model."""

from __future__ import annotations

from pathlib import Path

import torch

from ..config.model import ModelConfig, load_model_config
from ..models.decoder import DecoderModel
from ..parts.base import BuildContext
from ..registry import architecture
from ..weights import fill_random_weights, load_weights

DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"the engine computes in bfloat16 or float32, not {name}")
        return name
    try:
        return DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"unknown dtype '{name}' (bfloat16 or float32)") from None


def require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda":
        raise RuntimeError("the engine runs on an AMD GPU only (device 'cuda:N'); there is no CPU path")
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible to PyTorch; the engine has no CPU path")
    return device


def build_model(config: ModelConfig, *, dtype, device) -> DecoderModel:
    """The model of the configuration's architecture, without weights."""
    plan = architecture(config.architecture).plan(config)
    return DecoderModel(plan, BuildContext(torch.device(device), parse_dtype(dtype)))


def load_model(folder: str | Path, *, dtype="bfloat16", device="cuda:0") -> tuple[ModelConfig, DecoderModel]:
    """config.json chooses the model class; the safetensors files fill it."""
    folder = Path(folder)
    config = load_model_config(folder)
    model = build_model(config, dtype=dtype, device=device)
    load_weights(model, folder, device=model.ctx.device, dtype=model.ctx.dtype)
    return config, model


def random_model(config: ModelConfig, seed: int, *, dtype="bfloat16", device="cuda:0") -> DecoderModel:
    """A model with weights drawn on the device (no file is written)."""
    model = build_model(config, dtype=dtype, device=device)
    fill_random_weights(model, seed, device=model.ctx.device, dtype=model.ctx.dtype)
    return model
