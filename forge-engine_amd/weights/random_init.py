"""Random weights from a configuration and a seed.

Matrices are drawn from N(0, 0.02) and norm weights from 1 + N(0, 0.05), in
float32, in the fixed order in which the model declares its tensors, and then
rounded to the storage dtype.  ``write_random_model`` writes a model folder
(config.json, model.safetensors) that loads like any checkpoint;
``fill_random_weights`` draws straight onto the device for large models.
"""

from __future__ import annotations

from pathlib import Path

import torch
from safetensors.torch import save_file

from ..config.model import ModelConfig
from ..parts.base import BuildContext, ParamSpec
from ..registry import architecture

MATRIX_STD = 0.02
NORM_STD = 0.05


def _draw(spec: ParamSpec, generator: torch.Generator, device) -> torch.Tensor:
    if spec.kind == "int_table":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=torch.float32, device=device)
    noise = torch.randn(spec.shape, generator=generator, dtype=torch.float32, device=device)
    if spec.init == "norm":
        return 1.0 + noise * NORM_STD
    return noise * MATRIX_STD


def declared_tensors(config: ModelConfig) -> dict[str, ParamSpec]:
    """Names and specs of the tensors the architecture's model reads."""
    from ..models.decoder import DecoderModel

    plan = architecture(config.architecture).plan(config)
    skeleton = DecoderModel(plan, BuildContext(torch.device("cpu"), torch.bfloat16))
    return skeleton.param_specs()


def random_tensors(config: ModelConfig, seed: int, dtype: torch.dtype = torch.bfloat16) -> dict[str, torch.Tensor]:
    generator = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, spec in declared_tensors(config).items():
        value = _draw(spec, generator, "cpu")
        tensors[name] = value if spec.kind == "int_table" else value.to(dtype)
    return tensors


def write_random_model(config: ModelConfig, seed: int, folder: str | Path,
                       dtype: torch.dtype = torch.bfloat16) -> Path:
    """Write ``config.json`` and ``model.safetensors`` into ``folder``."""
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    config.save(folder)
    tensors = {name: t.contiguous() for name, t in random_tensors(config, seed, dtype).items()}
    save_file(tensors, str(folder / "model.safetensors"), metadata={"format": "pt"})
    return folder


def fill_random_weights(model, seed: int, *, device: torch.device, dtype: torch.dtype) -> None:
    """Draw every tensor of ``model`` on ``device`` (values differ from the
    folder mode's: the device generator is another stream)."""
    from .loader import storage_dtype

    generator = torch.Generator(device=device).manual_seed(seed)
    for name, spec in model.param_specs().items():
        value = _draw(spec, generator, device)
        stored = torch.int32 if spec.kind == "int_table" else torch.bfloat16
        model.set_param(name, value.to(storage_dtype(spec.kind, stored, dtype)))
        del value
    model.finalize()
