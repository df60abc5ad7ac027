"""Load a model's tensors from safetensors files by tensor name.

One tensor is read, checked, cast and handed to its part at a time, as the
reference stages its copy (src/forge_engine/weights.py:202-243), so the host
never holds more than one tensor.  Before anything is read, names and shapes of
the whole checkpoint are compared with what the model declares, and one error
lists every missing tensor, every unexpected tensor and every wrong shape.

Storage policy: matrices stay in bfloat16 for a bfloat16 model and are widened
for a float32 model; a tensor that the file stores in 32-bit stays 32-bit;
norm weights and biases are widened to float32 (exact); integer tables become
int32.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors import safe_open

INDEX_NAME = "model.safetensors.index.json"
SINGLE_NAME = "model.safetensors"
_SAFETENSORS_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}


class WeightsError(ValueError):
    """The checkpoint does not fit the model.  ``missing``, ``unexpected`` and
    ``wrong_shape`` hold the full lists; the message shows them."""

    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=()) -> None:
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)


def storage_dtype(kind: str, stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    """The dtype a loaded tensor is kept in."""
    if kind == "int_table" or not stored.is_floating_point:
        return torch.int32
    if kind == "vector" or stored in (torch.float32, torch.float64):
        return torch.float32
    return compute


def checkpoint_files(folder: Path) -> dict[str, Path]:
    """Tensor name -> file that holds it."""
    folder = Path(folder)
    index = folder / INDEX_NAME
    if index.exists():
        weight_map = json.loads(index.read_text()).get("weight_map")
        if not isinstance(weight_map, dict):
            raise WeightsError(f"{index} has no 'weight_map'")
        return {name: folder / shard for name, shard in weight_map.items()}
    files = [folder / SINGLE_NAME] if (folder / SINGLE_NAME).exists() else sorted(folder.glob("*.safetensors"))
    if not files:
        raise WeightsError(f"no safetensors file in {folder}")
    names: dict[str, Path] = {}
    for path in files:
        with safe_open(str(path), framework="pt", device="cpu") as handle:
            for name in handle.keys():
                if name in names:
                    raise WeightsError(f"tensor '{name}' appears in {names[name].name} and {path.name}")
                names[name] = path
    return names


def _short(items, limit: int = 12) -> str:
    items = list(items)
    shown = ", ".join(str(item) for item in items[:limit])
    return shown + (f", ... ({len(items)} in all)" if len(items) > limit else "")


def load_weights(model, folder: str | Path, *, device: torch.device, dtype: torch.dtype,
                 check_finite: bool = True) -> None:
    """Fill ``model`` (a DecoderModel) from the safetensors files in ``folder``."""
    folder = Path(folder)
    specs = model.param_specs()
    ignorable = model.ignorable_names() if hasattr(model, "ignorable_names") else set()
    files = checkpoint_files(folder)
    missing = sorted(n for n, s in specs.items() if n not in files and not s.optional)
    unexpected = sorted(n for n in files if n not in specs and n not in ignorable)
    by_file: dict[Path, list[str]] = {}
    for name, path in files.items():
        if name in specs:
            by_file.setdefault(path, []).append(name)
    wrong_shape = []
    for path, names in sorted(by_file.items()):
        if not path.exists():
            raise WeightsError(f"the index names {path.name}, which is not in {folder}")
        with safe_open(str(path), framework="pt", device="cpu") as handle:
            present = set(handle.keys())
            for name in names:
                if name not in present:
                    missing.append(name)
                    continue
                shape = tuple(handle.get_slice(name).get_shape())
                if shape != tuple(specs[name].shape):
                    wrong_shape.append(f"{name}: file {shape}, model {tuple(specs[name].shape)}")
    if missing or unexpected or wrong_shape:
        parts = []
        if missing:
            parts.append(f"missing tensors: {_short(sorted(missing))}")
        if unexpected:
            parts.append(f"unexpected tensors: {_short(unexpected)}")
        if wrong_shape:
            parts.append(f"wrong shapes: {_short(wrong_shape)}")
        raise WeightsError(f"checkpoint in {folder} does not fit the model; " + "; ".join(parts),
                           missing, unexpected, wrong_shape)
    for path, names in sorted(by_file.items()):
        with safe_open(str(path), framework="pt", device="cpu") as handle:
            for name in names:
                source = handle.get_tensor(name)
                if check_finite and source.is_floating_point() and not torch.isfinite(source).all():
                    raise WeightsError(f"tensor '{name}' holds non-finite values")
                target = storage_dtype(specs[name].kind, source.dtype, dtype)
                model.set_param(name, source.to(device=device, dtype=target))
                del source
    model.finalize()
