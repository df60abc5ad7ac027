"""The ``forge-engine`` command line: ``generate`` and ``doctor``.

In the manner of the reference's command line (src/forge_engine/cli.py:22-168):
the generation options keep its names and defaults (``--max-new-tokens 256``,
``--temperature 0.0``, ``--top-k``, ``--top-p 1.0``, ``--min-p 0.0``, ``--stop``
repeatable, ``--seed``), the scheduler options those of its ``serve`` command
(``--max-requests 16``, ``--max-batch-size 8``, ``--token-budget 256``,
``--block-size 16``, ``--block-capacity 1024``); errors print as
``forge-engine: ...`` with exit code 1; ``doctor`` prints ``key=value`` lines
without loading weights.  ``chat`` and ``serve`` are not part of this engine;
the model comes from ``--model DIR`` (config.json + safetensors) or from
``--random-config FILE`` and a seed.
"""

from __future__ import annotations

import argparse
import json
import platform
import shutil
import sys
from typing import Sequence

from . import __version__


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="forge-engine")
    parser.add_argument("--version", action="version", version=f"%(prog)s {__version__}")
    commands = parser.add_subparsers(dest="command", required=True)
    generate = commands.add_parser("generate", help="generate tokens for one or more prompts on the GPU")
    source = generate.add_mutually_exclusive_group(required=True)
    source.add_argument("--model", help="folder with config.json and safetensors weights")
    source.add_argument("--random-config", help="a config.json; weights are drawn from --weights-seed")
    generate.add_argument("--weights-seed", type=int, default=0)
    generate.add_argument("--prompt-ids", action="append", default=[],
                          help="comma-separated token ids; may be supplied more than once")
    generate.add_argument("--prompt", action="append", default=[],
                          help="text prompt (needs tokenizer.json in the model folder); may be repeated")
    _add_generation_arguments(generate)
    generate.add_argument("--max-requests", type=int, default=16)
    generate.add_argument("--max-batch-size", type=int, default=8)
    generate.add_argument("--token-budget", type=int, default=256)
    generate.add_argument("--block-size", type=int, default=16)
    generate.add_argument("--block-capacity", type=int, default=1_024)
    generate.add_argument("--prefill-chunk", type=int)
    generate.add_argument("--admission", choices=("reserve", "preempt"), default="reserve")
    generate.add_argument("--dtype", choices=("bfloat16", "bf16", "float32", "fp32"), default="bfloat16")
    generate.add_argument("--device", default="cuda:0")
    commands.add_parser("doctor", help="print the local forge-engine and ROCm environment")
    return parser


def _add_generation_arguments(command: argparse.ArgumentParser) -> None:
    command.add_argument("--max-new-tokens", type=int, default=256)
    command.add_argument("--temperature", type=float, default=0.0)
    command.add_argument("--top-k", type=int)
    command.add_argument("--top-p", type=float, default=1.0)
    command.add_argument("--min-p", type=float, default=0.0)
    command.add_argument("--stop", action="append", help="stop string; may be supplied more than once")
    command.add_argument("--seed", type=int)


def run_doctor() -> int:
    """Diagnostics as key=value lines; no weights are loaded."""
    import torch

    from .kernels import build, library
    from .registry import architectures

    available = bool(torch.cuda.is_available())
    properties = torch.cuda.get_device_properties(0) if available else None
    fields = (
        ("forge_engine_version", __version__),
        ("python_version", platform.python_version()),
        ("pytorch_version", torch.__version__),
        ("hip_version", getattr(torch.version, "hip", None) or "unavailable"),
        ("gpu_available", available),
        ("gpu_name", properties.name if available else "unavailable"),
        ("gcn_arch", getattr(properties, "gcnArchName", "unavailable") if available else "unavailable"),
        ("gpu_memory_gib", round(properties.total_memory / 2**30, 1) if available else "unavailable"),
        ("bf16_supported", bool(torch.cuda.is_bf16_supported()) if available else False),
        ("hipcc_available", shutil.which("hipcc") is not None),
        ("kernel_target", build.TARGET_ARCH),
        ("kernels_built", ",".join(n for n in build.source_names() if library.is_built(n)) or "none"),
        ("architectures", ",".join(architectures())),
    )
    for name, value in fields:
        print(f"{name}={value}")
    return 0


def run_generate(args) -> int:
    from .config import EngineConfig, SchedulerConfig, load_model_config
    from .engine import engine_from_folder, engine_from_random
    from .sampling import normalize_stop_strings

    engine_config = EngineConfig(
        max_new_tokens=args.max_new_tokens, temperature=args.temperature, top_k=args.top_k,
        top_p=args.top_p, min_p=args.min_p, stop_strings=normalize_stop_strings(args.stop), seed=args.seed)
    scheduler_config = SchedulerConfig(
        max_requests=args.max_requests, max_batch_size=args.max_batch_size, token_budget=args.token_budget,
        block_size=args.block_size, block_capacity=args.block_capacity, prefill_chunk=args.prefill_chunk,
        admission=args.admission)
    prompts: list = []
    for text in args.prompt_ids:
        try:
            prompts.append([int(part) for part in text.replace(" ", "").split(",") if part])
        except ValueError:
            raise ValueError(f"--prompt-ids must be comma-separated integers, got '{text}'") from None
    prompts.extend(args.prompt)
    if not prompts:
        raise ValueError("give at least one --prompt-ids or --prompt")
    if args.model:
        engine = engine_from_folder(args.model, engine_config=engine_config,
                                    scheduler_config=scheduler_config, dtype=args.dtype, device=args.device)
    else:
        engine = engine_from_random(load_model_config(args.random_config), args.weights_seed,
                                    engine_config=engine_config, scheduler_config=scheduler_config,
                                    dtype=args.dtype, device=args.device)
    # more prompts than --max-requests or than the pages hold at once wait their turn
    failed = False
    for index, view in enumerate(engine.run(prompts)):
        record = {"prompt": index, "status": view.status.value, "finish_reason": view.finish_reason,
                  "token_ids": list(view.output_token_ids)}
        if view.text:
            record["text"] = view.text
        if view.error:
            record["error"] = view.error
            failed = True
        print(json.dumps(record))
    return 1 if failed else 0


def main(argv: Sequence[str] | None = None) -> int:
    args = build_parser().parse_args(argv)
    try:
        if args.command == "doctor":
            return run_doctor()
        if args.command == "generate":
            return run_generate(args)
    except (ValueError, RuntimeError, KeyError) as error:
        print(f"forge-engine: {error}", file=sys.stderr)
        return 1
    return 2


if __name__ == "__main__":
    raise SystemExit(main())
