"""Command line: options with the reference's names and defaults, doctor fields."""

from __future__ import annotations

import pytest

from forge_engine_amd import __version__
from forge_engine_amd.cli import build_parser, main


def test_generation_options_keep_the_reference_names_and_defaults():
    # src/forge_engine/cli.py:38-66 of the reference
    args = build_parser().parse_args(["generate", "--model", "m", "--prompt-ids", "1,2"])
    assert (args.max_new_tokens, args.temperature, args.top_k, args.top_p, args.min_p, args.stop, args.seed) == \
        (256, 0.0, None, 1.0, 0.0, None, None)
    assert (args.max_requests, args.max_batch_size, args.token_budget, args.block_size, args.block_capacity) == \
        (16, 8, 256, 16, 1024)
    args = build_parser().parse_args(["generate", "--random-config", "c.json", "--stop", "a", "--stop", "b",
                                      "--top-k", "5", "--seed", "9", "--prompt-ids", "1", "--prompt-ids", "2,3"])
    assert args.stop == ["a", "b"] and args.top_k == 5 and args.seed == 9 and args.prompt_ids == ["1", "2,3"]


def test_version_and_unknown_commands(capsys):
    with pytest.raises(SystemExit) as done:
        main(["--version"])
    assert done.value.code == 0 and __version__ in capsys.readouterr().out
    for argv in (["chat"], ["serve"], [], ["generate", "--prompt-ids", "1"]):
        with pytest.raises(SystemExit) as done:
            main(argv)
        assert done.value.code == 2


def test_doctor_prints_key_value_lines_without_loading_weights(capsys):
    assert main(["doctor"]) == 0
    lines = capsys.readouterr().out.strip().splitlines()
    keys = [line.split("=", 1)[0] for line in lines]
    assert keys == ["forge_engine_version", "python_version", "pytorch_version", "hip_version", "gpu_available",
                    "gpu_name", "gcn_arch", "gpu_memory_gib", "bf16_supported", "hipcc_available",
                    "kernel_target", "kernels_built", "architectures"]
    assert f"forge_engine_version={__version__}" in lines and "kernel_target=gfx950" in lines


def test_errors_print_with_the_program_name_and_exit_1(capsys, tmp_path):
    assert main(["generate", "--model", str(tmp_path), "--prompt-ids", "1,x"]) == 1
    assert capsys.readouterr().err.startswith("forge-engine: ")
    assert main(["generate", "--model", str(tmp_path), "--prompt-ids", "1", "--temperature", "-1"]) == 1
    assert "temperature" in capsys.readouterr().err
    assert main(["generate", "--model", str(tmp_path / "none"), "--prompt-ids", "1"]) == 1   # no GPU here or no folder
    assert capsys.readouterr().err.startswith("forge-engine: ")
