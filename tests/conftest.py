"""Shared fixtures: tiny Qwen3 configurations (config.json form) and markers."""

from __future__ import annotations

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))
if str(ROOT / "tests") not in sys.path:
    sys.path.insert(0, str(ROOT / "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _qwen3(**sizes) -> dict:
    base = {
        "architectures": ["Qwen3ForCausalLM"],
        "model_type": "qwen3",
        "hidden_act": "silu",
        "attention_bias": False,
        "sliding_window": None,
        "eos_token_id": 1,
    }
    base.update(sizes)
    return base


# Two configurations that differ in every size and option, plus one with the
# head size and page size of the large model so that the bf16 fast kernels run
# through the same replay tests.
TINY_A = _qwen3(
    vocab_size=256, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
    num_attention_heads=4, num_key_value_heads=2, head_dim=16,
    max_position_embeddings=128, rms_norm_eps=1e-6, rope_theta=10000.0,
    tie_word_embeddings=True,
)
TINY_B = _qwen3(
    vocab_size=384, hidden_size=96, intermediate_size=224, num_hidden_layers=3,
    num_attention_heads=6, num_key_value_heads=2, head_dim=32,
    max_position_embeddings=256, rms_norm_eps=1e-5, rope_theta=1000000.0,
    tie_word_embeddings=False,
)
TINY_C = _qwen3(
    vocab_size=1003, hidden_size=200, intermediate_size=328, num_hidden_layers=2,
    num_attention_heads=10, num_key_value_heads=2, head_dim=128,
    max_position_embeddings=512, rms_norm_eps=1e-6, rope_theta=5000000.0,
    tie_word_embeddings=True,
)
# the tiny configuration of the reference's own model tests (tests/test_qwen3.py:12-28): heads of 4
TINY_R = _qwen3(
    vocab_size=32, hidden_size=8, intermediate_size=16, num_hidden_layers=2,
    num_attention_heads=2, num_key_value_heads=1, head_dim=4,
    max_position_embeddings=64, rms_norm_eps=1e-6, rope_theta=10000.0,
    tie_word_embeddings=True, eos_token_id=2,
)
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
BLOCK_SIZE = {"A": 4, "B": 8, "C": 16}


@pytest.fixture(params=["A", "B"])
def tiny_name(request):
    return request.param
