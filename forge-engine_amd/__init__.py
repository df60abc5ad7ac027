"""forge-engine for MI355X: a one-GPU inference engine for Qwen3 dense, built
from parameterised parts over hand-written HIP kernels for gfx950."""

__version__ = "0.1.0"
