"""The parts a decoder is assembled from; importing this package registers the
built-in kinds."""

from . import attention, block, embedding, mlp, norm, rotary  # noqa: F401
from .base import (Block, BuildContext, Embedding, FeedForward, Head, Mixer, Norm, ParamSpec, Part,
                   PositionEncoding, Residual, build_part)
from .plan import LayerCall, LayerSpec, ModelPlan, PartSpec

__all__ = ["Block", "BuildContext", "Embedding", "FeedForward", "Head", "LayerCall", "LayerSpec",
           "Mixer", "ModelPlan", "Norm", "ParamSpec", "Part", "PartSpec", "PositionEncoding", "Residual",
           "build_part"]
