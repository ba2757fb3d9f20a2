"""Model descriptions and the generic decoder. Importing registers the architectures."""

from .decoder import DecoderModel, build_model, expected_tensors
from .spec import LayerSpec, ModelSpec, RunStep, Slot, pre_norm_layer
from . import qwen3  # noqa: F401

__all__ = ["DecoderModel", "build_model", "expected_tensors", "LayerSpec", "ModelSpec", "RunStep", "Slot",
           "pre_norm_layer"]
