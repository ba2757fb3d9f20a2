"""A single-GPU inference engine for the Qwen3 dense decoder on AMD MI355X (gfx950).

Importing the package registers the architectures and parts it ships; nothing is
compiled or loaded from the GPU until an operation is first called.
"""

from .config import ModelConfig, load_model_config, register_architecture, architectures
from . import parts as _parts  # registers the parts  # noqa: F401
from . import models as _models  # registers the architectures  # noqa: F401

__all__ = [
    "ModelConfig",
    "load_model_config",
    "register_architecture",
    "architectures",
]
