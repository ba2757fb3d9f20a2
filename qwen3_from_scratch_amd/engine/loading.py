"""From a model folder (or a configuration and a seed) to a runner."""

import torch

from ..config.registry import load_model_config
from ..models.decoder import build_model
from ..parts.base import Precision
from ..weights import Checkpoint, RandomWeights


def load_model(model_dir, dtype="bfloat16", device="cuda", tiled_weights=True, components=None):
    """Read config.json, pick the model by its architecture, load model.safetensors.
    `tiled_weights`: keep the second, tile-ordered copy of every bfloat16 matrix that makes steps
    of few rows fast (see `Precision`); without it the matrices are held once.
    `components`: {slot: part name, or {name, kwargs}}, other registered implementations for
    some kinds of parts (src/qwen3_from_scratch/inference/model_loader.py:18-35)."""
    config = load_model_config(model_dir)
    model = build_model(config, Precision.named(dtype, tiled=tiled_weights), device, components=components)
    model.load(Checkpoint(model_dir))
    model.config = config
    return model


def random_model(config, dtype="bfloat16", device="cuda", seed=0, std=0.02, norm_jitter=0.1, tiled_weights=True):
    """A model of `config` with seeded random weights drawn on the device."""
    model = build_model(config, Precision.named(dtype, tiled=tiled_weights), device)
    on = device if torch.device(device).type == "cuda" else None
    model.load(RandomWeights(model.tensors(), seed=seed, std=std, norm_jitter=norm_jitter, generate_on=on))
    model.config = config
    return model


def load_runner(model_dir, dtype="bfloat16", device="cuda", page_size=16, max_tokens=8192, max_requests=32,
                use_graphs=True, tiled_weights=True, prefix_cache=False, components=None):
    from .runner import ModelRunner

    model = load_model(model_dir, dtype, device, tiled_weights=tiled_weights, components=components)
    num_pages = -(-max_tokens // page_size)
    return ModelRunner(model, page_size, num_pages, max_requests, use_graphs=use_graphs, prefix_cache=prefix_cache)
