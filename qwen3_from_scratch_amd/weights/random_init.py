"""Seeded random weights: as a tensor source in memory, or written out as a
model folder (config.json + model.safetensors) that the ordinary loader reads.

The reference has no such mode; its tests use default module initialisation
(e.g. test/models/test_transformer_block.py:52-54). Every tensor is drawn from
a generator seeded by (seed, tensor name), so values do not depend on the order
in which tensors are asked for.
"""

import hashlib
import json
import os

import torch

from .checkpoint import TensorSource


def _tensor_seed(seed, name):
    digest = hashlib.sha256(("%d:%s" % (seed, name)).encode()).digest()
    return int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF


class RandomWeights(TensorSource):
    """Each tensor by what its part says it is (`TensorShape.kind`): a matrix
    (also a table, and any tensor whose part says nothing) N(0, std), a scale
    1 + U(-jitter, jitter), a bias N(0, std). All in bfloat16."""

    def __init__(self, expected, seed=0, std=0.02, norm_jitter=0.1, generate_on=None):
        self.where = "<random weights, seed %d>" % seed
        self._expected = dict(expected)
        self.seed = seed
        self.std = std
        self.norm_jitter = norm_jitter
        self.generate_on = generate_on

    def names(self):
        return list(self._expected)

    def shape(self, name):
        return tuple(self._expected[name])

    def get(self, name, device):
        shape = self.shape(name)
        on = torch.device(self.generate_on) if self.generate_on is not None else torch.device("cpu")
        gen = torch.Generator(device=on)
        gen.manual_seed(_tensor_seed(self.seed, name))
        if getattr(self._expected[name], "kind", "matrix") == "scale":
            t = torch.rand(shape, generator=gen, device=on, dtype=torch.float32)
            t = 1.0 + (2.0 * t - 1.0) * self.norm_jitter
        else:
            t = torch.randn(shape, generator=gen, device=on, dtype=torch.float32) * self.std
        return t.to(torch.bfloat16).to(device)


def write_random_model(folder, config, seed=0, std=0.02, norm_jitter=0.1):
    """Write `config` as config.json and seeded random weights as
    model.safetensors into `folder`; returns the folder."""
    from safetensors.torch import save_file

    from ..config import lookup_architecture
    from ..models.decoder import expected_tensors

    _, build_spec = lookup_architecture(config.architecture)
    expected = expected_tensors(build_spec(config))
    source = RandomWeights(expected, seed=seed, std=std, norm_jitter=norm_jitter)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(config.to_dict(), fh, indent=2)
    tensors = {name: source.get(name, "cpu").contiguous() for name in source.names()}
    save_file(tensors, os.path.join(folder, "model.safetensors"), metadata={"format": "pt"})
    return folder
