"""Output heads: hidden rows to float32 logits."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import Part
from .linear import LinearWeight


@register_part("head", "linear")
class LinearHead(Part):
    """logits = h @ W^T, no bias (src/qwen3_from_scratch/models/qwen3.py:63-65,83-84).
    `weight_name` is the full checkpoint name of W: the embedding's name ties
    the head to it (qwen3.py:69-70) and both then share one tensor."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, vocab_size, weight_name):
        super().__init__(prefix, precision, device)
        self.hidden_size = hidden_size
        self.vocab_size = vocab_size
        self.weight_name = weight_name
        self.weight = None

    def tensors(self):
        return {self.weight_name: (self.vocab_size, self.hidden_size)}

    def load(self, fetch):
        self.weight = LinearWeight(fetch(self.weight_name, self.precision.act), self.precision)

    def forward(self, h):
        return self.weight.forward(h, out_dtype=torch.float32)
