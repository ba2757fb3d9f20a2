"""Feed-forward parts."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import Part


@register_part("feed_forward", "swiglu")
class SwiGLU(Part):
    """down(silu(gate(x)) * up(x)), no biases
    (src/qwen3_from_scratch/models/feedback.py:28-34). gate and up are kept as
    one matrix [gate | up] so that one product feeds the activation kernel."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, intermediate_size):
        super().__init__(prefix, precision, device)
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up = None
        self.down = None

    def tensors(self):
        H, I = self.hidden_size, self.intermediate_size
        return {
            self._name("gate_proj.weight"): (I, H),
            self._name("up_proj.weight"): (I, H),
            self._name("down_proj.weight"): (H, I),
        }

    def load(self, fetch):
        act = self.precision.act
        I, H = self.intermediate_size, self.hidden_size
        self.gate_up = torch.empty((2 * I, H), dtype=act, device=self.device)
        self.gate_up[:I].copy_(fetch(self._name("gate_proj.weight"), act, keep=False))
        self.gate_up[I:].copy_(fetch(self._name("up_proj.weight"), act, keep=False))
        self.down = fetch(self._name("down_proj.weight"), act)

    def forward(self, x, batch=None):
        gate_up = ops.linear(x, self.gate_up)
        return ops.linear(ops.swiglu(gate_up), self.down)
