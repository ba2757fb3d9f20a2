"""Token embedding: a row gather into the float32 residual stream."""

from .. import ops
from ..config.registry import register_part
from .base import Part


@register_part("embedding", "token")
class TokenEmbedding(Part):
    """x[t] = E[ids[t]], no scaling, no padding row
    (src/qwen3_from_scratch/models/qwen3.py:17-19,45)."""

    graph_safe = True

    def __init__(self, prefix, precision, device, vocab_size, hidden_size):
        super().__init__(prefix, precision, device)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.weight = None

    def tensors(self):
        return {self._name("weight"): (self.vocab_size, self.hidden_size)}

    def load(self, fetch):
        self.weight = fetch(self._name("weight"), self.precision.act)

    def forward(self, token_ids):
        return ops.embed_rows(token_ids, self.weight)
