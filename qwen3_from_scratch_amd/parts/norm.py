"""Norms over the last dimension."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import NormSink, Part, TensorShape


@register_part("norm", "rms")
class RMSNorm(Part):
    """y = x * rsqrt(mean(x^2) + eps) * weight, eps inside the root, plain weight
    (src/qwen3_from_scratch/models/norm.py:18-22,51-53). It reads the float32
    residual stream and can fold the pending addition `x += delta` into the
    same pass; the sum, the mean and the products are float32 and the result
    is rounded once."""

    graph_safe = True

    def __init__(self, prefix, precision, device, size, eps):
        super().__init__(prefix, precision, device)
        self.size = size
        self.eps = float(eps)
        self.weight = None

    def tensors(self):
        return {self._name("weight"): TensorShape((self.size,), "scale")}

    def load(self, fetch):
        self.weight = fetch(self._name("weight"))

    def forward(self, x, delta=None, rows=None):
        """Normalised rows in the activation dtype. With `delta`, x += delta
        first (in place, unless `rows` selects a subset: then x is left alone)."""
        return ops.rmsnorm(x, self.weight, self.eps, self.precision.act, delta=delta,
                           rows=rows, write_back=rows is None)

    def sink_for(self, x):
        """A NormSink for the residual `x` if this step may have the addition
        and this norm fused into the neighbouring products (bfloat16 with
        tiled matrices; at most 16 rows and a width in steps of 16, or up to
        128 rows and a width in steps of 64), else None."""
        rows = x.shape[0]
        if self.precision.act != torch.bfloat16 or not self.precision.tiled or self.weight is None:
            return None
        if not 1 <= rows <= ops.FUSED_ROWS_MOST or self.size % (16 if rows <= ops.FUSED_ROWS_FEW else 64):
            return None
        return NormSink(x, self.weight, self.eps, self.size)
