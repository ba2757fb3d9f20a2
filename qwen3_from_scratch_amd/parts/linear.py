"""A weight matrix as the parts hold it: row-major, and for bfloat16 a second copy
in the order the few-row product kernel streams it."""

import torch

from .. import ops


class LinearWeight:
    """y = x @ W^T, no bias. W (N, K) is kept row-major for products with many
    rows (the vendor library's) and for float32; when the precision asks for
    it, a tile-ordered bfloat16 copy serves steps with at most 16 rows, where
    every weight is read once and the order in memory decides the bandwidth.
    The copy doubles the weight's memory."""

    def __init__(self, weight, precision):
        self.weight = weight
        self.tiled = ops.tile_weight(weight) if precision.tiled else None

    def forward(self, x, out_dtype=None):
        return ops.linear(x, self.weight, out_dtype=out_dtype, tiled=self.tiled)

    def forward_swiglu(self, x):
        """swiglu(x @ W^T) for a W whose rows interleave gate and up."""
        return ops.linear_swiglu(x, self.weight, tiled=self.tiled)
