from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import register_stream
from ..weights.loader import ParamSpec
from .base import Part


@register_stream("reinject")
class Reinject(Part):
    """x <- W [x; x0]: the residual stream and the embedding's output side by side through one matrix
    [hidden, 2 hidden] (x's columns first).  Used before the first layer of every pass of a stretch of layers that
    runs several times with the same weights.  ``name``: local name of the matrix."""

    def __init__(self, *, hidden_size, name="weight", prefix, dtype, device):
        self.hidden_size, self.name = hidden_size, name
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.weight = None

    def params(self):
        return {self.name: ParamSpec((self.hidden_size, 2 * self.hidden_size))}

    def bind(self, tensors):
        self.weight = ops.prepare_weight(tensors[self.name])

    def forward(self, x, x0, ctx):
        """A new float32 tensor; ``x`` and ``x0`` stay as they are."""
        return ops.linear(ops.concat_cast(x, x0, self.dtype), self.weight, out_dtype=torch.float32)
