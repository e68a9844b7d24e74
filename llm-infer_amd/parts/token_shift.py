from __future__ import annotations

from ..cache.specs import StateSpec
from ..kernels import ops
from ..registry import lookup, register_mixer
from ..weights.loader import ParamSpec
from .base import Part, cache_specs_of, views_for


@register_mixer("token_shift")
class ShiftedMixer(Part):
    """A mixer whose input is first mixed with the input of the token before, channel by channel:
    h_t <- h_t + (h_{t-1} - h_t) * mu, with h_{t-1} as it was before this mixing and zeros before a
    sequence's first token.  ``inner`` (a ``PartSpec``) is the mixer that reads the result.

    The row before is found in the step itself or, for the first token that a sequence brings to a step,
    in the sequence's state: the last row of the step before, float32 [hidden], kept for every layer
    (``StateSpec``).  The part reads the float32 residual rows themselves (``reads_residual``) and hands the
    inner mixer its input in the compute dtype.  ``name``: local name of mu's tensor [hidden]."""

    reads_residual = True

    def __init__(self, *, hidden_size, inner, name="shift", position=None, prefix, dtype, device):
        self.hidden_size, self.name = hidden_size, name
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.inner = lookup("mixer", inner.kind)(**inner.params, position=position, prefix=inner.prefix, dtype=dtype,
                                                 device=device)
        self.mu = None

    def children(self):
        return [self.inner]

    def params(self):
        return {self.name: ParamSpec((self.hidden_size,), "vector", "half")}

    def bind(self, tensors):
        self.mu = tensors[self.name]

    def cache_specs(self):
        return [StateSpec((self.hidden_size,), "float32")] + cache_specs_of(self.inner)

    def _shift(self, x, ctx, views):
        return ops.token_shift(x, self.mu, views[0].state, ctx.pos, ctx.tok_slot, self.dtype,
                               single=ctx.n_tokens == ctx.n_seqs)

    def addends(self, x, ctx, views, owns_cache=True):
        if not owns_cache:
            raise ValueError("a token-shift mixer keeps a state of its own in every run")
        h = self._shift(x, ctx, views)
        inner_views, _ = views_for(self.inner, views, 1)
        if hasattr(self.inner, "addends"):
            return self.inner.addends(h, ctx, inner_views, owns_cache)
        import torch
        y = torch.zeros_like(x)
        self.inner.forward(h, ctx, inner_views, y, owns_cache)
        return [(y, 1.0)]

    def forward(self, x, ctx, views, residual, owns_cache=True):
        """``x``: float32 rows (the stream or a norm of it); the inner mixer's result is added into ``residual``."""
        adds = self.addends(x, ctx, views, owns_cache)
        for i in range(0, len(adds), 2):
            ops.add_scaled(residual, adds[i:i + 2])
