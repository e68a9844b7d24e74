from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import lookup, register_mixer
from .base import Part, cache_specs_of, views_for


@register_mixer("parallel")
class ParallelMixers(Part):
    """Several mixers side by side that read the same input; the result is the sum of theirs, each times its
    scale.  ``branches``: a tuple of (``PartSpec``, scale).  What the branches ask of the cache is asked for
    one after the other, and each branch is handed its own views."""

    def __init__(self, *, branches, position=None, prefix, dtype, device):
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.scales = [float(s) for _, s in branches]
        self.branches = [lookup("mixer", spec.kind)(**spec.params, position=position, prefix=spec.prefix, dtype=dtype,
                                                    device=device) for spec, _ in branches]
        if not self.branches:
            raise ValueError("parallel mixers: at least one branch")

    def children(self):
        return list(self.branches)

    def cache_specs(self):
        return [s for b in self.branches for s in cache_specs_of(b)]

    def addends(self, h, ctx, views, owns_cache=True):
        out, at = [], 0
        for branch, scale in zip(self.branches, self.scales):
            view, at = views_for(branch, views, at)
            if hasattr(branch, "addends"):
                out += [(y, s * scale) for y, s in branch.addends(h, ctx, view, owns_cache)]
            else:
                y = torch.zeros((h.shape[0], branch.hidden_size), dtype=torch.float32, device=h.device)
                branch.forward(h, ctx, view, y, owns_cache)
                out.append((y, scale))
        return out

    def forward(self, h, ctx, views, residual, owns_cache=True):
        adds = self.addends(h, ctx, views, owns_cache)
        for i in range(0, len(adds), 2):
            ops.add_scaled(residual, adds[i:i + 2])
