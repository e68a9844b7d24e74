from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import lookup, register_mixer
from .base import Part, cache_specs_of, views_for


@register_mixer("parallel")
class ParallelMixers(Part):
    """Several mixers side by side that read the same input; the result is the sum of theirs, each times its
    scale.  ``branches``: a tuple of (``PartSpec``, scale).  What the branches ask of the cache is asked for
    one after the other, and each branch is handed its own views.

    Branches that keep a stacked input matrix (``w_in`` [``in_rows()``, hidden], and ``addends(..., proj=, col0=)``)
    share one product: once all tensors are bound their matrices are stacked once more, the rows of the input
    are multiplied once, and each branch is handed its columns.  No row's sum changes by that."""

    def __init__(self, *, branches, position=None, prefix, dtype, device):
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.scales = [float(s) for _, s in branches]
        self.branches = [lookup("mixer", spec.kind)(**spec.params, position=position, prefix=spec.prefix, dtype=dtype,
                                                    device=device) for spec, _ in branches]
        if not self.branches:
            raise ValueError("parallel mixers: at least one branch")

    def children(self):
        return list(self.branches)

    def finish_bind(self):
        self.w_in, self._col0 = None, []
        shared = [b for b in self.branches if getattr(b, "w_in", None) is not None and hasattr(b, "in_rows")]
        if len(shared) < 2 or len({(ops.matrix_shape(b.w_in)[1], b.w_in.dtype) for b in shared}) != 1:
            return
        rows = [ops.untile(b.w_in)[:b.in_rows()] if ops.is_tiled(b.w_in) else b.w_in.as_subclass(torch.Tensor) for b in shared]
        self.w_in = ops.prepare_weight(torch.cat(rows, 0).contiguous())
        at = 0
        for b in self.branches:
            self._col0.append(at if b in shared else None)
            if b in shared:
                at += b.in_rows()
                b.w_in = None                    # the shared product has taken its place

    def cache_specs(self):
        return [s for b in self.branches for s in cache_specs_of(b)]

    def addends(self, h, ctx, views, owns_cache=True):
        out, at = [], 0
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32) if getattr(self, "w_in", None) is not None else None
        for i, (branch, scale) in enumerate(zip(self.branches, self.scales)):
            view, at = views_for(branch, views, at)
            if proj is not None and self._col0[i] is not None:
                out += [(y, s * scale) for y, s in branch.addends(h, ctx, view, owns_cache, proj=proj, col0=self._col0[i])]
            elif hasattr(branch, "addends"):
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
