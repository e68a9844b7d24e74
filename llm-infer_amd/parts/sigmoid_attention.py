from __future__ import annotations

import torch

from ..cache.specs import KVSpec
from ..kernels import ops
from ..registry import register_mixer
from ..weights.loader import ParamSpec
from .base import Part

_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight", "bias": "head_bias"}


@register_mixer("sigmoid_attention")
class SigmoidAttention(Part):
    """Causal grouped-query attention over the paged cache whose weights are not a softmax: a visible key j
    weighs sigmoid(q . k_j * scale + bias[head]) and the weights are not normalised over the keys.
    Queries and keys have ``head_dim`` dimensions, values ``v_head_dim``; query head h reads key/value head
    h // (H / G).  q and k are rotated by the layer's position part (its frequencies, rotated dimensions and
    pairing are read off it; the kernel rotates half-paired heads as they are stored) and then, with
    ``unit_norm_eps`` not None, each head is divided by its root mean square (no weight).  Scores, weights
    and sums are float32 in every dtype.  ``head_bias`` False: no bias tensor.  ``names``: local tensor
    names for q, k, v, o and bias.

    In the pages keys are as wide as the next multiple of 16 and values likewise (what the matrix kernels
    take); the added dimensions hold zeros."""

    def __init__(self, *, hidden_size, n_heads, n_kv_heads, head_dim, v_head_dim=None, scale, unit_norm_eps=None,
                 head_bias=True, window=None, names=None, position=None, prefix, dtype, device):
        if n_heads % n_kv_heads != 0:
            raise ValueError("n_heads must be a multiple of n_kv_heads")
        v_head_dim = v_head_dim or head_dim
        if not (1 <= head_dim <= 256 and 1 <= v_head_dim <= 256):
            raise ValueError(f"head sizes {head_dim} / {v_head_dim}: the attention kernels take head sizes up to 256")
        self.hidden_size, self.n_heads, self.n_kv_heads = hidden_size, n_heads, n_kv_heads
        self.head_dim, self.v_head_dim = head_dim, v_head_dim
        self.k_dim, self.v_dim = (head_dim + 15) // 16 * 16, (v_head_dim + 15) // 16 * 16      # in the pages
        self.scale, self.window, self.position = float(scale), window, position
        self.unit_norm_eps = None if unit_norm_eps is None else float(unit_norm_eps)
        self.head_bias = bool(head_bias)
        self.names = {**_NAMES, **(names or {})}
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.w_in = self.wo = self.bias = None

    def params(self):
        H, G, d, dv, w, n = self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim, self.hidden_size, self.names
        out = {n["q"]: ParamSpec((H * d, w)), n["k"]: ParamSpec((G * d, w)), n["v"]: ParamSpec((G * dv, w)),
               n["o"]: ParamSpec((w, H * dv))}
        if self.head_bias:
            out[n["bias"]] = ParamSpec((H,), "vector", "small")
        return out

    def bind(self, tensors):
        n = self.names
        # ``w_in``: the stacked input matrix [Wq; Wk; Wv]; a mixer that runs this one beside others on the same rows
        # may take it into a product of its own (``ParallelMixers``) and hand over the columns instead
        self.w_in = ops.prepare_weight(torch.cat([tensors[n["q"]], tensors[n["k"]], tensors[n["v"]]], 0).contiguous())
        self.wo = ops.prepare_weight(tensors[n["o"]])
        self.bias = tensors[n["bias"]] if self.head_bias else None

    def cache_spec(self):
        return KVSpec(self.n_kv_heads, self.k_dim, self.window, self.v_dim)

    def _rotation(self):
        p = self.position
        rot = getattr(p, "rotary_dim", 0) if p is not None else 0
        if rot == 0:
            return None, 0, False
        return p.inv_freq, rot, getattr(p, "pairing", "adjacent") == "half"

    def in_rows(self) -> int:
        return (self.n_heads + self.n_kv_heads) * self.head_dim + self.n_kv_heads * self.v_head_dim

    def addends(self, h, ctx, view, owns_cache=True, proj=None, col0=0):
        """``proj`` (float32 [T, n]) with this mixer's q, k, v from column ``col0`` on: the product is not run here."""
        if not owns_cache:
            raise ValueError("sigmoid attention writes its own keys and values in every run")
        H, G, d, dv = self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim
        if proj is None:
            proj, col0 = ops.linear(h, self.w_in, out_dtype=torch.float32), 0
        inv_freq, rot, half = self._rotation()
        kv = view.as_tuple()
        # the angles of the step's tokens: one table for all layers that rotate with these frequencies (the
        # position part shares it through the step; a float32 model computes them where they are used)
        table = self.position._table(ctx) if rot and hasattr(self.position, "_table") else None
        q = ops.rope_norm_store(proj, inv_freq, rot, half, self.unit_norm_eps, ctx.pos, ctx.tok_slot, kv, H, G, d, dv,
                                self.k_dim, self.k_dim, self.v_dim, self.dtype, col0=col0, cos_sin=table)
        if self.dtype == torch.float32:
            a = ops.sigmoid_attention(q, kv, ctx.pos, ctx.tok_slot, self.bias, H, G, self.k_dim, dv, self.v_dim,
                                      self.scale, self.window)
        elif ctx.is_decode:
            a = ops.sigmoid_attention_decode(q, kv, ctx.seq_slot, ctx.seq_ctx, ctx.n_seqs, self.bias, H, G, self.k_dim,
                                             dv, self.v_dim, self.scale, self.window, ctx.decode_splits(G, H))
        else:
            a = ops.sigmoid_attention_prefill(q, kv, ops.prefill_meta(ctx), self.bias, H, G, self.k_dim, dv,
                                              self.v_dim, self.scale, self.window)
        return [(ops.linear(a.view(a.shape[0], H * dv), self.wo, out_dtype=torch.float32), 1.0)]

    def forward(self, h, ctx, view, residual, owns_cache=True):
        ops.add_scaled(residual, self.addends(h, ctx, view, owns_cache))
