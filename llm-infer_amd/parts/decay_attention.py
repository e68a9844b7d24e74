from __future__ import annotations

import torch

from ..cache.specs import StateSpec
from ..kernels import ops
from ..registry import register_mixer
from ..weights.loader import ParamSpec
from .base import Part

_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "g": "g_proj.weight",
          "o": "o_proj.weight", "norm": "norm.weight"}


@register_mixer("decay_attention")
class DecayLinearAttention(Part):
    """Linear attention with a constant decay per head: q, k (heads x head_dim) and v (heads x v_head_dim) are
    silu of their projections; per head S_t = decay_h S_{t-1} + k_t v_t^T and o_t = S_t^T q_t, no other scale.
    The heads of a token together are RMS-normed with a weight, multiplied by sigmoid(W_g h), and projected.

    The state S is float32 [heads, head_dim, v_head_dim] for every sequence (``StateSpec``), zero when the
    sequence starts and carried from step to step; the recurrence runs in float32 whatever the dtype of the
    matrices.  The four input projections are one product against [Wq; Wk; Wv; Wg].  ``decay``: one
    number per head.  ``names``: local tensor names for q, k, v, g, o and norm."""

    def __init__(self, *, hidden_size, n_heads, head_dim, v_head_dim, decay, norm_eps, names=None, position=None,
                 prefix, dtype, device):
        if len(decay) != n_heads:
            raise ValueError(f"decay attention: {len(decay)} decays for {n_heads} heads")
        if not (1 <= head_dim <= 256 and 1 <= v_head_dim <= 256):
            raise ValueError(f"head sizes {head_dim} / {v_head_dim}: the kernel takes head sizes up to 256")
        self.hidden_size, self.n_heads, self.head_dim, self.v_head_dim = hidden_size, n_heads, head_dim, v_head_dim
        self.norm_eps = float(norm_eps)
        self.names = {**_NAMES, **(names or {})}
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.decay = torch.tensor([float(x) for x in decay], dtype=torch.float32, device=device or "cpu")
        self.w_in = self.wo = self.norm = None

    def params(self):
        H, d, dv, w, n = self.n_heads, self.head_dim, self.v_head_dim, self.hidden_size, self.names
        return {n["q"]: ParamSpec((H * d, w)), n["k"]: ParamSpec((H * d, w)), n["v"]: ParamSpec((H * dv, w)),
                n["g"]: ParamSpec((H * dv, w)), n["o"]: ParamSpec((w, H * dv)),
                n["norm"]: ParamSpec((H * dv,), "vector", "ones")}

    def bind(self, tensors):
        n = self.names
        self.w_in = ops.prepare_weight(torch.cat([tensors[n[k]] for k in ("q", "k", "v", "g")], 0).contiguous())
        self.wo = ops.prepare_weight(tensors[n["o"]])
        self.norm = tensors[n["norm"]]

    def cache_spec(self):
        return StateSpec((self.n_heads, self.head_dim, self.v_head_dim), "float32")

    def in_rows(self) -> int:
        return 2 * self.n_heads * (self.head_dim + self.v_head_dim)

    def addends(self, h, ctx, view, owns_cache=True, proj=None, col0=0):
        """``proj`` (float32 [T, n]) with this mixer's q, k, v, g from column ``col0`` on: the product is not run here."""
        if not owns_cache:
            raise ValueError("decay attention keeps a state of its own in every run")
        H, d, dv = self.n_heads, self.head_dim, self.v_head_dim
        if proj is None:
            proj, col0 = ops.linear(h, self.w_in, out_dtype=torch.float32), 0
        # a 16-bit model: prompts run 32 tokens at a time on the matrix cores, decoding token by token on the same
        # 16-bit values of q, k and v; a float32 model runs token by token throughout
        sixteen = self.dtype != torch.float32
        chunked = sixteen and not ctx.is_decode
        o = ops.decay_attention(proj, col0, col0 + H * d, col0 + 2 * H * d, view.state, self.decay, ctx.seq_slot,
                                getattr(ctx, "seq_qstart", None), getattr(ctx, "seq_qlen", None), ctx.n_seqs, H, d, dv,
                                round_to=self.dtype if sixteen else None, chunked=chunked,
                                chunks=ops.decay_chunks(ctx) if chunked else None)
        a = ops.gated_rmsnorm(o, self.norm, proj, col0 + 2 * H * d + H * dv, self.norm_eps, self.dtype)
        return [(ops.linear(a, self.wo, out_dtype=torch.float32), 1.0)]

    def forward(self, h, ctx, view, residual, owns_cache=True):
        ops.add_scaled(residual, self.addends(h, ctx, view, owns_cache))
