from __future__ import annotations

import torch

from ..cache.specs import StateSpec
from ..kernels import ops
from ..registry import register_mixer
from ..weights.loader import ParamSpec
from .base import Part

_NAMES = {"in": "in_proj.weight", "conv": "conv1d.weight", "conv_bias": "conv1d.bias", "dt_bias": "dt_bias",
          "a_log": "A_log", "d": "D", "norm": "norm.weight", "o": "out_proj.weight"}


@register_mixer("state_space")
class SelectiveStateSpace(Part):
    """The selective state-space mixer with a scalar decay per head and step (state-space duality form).
    With P heads of ``head_dim`` values, a state of ``n_state`` per value, ``n_groups`` groups of heads that
    share B and C (head h uses group h // (P / groups)) and inner = P * head_dim, the input product yields
    [z: inner | x: inner | B: groups * n_state | C: groups * n_state | dt: P].  x, B and C pass a causal
    convolution per channel over ``conv_taps`` tokens (weight [channels, taps], the last column the current
    token's, a bias, zeros before the sequence) and silu.  Then per head

        dt = softplus(dt + dt_bias),   S_t = exp(-exp(A_log) dt) S_{t-1} + dt B_t x_t^T,   y_t = S_t^T C_t + D x_t

    The heads' y side by side are multiplied by silu(z) and then, in ``norm_groups`` equal parts, divided by
    each part's root mean square and multiplied by a weight; the output product adds into the residual stream.
    Step sizes, decays, the state S (float32 [P, n_state, head_dim] for every sequence, zero at its start) and
    the norm are float32 whatever the matrices' type; the convolution's last taps - 1 inputs are kept for every
    sequence too, so that a prompt may be cut anywhere.  ``names``: local tensor names."""

    takes_lazy_norm = True

    def __init__(self, *, hidden_size, n_heads, head_dim, n_state, n_groups=1, conv_taps=4, norm_groups=1, norm_eps,
                 names=None, position=None, prefix, dtype, device):
        if n_heads % n_groups != 0:
            raise ValueError("state space: heads must be a multiple of groups")
        if (n_heads * head_dim) % norm_groups != 0:
            raise ValueError("state space: the norm's groups must divide heads * head_dim")
        if not 1 <= n_state <= 256:
            raise ValueError(f"state space: a state of {n_state} (the kernel keeps up to 256 a value)")
        if not 1 <= conv_taps <= 16:
            raise ValueError(f"state space: a convolution over {conv_taps} tokens (up to 16)")
        self.hidden_size, self.n_heads, self.head_dim, self.n_state = hidden_size, n_heads, head_dim, n_state
        self.n_groups, self.conv_taps, self.norm_groups, self.norm_eps = n_groups, conv_taps, norm_groups, float(norm_eps)
        self.inner = n_heads * head_dim
        self.channels = self.inner + 2 * n_groups * n_state
        self.names = {**_NAMES, **(names or {})}
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.w_in = self.wo = None

    def params(self):
        n, w, P = self.names, self.hidden_size, self.n_heads
        return {n["in"]: ParamSpec((self.inner + self.channels + P, w)),
                n["conv"]: ParamSpec((self.channels, self.conv_taps), "vector", "wide"),
                n["conv_bias"]: ParamSpec((self.channels,), "vector", "small"),
                n["dt_bias"]: ParamSpec((P,), "vector", "small"), n["a_log"]: ParamSpec((P,), "vector", "small"),
                n["d"]: ParamSpec((P,), "vector", "ones"), n["norm"]: ParamSpec((self.inner,), "vector", "ones"),
                n["o"]: ParamSpec((w, self.inner))}

    def bind(self, tensors):
        n = self.names
        self.w_in, self.wo = ops.prepare_weight(tensors[n["in"]]), ops.prepare_weight(tensors[n["o"]])
        self.conv, self.conv_bias = tensors[n["conv"]], tensors[n["conv_bias"]]
        self.dt_bias, self.a_log, self.d_skip, self.norm = tensors[n["dt_bias"]], tensors[n["a_log"]], tensors[n["d"]], tensors[n["norm"]]

    def cache_specs(self):
        return [StateSpec((self.n_heads, self.n_state, self.head_dim), "float32"),
                StateSpec((max(self.conv_taps - 1, 1), self.channels), "float32")]

    def forward(self, h, ctx, views, residual, owns_cache=True):
        if not owns_cache:
            raise ValueError("a state-space mixer keeps a state of its own in every run")
        state, history = views[0].state, views[1].state
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        xbc = ops.conv_silu(proj, self.inner, self.channels, self.conv, self.conv_bias, history, ctx)
        # a 16-bit model walks long prompts in segments side by side; a float32 model (and every decode step) walks each
        # sequence in order, which gives the same bits however a prompt is cut
        segments = None
        if self.dtype != torch.float32 and not ctx.is_decode and getattr(ctx, "host_qlens", None):
            # segments short enough that some 3,000 waves run (three a SIMD), between 16 and SSM_SEGMENT tokens
            waves_a_token = self.n_heads * ((self.head_dim + 63) // 64)
            length = max(16, min(ops.SSM_SEGMENT, 1 << max(0, (ctx.n_tokens * waves_a_token // ops.SSM_WAVES).bit_length() - 1)))
            if max(ctx.host_qlens) > length:
                segments = ops.ssm_segments(ctx, length)
        y = ops.ssm_scan(xbc, proj, self.inner + self.channels, self.dt_bias, self.a_log, self.d_skip, state, ctx,
                         self.n_heads, self.n_groups, self.n_state, self.head_dim, segments)
        a = ops.gated_group_norm(y, proj, 0, self.norm, self.norm_groups, self.norm_eps, self.dtype)
        ops.linear(a, self.wo, ops.EPI_ADD, out=residual)
