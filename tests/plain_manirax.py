"""Plain, slow Manirax decoder: whole sequences, no cache, one function per mechanism.

Written from the design's equations and sharing no code with the engine.  All arithmetic runs in
the dtype of the weights handed in (float64 when the caller widens them), token by token where the
design is recurrent.

The design, in this file's notation.  The residual stream x is [T, width].  A layer is
    x <- LN1(alpha x + mixer(shift(x)));   x <- LN2(alpha x + ff(x))        (the second only with a feed-forward)
with LN a layer norm with a weight and no bias.  shift mixes each token's vector with its
predecessor's, channel by channel.  The mixer is the weighted sum of two mixers that read the same
input: causal attention whose weights are sigmoids of the biased scores (no normalisation over
keys), with partly rotated and then unit-RMS queries and keys; and linear attention with a
constant decay per head whose output is RMS-normed, gated and projected.  The feed-forward is
down(PolyNorm(up(x))).  The logits are x's final layer norm times the embedding table.
"""
from __future__ import annotations

import json
import math
import os

import torch


def read_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def load_weights(folder: str, dtype=torch.float64) -> dict:
    """name -> tensor, floating tensors widened to ``dtype``."""
    from safetensors import safe_open
    out = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            out[name] = t.to(dtype) if t.is_floating_point() else t
    return out


# --------------------------------------------------------------------------
# mechanisms
# --------------------------------------------------------------------------
def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w; var is the mean squared deviation; no bias."""
    mu = x.mean(-1, keepdim=True)
    dev = x - mu
    var = (dev * dev).mean(-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * w


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last dimension, no weight."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def token_shift(h, mu):
    """h_t + (h_{t-1} - h_t) * mu, with h_{-1} = 0; the predecessor is taken before the mixing."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu


def rotate_half_layout(v, positions, base, dims, factor):
    """v [T, heads, dim].  Among the first ``dims`` dimensions of each head, dimension i is paired
    with i + dims/2; the pair is turned by the angle position * base^(-2i/dims) / factor."""
    half = dims // 2
    out = v.clone()
    for i in range(half):
        f = base ** (-2.0 * i / dims) / factor
        a = positions.to(v.dtype) * f
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, w = v[..., i], v[..., i + half]
        out[..., i] = u * c - w * s
        out[..., i + half] = w * c + u * s
    return out


def sigmoid_attention(q, k, v, scale, bias, window=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv], bias [H].  Token t takes sum over j <= t of
    sigmoid(q_t . k_j * scale + bias_h) v_j; query head h reads key/value head h // (H / G).
    ``window`` (not part of the design; the library's mixer offers it): only the last ``window`` keys, t included."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros((T, H, v.shape[-1]), dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        for t in range(T):
            lo = 0 if window is None else max(0, t - window + 1)
            s = (k[lo:t + 1, g] @ q[t, h]) * scale + bias[h]
            out[t, h] = torch.sigmoid(s) @ v[lo:t + 1, g]
    return out


def decayed_linear_attention(q, k, v, decay):
    """q, k [T, H, d], v [T, H, dv], decay [H].  S_t = decay S_{t-1} + k_t v_t^T, o_t = S_t^T q_t."""
    T, H, d = q.shape
    dv = v.shape[-1]
    out = torch.zeros((T, H, dv), dtype=q.dtype)
    for h in range(H):
        S = torch.zeros((d, dv), dtype=q.dtype)
        for t in range(T):
            S = decay[h] * S + torch.outer(k[t, h], v[t, h])
            out[t, h] = S.t() @ q[t, h]
    return out


def silu(z):
    return z * torch.sigmoid(z)


def poly_norm(z, coef, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e, N = division by the vector's root mean square."""
    a, b, c, e = (coef[i] for i in range(4))
    return a * unit_rms(z, eps) + b * unit_rms(z * z, eps) + c * unit_rms(z * z * z, eps) + e


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
def left_mixer(W, p, h, positions, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].t()).view(T, H, d)
    k = (h @ W[p + "k"].t()).view(T, G, d)
    v = (h @ W[p + "v"].t()).view(T, G, dv)
    rot = m.get("rot")
    if rot:
        factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        q = rotate_half_layout(q, positions, float(rot["base"]), int(rot["dims"]), factor)
        k = rotate_half_layout(k, positions, float(rot["base"]), int(rot["dims"]), factor)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    o = sigmoid_attention(q, k, v, float(m["scale"]), W[p + "pb"])
    return o.reshape(T, H * dv) @ W[p + "o"].t()


def right_mixer(W, p, h, m, eps):
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W[p + "q"].t()).view(T, H, d)
    k = silu(h @ W[p + "k"].t()).view(T, H, d)
    v = silu(h @ W[p + "v"].t()).view(T, H, dv)
    o = decayed_linear_attention(q, k, v, torch.tensor(m["decay"], dtype=h.dtype)).reshape(T, H * dv)
    o = unit_rms(o, eps) * W[p + "norm"] * torch.sigmoid(h @ W[p + "g"].t())
    return o @ W[p + "o"].t()


def feed_forward(W, p, x, eps):
    return poly_norm(x @ W[p + "up"].t(), W[p + "act"], eps) @ W[p + "down"].t()


def forward(W: dict, cfg: dict, tokens, return_layers: bool = False):
    """Logits [T, vocab] of one sequence from its first token (and the residual stream after every layer)."""
    eps, alpha = float(cfg["norm"]["eps"]), float(cfg["postln_alpha"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    x = W["embed"][tokens]
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        assert layer["type"] == "parallel"
        m = layer["mixer"]
        h = token_shift(x, W[p + "shift"])
        y = (float(m["left_scale"]) * left_mixer(W, p + "mix.left.", h, positions, m["left"], eps)
             + float(m["right_scale"]) * right_mixer(W, p + "mix.right.", h, m["right"], eps))
        x = layer_norm(alpha * x + y, W[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            assert layer["mlp"]["kind"] == "dense"
            x = layer_norm(alpha * x + feed_forward(W, p + "mlp.", x, eps), W[p + "norm2"], eps)
        streams.append(x)
    logits = layer_norm(x, W["final.norm"], eps) @ W["embed"].t()
    return (logits, torch.stack(streams)) if return_layers else logits
