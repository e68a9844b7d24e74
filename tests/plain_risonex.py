"""A plain, slow implementation of the Risonex decoder: whole sequences, no cache, no batching, one function
per mechanism, torch on the CPU.  It shares no code with the engine and is what the engine is compared with.

``forward(config, tensors, tokens)`` takes the dict of config.json, a dict name -> tensor and the token ids of
one sequence and returns the logits of every position (and, when asked, the residual stream after every run
of a layer).  ``dtype`` float64 gives the yardstick against which float32 rounding is measured.
"""
from __future__ import annotations

import math

import torch


# ------------------------------------------------------------------ small pieces
def rms_div(x, eps):
    """x divided by its root mean square over the last dimension (eps inside the root)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """The layer's norm: the weight is stored around zero and acts as 1 + w."""
    return rms_div(x, eps) * (1.0 + w)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def sinusoid(positions, width, dtype):
    """Entry 2i: sin(p * 10000^(-2i/width)); entry 2i+1: cos of the same angle."""
    out = torch.zeros((len(positions), width), dtype=dtype)
    p = torch.as_tensor(positions, dtype=dtype)[:, None]
    two_i = torch.arange(0, width, 2, dtype=dtype)
    angle = p * torch.pow(torch.tensor(10000.0, dtype=dtype), -two_i / width)[None, :]
    out[:, 0::2] = torch.sin(angle)[:, :out[:, 0::2].shape[1]]
    out[:, 1::2] = torch.cos(angle)[:, :out[:, 1::2].shape[1]]
    return out


def embed(tokens, table, scale, width):
    x = table[torch.as_tensor(tokens, dtype=torch.long)] * scale
    return x + sinusoid(list(range(len(tokens))), width, x.dtype)


# ------------------------------------------------------------------ differential attention in chunks
def chunk_mask(n, size):
    """True where query i may see key j: j <= i and both in the same block of ``size`` positions."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & (i // size == j // size)


def diff_attention_core(q, k, v, scale, lam, size, eps, out_scale):
    """q [n, H, 2, d], k [n, G, 2, d], v [n, G, dv] -> [n, H, dv]: two softmax maps over the same values, their
    difference divided by its root mean square (``eps`` None: left as it is) and multiplied by ``out_scale``."""
    n, H, G = q.shape[0], q.shape[1], k.shape[1]
    see = chunk_mask(n, size)
    out = torch.zeros((n, H, v.shape[-1]), dtype=q.dtype)
    for head in range(H):
        g = head // (H // G)
        maps = []
        for which in range(2):
            s = (q[:, head, which] @ k[:, g, which].T) * scale
            s = s.masked_fill(~see, float("-inf"))
            maps.append(torch.softmax(s, dim=-1) @ v[:, g])
        o = maps[0] - lam * maps[1]
        out[:, head] = (o if eps is None else rms_div(o, eps)) * out_scale
    return out


def diff_lambda(t, diff):
    return torch.exp((t["lq1"] * t["lk1"]).sum()) - torch.exp((t["lq2"] * t["lk2"]).sum()) + diff


def diff_attention(h, t, m, eps, store=None):
    """``t``: the mixer's tensors by local name (q, k, v, o, q.norm, k.norm, lq1, lk1, lq2, lk2); ``m``: its sizes.
    ``store`` (a 16-bit type): q, k, v and the heads' outputs take that type's values where a 16-bit engine stores
    them, which measures what that rounding alone does to the result."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    r = (lambda x: x.to(store).to(x.dtype)) if store is not None else (lambda x: x)
    q = r(rms_div((h @ t["q"].T).view(n, H, 2, d), eps) * t["q.norm"])
    k = r(rms_div((h @ t["k"].T).view(n, G, 2, d), eps) * t["k.norm"])
    v = r((h @ t["v"].T).view(n, G, dv))
    out = diff_attention_core(q, k, v, m["scale"], diff_lambda(t, m["diff"]), int(m["mask"]["size"]), eps, 1.0 - m["diff"])
    return r(out.reshape(n, H * dv)) @ t["o"].T


# ------------------------------------------------------------------ the state-space mixer
def causal_conv(u, w, b):
    """u [n, channels]; w [channels, taps], the last column weighs the current token; zeros before the start."""
    n, taps = u.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros((taps - 1, u.shape[1]), dtype=u.dtype), u], 0)
    out = torch.zeros_like(u)
    for j in range(taps):
        out = out + padded[j:j + n] * w[:, j]
    return out + b


def mamba2(h, t, m, eps):
    """``t``: in, conv, conv.b, dt_bias, A_log, D, norm, o."""
    P, dv, N, G, parts = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner, n = P * dv, h.shape[0]
    proj = h @ t["in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, t["conv"], t["conv.b"]))
    x = xbc[:, :inner].view(n, P, dv)
    B = xbc[:, inner:inner + G * N].view(n, G, N)
    C = xbc[:, inner + G * N:].view(n, G, N)
    dt = softplus(dt + t["dt_bias"])
    decay = torch.exp(-torch.exp(t["A_log"]) * dt)                  # [n, P]
    y = torch.zeros((n, P, dv), dtype=h.dtype)
    for head in range(P):
        g = head // (P // G)
        S = torch.zeros((N, dv), dtype=h.dtype)
        for i in range(n):
            S = decay[i, head] * S + dt[i, head] * torch.outer(B[i, g], x[i, head])
            y[i, head] = S.T @ C[i, g] + t["D"][head] * x[i, head]
    y = y.reshape(n, inner) * silu(z)
    y = rms_div(y.view(n, parts, inner // parts), eps).reshape(n, inner) * t["norm"]
    return y @ t["o"].T


# ------------------------------------------------------------------ feed-forwards
def dense_ff(h, t):
    return gelu_erf(h @ t["up"].T) @ t["down"].T


def gated_expert(h, t, prefix):
    return (silu(h @ t[prefix + "gate"].T) * (h @ t[prefix + "up"].T)) @ t[prefix + "down"].T


def route(h, t, r):
    """For every token the chosen experts and their weights."""
    s = torch.softmax(h @ t["router"].T, dim=-1)
    chosen = torch.topk(s + t["correction"], int(r["top"]), dim=-1).indices
    w = torch.gather(s, 1, chosen)
    return chosen, w / (w.sum(-1, keepdim=True) + 1e-20) * r["scale"]


def moe_ff(h, t, mlp):
    r = mlp["router"]
    real = int(r["experts"])             # the router has ``identity`` outputs more: experts that pass h on
    chosen, w = route(h, t, r)
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e, we in zip(chosen[i].tolist(), w[i]):
            out[i] += we * (h[i] if e >= real else gated_expert(h[i:i + 1], t, f"e{e}.")[0])
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ t["shared.sg"].T) * gated_expert(h, t, "shared.")
    return out


# ------------------------------------------------------------------ the model
def _local(tensors, prefix, dtype):
    return {k[len(prefix):]: v.to(dtype) for k, v in tensors.items() if k.startswith(prefix)}


def layer(x, i, spec, tensors, eps, dtype):
    h = norm_one_plus(x, tensors[f"l{i}.norm1"].to(dtype), eps)
    t = _local(tensors, f"l{i}.mix.", dtype)
    x = x + (diff_attention(h, t, spec["mixer"], eps) if spec["type"] == "attention" else mamba2(h, t, spec["mixer"], eps))
    mlp = spec.get("mlp")
    if mlp is not None:
        h = norm_one_plus(x, tensors[f"l{i}.norm2"].to(dtype), eps)
        t = _local(tensors, f"l{i}.mlp.", dtype)
        x = x + (dense_ff(h, t) if mlp["kind"] == "dense" else moe_ff(h, t, mlp))
    return x


def layer_runs(config):
    """The order in which layers run: (layer, starts a pass of the loop)."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    lo, hi, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, False) for i in range(lo)]
    for _ in range(times):
        runs += [(i, i == lo) for i in range(lo, hi)]
    return runs + [(i, False) for i in range(hi, n)]


def forward(config, tensors, tokens, dtype=torch.float32, streams=False):
    eps, width = float(config["norm"]["eps"]), int(config["width"])
    x0 = embed(tokens, tensors["embed"].to(dtype), float(config["embedding"]["scale"]), width)
    x, after = x0, []
    for i, starts_pass in layer_runs(config):
        if starts_pass:
            x = torch.cat([x, x0], -1) @ tensors["loop.in"].to(dtype).T
        x = layer(x, i, config["layers"][i], tensors, eps, dtype)
        after.append(x)
    logits = norm_one_plus(x, tensors["final.norm"].to(dtype), eps) @ tensors["head"].to(dtype).T
    return (logits, torch.stack(after)) if streams else logits
