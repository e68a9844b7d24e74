"""Small Risonex configurations, random weights for them, and model folders: for the tests only, written
without the library (the safetensors package writes the files)."""
import json
import os

import torch


def attention(heads, kv_heads, dim, vdim, block, diff=0.25, scale=None):
    return "attention", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
                         "scale": dim ** -0.5 if scale is None else scale, "mask": {"size": block}}


def mamba(heads, vdim, state, groups=1, conv=4, norm_groups=1):
    return "mamba2", {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, identity=0, scale=1.0, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top, "scale": scale}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def config(width, vocab, layers, loop=None, eps=1e-5, scale=1.0):
    out = {"architecture": "Risonex", "embedding": {"scale": scale}, "layers": layers, "norm": {"eps": eps}, "vocab": vocab,
           "width": width}
    if loop:
        out["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return out


# a layer before the loop (the stream is copied before it is changed), a layer without feed-forward, three query
# heads on a key head, a block of 50 positions (no multiple of a page) and one of 7, three of six router outputs
# chosen, one of them an identity, a shared expert; a second routed layer with one expert chosen and neither
TINY_A = config(96, 131, [
    layer(mamba(4, 24, 20, groups=1, conv=3, norm_groups=1), None),
    layer(attention(6, 2, 20, 36, 50, diff=0.2), moe(5, 3, 40, identity=1, scale=2.0, shared=24)),
    layer(mamba(6, 16, 33, groups=3, conv=5, norm_groups=4), dense(72)),
    layer(attention(2, 2, 64, 16, 7, diff=0.45, scale=0.2), moe(3, 1, 56)),
], loop=(1, 3, 2), eps=1e-6, scale=2.5)

# a width that the matrix kernels cannot tile, no loop; values 130 wide, a block of 200 positions (four pages),
# 80 values a head and a state of 130 in the recurrence, a convolution over two tokens, 70 router outputs
TINY_B = config(72, 97, [
    layer(attention(3, 1, 8, 130, 200, diff=0.1), dense(40)),
    layer(mamba(2, 80, 130, groups=2, conv=2, norm_groups=2), moe(66, 4, 8, identity=4, scale=0.7, shared=16)),
], eps=1e-4, scale=1.0)

# the sizes of real layers, few of them: 128-wide maps and values, a block of exactly one page; a state of 128, 64
# values a head; the loop is the first layer alone, three times
TINY_C = config(256, 211, [
    layer(mamba(8, 64, 128, groups=1, conv=4, norm_groups=8), dense(320)),
    layer(attention(4, 1, 128, 128, 64, diff=0.3), moe(4, 2, 96, identity=2, scale=1.5, shared=64)),
], loop=(0, 1, 3), eps=1e-5, scale=3.0)

ALL = {"A": TINY_A, "B": TINY_B, "C": TINY_C}


def mixer_weights(kind, m, w, g, dtype, sharp=1.0):
    """local name -> tensor of one mixer."""
    mat = lambda n, k, s=None: (torch.randn(n, k, generator=g) * (s if s is not None else k ** -0.5)).to(dtype)
    vec = lambda n, mean, s: (mean + s * torch.randn(n, generator=g)).to(dtype)
    if kind == "attention":
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        return {"q": mat(H * 2 * d, w, sharp * w ** -0.5), "k": mat(G * 2 * d, w, sharp * w ** -0.5), "v": mat(G * dv, w),
                "o": mat(w, H * dv), "q.norm": vec(d, 1.0, 0.2), "k.norm": vec(d, 1.0, 0.2),
                "lq1": vec(d, 0.0, 0.3), "lk1": vec(d, 0.0, 0.3), "lq2": vec(d, 0.0, 0.3), "lk2": vec(d, 0.0, 0.3)}
    P, dv, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner, ch = P * dv, P * dv + 2 * G * N
    return {"in": mat(inner + ch + P, w), "conv": mat(ch, m["conv"], 0.5), "conv.b": vec(ch, 0.0, 0.2),
            "dt_bias": vec(P, -2.0, 1.5), "A_log": vec(P, 0.0, 0.5), "D": vec(P, 1.0, 0.3), "norm": vec(inner, 1.0, 0.2),
            "o": mat(w, inner)}


def mlp_weights(mlp, w, g, dtype, fixed_choice=False):
    """local name -> tensor of one feed-forward.  ``fixed_choice``: the correction is far apart from output to output,
    so that the same outputs are chosen for every token whatever the rounding (their weights still follow the token)."""
    mat = lambda n, k, s=None: (torch.randn(n, k, generator=g) * (s if s is not None else k ** -0.5)).to(dtype)
    if mlp["kind"] == "dense":
        return {"up": mat(mlp["ff"], w), "down": mat(w, mlp["ff"])}
    r = mlp["router"]
    n_out, ff = r["experts"] + r.get("identity", 0), mlp["expert"]["ff"]
    out = {"router": mat(n_out, w, 2.0 * w ** -0.5)}
    if fixed_choice:
        order = torch.randperm(n_out, generator=g)
        out["correction"] = (order.float() * 3.0).to(dtype)
    else:
        out["correction"] = (0.3 * torch.randn(n_out, generator=g)).to(dtype)
    for e in range(r["experts"]):
        out.update({f"e{e}.gate": mat(ff, w), f"e{e}.up": mat(ff, w), f"e{e}.down": mat(w, ff)})
    if mlp.get("shared"):
        f = mlp["shared"]["ff"]
        out.update({"shared.gate": mat(f, w), "shared.up": mat(f, w), "shared.down": mat(w, f), "shared.sg": mat(1, w)})
    return out


def random_weights(cfg, seed, dtype=torch.bfloat16, sharp=1.0, fixed_choice=False):
    """name -> tensor as a file of the design holds it.  ``sharp`` scales the query and key matrices."""
    g = torch.Generator().manual_seed(seed)
    w, V = cfg["width"], cfg["vocab"]
    vec = lambda n, mean, s: (mean + s * torch.randn(n, generator=g)).to(dtype)
    out = {"embed": (torch.randn(V, w, generator=g)).to(dtype), "final.norm": vec(w, 0.0, 0.1),
           "head": (torch.randn(V, w, generator=g) * w ** -0.5).to(dtype)}
    if cfg.get("loop"):
        out["loop.in"] = (torch.randn(w, 2 * w, generator=g) * (2 * w) ** -0.5 * 1.4).to(dtype)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        out[p + "norm1"] = vec(w, 0.0, 0.1)
        out.update({p + "mix." + k: v for k, v in mixer_weights(L["type"], L["mixer"], w, g, dtype, sharp).items()})
        if L["mlp"] is not None:
            out[p + "norm2"] = vec(w, 0.0, 0.1)
            out.update({p + "mlp." + k: v for k, v in mlp_weights(L["mlp"], w, g, dtype, fixed_choice).items()})
    return out


def write_model(folder, cfg, weights):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))


def widen(weights, dtype=torch.float64):
    return {k: v.to(dtype) for k, v in weights.items()}


def row_error(got, ref):
    """For each row the root mean square of the difference (its mean taken off), relative to the reference's
    own spread: the measure by which logits are compared."""
    d = got.double() - ref.double()
    d = d - d.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / ref.double().std()).max().item()
