"""Small Manirax configurations, random weights for them, and model folders: for the tests only, written
without the library (the safetensors package writes the files)."""
import json
import os

import torch


def left(heads, kv_heads, dim, vdim, scale=None, rot=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
           "scale": dim ** -0.5 if scale is None else scale}
    if rot is not None:
        out["rot"] = rot
    return out


def right(heads, dim, vdim, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def layer(l, r, left_scale, right_scale, ff):
    return {"type": "parallel", "mixer": {"left": l, "right": r, "left_scale": left_scale, "right_scale": right_scale},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def config(width, vocab, layers, eps=1e-5, alpha=1.0):
    return {"architecture": "Manirax", "layers": layers, "norm": {"eps": eps}, "postln_alpha": alpha, "vocab": vocab,
            "width": width}


# heads 6 on 2, key size 40 (no multiple of 16) beside value size 24, 16 of 40 dimensions rotated with scaled
# positions; three linear heads 24 x 40; the second layer has no feed-forward and other sizes
TINY_P = config(72, 131, [
    layer(left(6, 2, 40, 24, rot={"base": 10000.0, "dims": 16, "scaling": {"factor": 2.0}}),
          right(3, 24, 40, [0.5, 0.9, 0.99]), 0.7, 1.3, 100),
    layer(left(2, 1, 16, 32, scale=0.3, rot={"base": 500.0, "dims": 16}),
          right(2, 8, 16, [0.95, 0.8]), 1.0, 0.5, None),
], eps=1e-6, alpha=1.7)

# every head its own keys, whole heads rotated and no scaling; one linear head with decay 1; alpha 1; no rotation
# at all in the second layer; three layers
TINY_Q = config(64, 97, [
    layer(left(4, 4, 32, 48, rot={"base": 100.0, "dims": 32}), right(1, 16, 16, [1.0]), 1.0, 1.0, 48),
    layer(left(3, 1, 48, 16), right(4, 16, 8, [0.3, 0.6, 0.9, 0.97]), 0.5, 2.0, 136),
    layer(left(1, 1, 64, 64, rot={"base": 2e5, "dims": 2, "scaling": {"factor": 8.0}}),
          right(2, 32, 32, [0.999, 0.5]), 1.2, 0.8, 64),
], eps=1e-4, alpha=1.0)

# wider heads (the sizes of real layers, few of them): 128-wide keys and values, a linear state of 128 x 128
TINY_R = config(256, 211, [
    layer(left(4, 2, 128, 128, rot={"base": 10000.0, "dims": 64, "scaling": {"factor": 3.0}}),
          right(2, 128, 128, [0.9, 0.99]), 0.9, 1.1, 384),
], eps=1e-5, alpha=2.0)

ALL = {"P": TINY_P, "Q": TINY_Q, "R": TINY_R}


def random_weights(cfg, seed, dtype=torch.bfloat16, sharp=1.0):
    """name -> tensor as a file of the design holds it.  ``sharp`` scales the query and key matrices."""
    g = torch.Generator().manual_seed(seed)
    w, V = cfg["width"], cfg["vocab"]

    def mat(n, k, s=None):
        return (torch.randn(n, k, generator=g) * (s if s is not None else k ** -0.5)).to(dtype)

    def vec(n, mean, s):
        return (mean + s * torch.randn(n, generator=g)).to(dtype)

    out = {"embed": mat(V, w, 1.0), "final.norm": vec(w, 1.0, 0.1)}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        l, r = L["mixer"]["left"], L["mixer"]["right"]
        out[p + "norm1"] = vec(w, 1.0, 0.1)
        out[p + "shift"] = torch.rand(w, generator=g).to(dtype)
        out[p + "mix.left.q"] = mat(l["heads"] * l["dim"], w, sharp * w ** -0.5)
        out[p + "mix.left.k"] = mat(l["kv_heads"] * l["dim"], w, sharp * w ** -0.5)
        out[p + "mix.left.v"] = mat(l["kv_heads"] * l["vdim"], w)
        out[p + "mix.left.pb"] = vec(l["heads"], -1.0, 1.0)
        out[p + "mix.left.o"] = mat(w, l["heads"] * l["vdim"])
        out[p + "mix.right.q"] = mat(r["heads"] * r["dim"], w)
        out[p + "mix.right.k"] = mat(r["heads"] * r["dim"], w)
        out[p + "mix.right.v"] = mat(r["heads"] * r["vdim"], w)
        out[p + "mix.right.g"] = mat(r["heads"] * r["vdim"], w)
        out[p + "mix.right.o"] = mat(w, r["heads"] * r["vdim"])
        out[p + "mix.right.norm"] = vec(r["heads"] * r["vdim"], 1.0, 0.1)
        if L["mlp"] is not None:
            out[p + "norm2"] = vec(w, 1.0, 0.1)
            out[p + "mlp.up"] = mat(L["mlp"]["ff"], w)
            out[p + "mlp.down"] = mat(w, L["mlp"]["ff"])
            out[p + "mlp.act"] = torch.tensor([0.6, 0.3, -0.2, 0.1]).to(dtype) + vec(4, 0.0, 0.05)
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
