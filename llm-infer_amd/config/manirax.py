"""Typed configuration of the Manirax decoder, read from its own config.json keys.

A model of this design is a list of layers (``layers``: each names its mixer's type with the mixer's
sizes and its feed-forward, or null for none), the residual stream's ``width``, the vocabulary ``vocab``,
the norms' ``norm.eps`` and ``postln_alpha``, the factor on the stream's own share of every residual sum.
Every size and constant is read from the file; nothing here knows a particular model's values.

The layer: x <- LN(alpha x + mixer(shift(x))), then x <- LN(alpha x + ff(x)) if it has a feed-forward; LN is
a layer norm with a weight and no bias.  The mixer type "parallel" is two mixers on the same token-shifted
input whose results are added with the scales ``left_scale`` and ``right_scale``: attention with sigmoid
weights (``left``: grouped-query heads, rotation of part of each head in the half layout with linearly
scaled positions, unit-RMS q and k, a bias per head) and linear attention with a constant decay per head
(``right``).  The feed-forward kind "dense" is down(PolyNorm(up(x))).  The logits are the final norm's rows
times the embedding table.  Tensor names: ``embed``, ``final.norm``, and per layer ``l<i>.norm1``,
``l<i>.norm2``, ``l<i>.shift``, ``l<i>.mix.left.{q,k,v,o,pb}``, ``l<i>.mix.right.{q,k,v,g,o,norm}``,
``l<i>.mlp.{up,down,act}``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass

from .spec import ConfigError, LayerSpec, ModelSpec, PartSpec, ScheduleEntry, SubLayerSpec

_DTYPES = ("float32", "float16", "bfloat16")


def _need(d: dict, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json: {where} lacks '{key}'")
    return d[key]


@dataclass(frozen=True)
class ManiraxConfig:
    width: int
    vocab: int
    norm_eps: float
    postln_alpha: float
    layers: tuple                   # the layers as config.json lists them (plain dicts)
    max_positions: int = 0          # the design sets no bound; an optional key may
    torch_dtype: str | None = None
    eos_token_ids: tuple = ()
    architecture: str = "Manirax"

    @classmethod
    def from_dict(cls, c: dict) -> "ManiraxConfig":
        layers = _need(c, "layers", "the model")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        eos = c.get("eos_token_id")
        cfg = cls(width=int(_need(c, "width", "the model")), vocab=int(_need(c, "vocab", "the model")),
                  norm_eps=float(_need(_need(c, "norm", "the model"), "eps", "norm")),
                  postln_alpha=float(_need(c, "postln_alpha", "the model")),
                  layers=tuple(copy.deepcopy(layers)), max_positions=int(c.get("max_positions") or 0),
                  torch_dtype=c.get("torch_dtype"),
                  eos_token_ids=() if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos])),
                  architecture=c.get("architecture") or (c.get("architectures") or ["Manirax"])[0])
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.width <= 0 or self.vocab <= 0:
            raise ConfigError("width and vocab must be positive")
        if not self.norm_eps >= 0:
            raise ConfigError("norm.eps must not be negative")
        if self.torch_dtype is not None and self.torch_dtype not in _DTYPES:
            raise ConfigError(f"Unsupported torch_dtype: {self.torch_dtype}")
        for i, layer in enumerate(self.layers):
            where = f"layer {i}"
            if _need(layer, "type", where) != "parallel":
                raise ConfigError(f"{where}: mixer type {layer['type']!r} is not built ('parallel' is)")
            m = _need(layer, "mixer", where)
            left, right = _need(m, "left", where + " mixer"), _need(m, "right", where + " mixer")
            for k in ("left_scale", "right_scale"):
                _need(m, k, where + " mixer")
            for k in ("heads", "kv_heads", "dim", "vdim", "scale"):
                _need(left, k, where + " left")
            if int(left["heads"]) <= 0 or int(left["kv_heads"]) <= 0 or int(left["heads"]) % int(left["kv_heads"]):
                raise ConfigError(f"{where} left: heads must be a positive multiple of kv_heads")
            rot = left.get("rot")
            if rot:
                dims = int(_need(rot, "dims", where + " rot"))
                if dims % 2 or not 0 <= dims <= int(left["dim"]) or not float(_need(rot, "base", where + " rot")) > 0:
                    raise ConfigError(f"{where} rot: dims even and within dim, base positive")
                scaling = rot.get("scaling")
                if scaling and not float(_need(scaling, "factor", where + " rot.scaling")) > 0:
                    raise ConfigError(f"{where} rot.scaling: factor must be positive")
            for k in ("heads", "dim", "vdim", "decay"):
                _need(right, k, where + " right")
            if len(right["decay"]) != int(right["heads"]):
                raise ConfigError(f"{where} right: one decay for each of the {right['heads']} heads")
            mlp = layer.get("mlp")
            if mlp is not None:
                if _need(mlp, "kind", where + " mlp") != "dense":
                    raise ConfigError(f"{where}: feed-forward kind {mlp['kind']!r} is not built ('dense' is)")
                if int(_need(mlp, "ff", where + " mlp")) <= 0:
                    raise ConfigError(f"{where} mlp: ff must be positive")

    context_key = "max_positions"                 # the optional key (and field) that bounds a sequence's positions

    def summary(self) -> list:
        """(label, value) lines for the command line's report."""
        left = [layer["mixer"]["left"] for layer in self.layers]
        right = [layer["mixer"]["right"] for layer in self.layers]
        span = lambda xs: str(xs[0]) if len(set(xs)) == 1 else f"{min(xs)}..{max(xs)}"
        return [("Layers", len(self.layers)), ("Dimensions", self.width),
                ("Heads", span([int(l["heads"]) for l in left]) + " sigmoid + " + span([int(r["heads"]) for r in right]) + " linear"),
                ("KV Heads", span([int(l["kv_heads"]) for l in left])), ("Vocab size", self.vocab)]

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        out = {"architecture": self.architecture, "layers": copy.deepcopy(list(self.layers)),
               "norm": {"eps": self.norm_eps}, "postln_alpha": self.postln_alpha, "vocab": self.vocab,
               "width": self.width}
        if self.max_positions:
            out["max_positions"] = self.max_positions
        if self.torch_dtype is not None:
            out["torch_dtype"] = self.torch_dtype
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    # ------------------------------------------------------------------ the model as data
    def _layer_spec(self, i: int, layer: dict) -> LayerSpec:
        p, w, eps = f"l{i}.", self.width, self.norm_eps
        m = layer["mixer"]
        left, right = m["left"], m["right"]
        rot = left.get("rot")
        position = PartSpec("none")
        if rot and int(rot["dims"]) > 0:
            factor = float((rot.get("scaling") or {}).get("factor", 1.0))
            position = PartSpec("rope", {"theta": float(rot["base"]), "rotary_dim": int(rot["dims"]),
                                         "head_dim": int(left["dim"]), "pairing": "half", "scaling_factor": factor})
        attn = PartSpec("sigmoid_attention", {
            "hidden_size": w, "n_heads": int(left["heads"]), "n_kv_heads": int(left["kv_heads"]),
            "head_dim": int(left["dim"]), "v_head_dim": int(left["vdim"]), "scale": float(left["scale"]),
            "unit_norm_eps": eps, "head_bias": True,
            "names": {"q": "q", "k": "k", "v": "v", "o": "o", "bias": "pb"}}, p + "mix.left.")
        lin = PartSpec("decay_attention", {
            "hidden_size": w, "n_heads": int(right["heads"]), "head_dim": int(right["dim"]),
            "v_head_dim": int(right["vdim"]), "decay": tuple(float(x) for x in right["decay"]), "norm_eps": eps,
            "names": {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm"}}, p + "mix.right.")
        both = PartSpec("parallel", {"branches": ((attn, float(m["left_scale"])), (lin, float(m["right_scale"])))},
                        p + "mix.")
        mixer = PartSpec("token_shift", {"hidden_size": w, "inner": both, "name": "shift"}, p)
        norm = lambda name: PartSpec("layernorm", {"size": w, "eps": eps, "name": name}, p)
        subs = [SubLayerSpec("mixer", mixer, post_norm=norm("norm1"))]
        if layer.get("mlp") is not None:
            ffn = PartSpec("poly_mlp", {"hidden_size": w, "intermediate_size": int(layer["mlp"]["ff"]), "eps": eps,
                                        "names": {"up": "up", "down": "down", "act": "act"}}, p + "mlp.")
            subs.append(SubLayerSpec("feed_forward", ffn, post_norm=norm("norm2")))
        return LayerSpec("post_norm", tuple(subs), position, {"alpha": self.postln_alpha})

    def model_spec(self) -> ModelSpec:
        spec = ModelSpec(
            hidden_size=self.width, vocab_size=self.vocab, max_positions=self.max_positions,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab, "hidden_size": self.width, "name": "embed"}, ""),
            layers=tuple(self._layer_spec(i, layer) for i, layer in enumerate(self.layers)),
            schedule=tuple(ScheduleEntry(i) for i in range(len(self.layers))),
            final_norm=PartSpec("layernorm", {"size": self.width, "eps": self.norm_eps, "name": "norm"}, "final."),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "hidden_size": self.width, "tied": True}, "lm_head."),
            stop_token_ids=self.eos_token_ids)
        spec.validate()
        return spec
