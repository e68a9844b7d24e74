"""Typed configuration of the Risonex decoder, read from its own config.json keys.

A model of this design is a list of pre-norm layers over a residual stream of ``width``: x <- x + mixer(norm1(x)),
then, if the layer has a feed-forward, x <- x + ff(norm2(x)); every norm is an RMS norm whose weight is stored
around zero and acts as 1 + w (``norm.eps``).  ``layers[i].type`` names the mixer, ``layers[i].mixer`` its sizes:

* ``attention``: differential attention of two softmax maps over the same values (``heads``, ``kv_heads``, ``dim``
  per map, ``vdim``, ``scale``, ``diff``: the constant in lambda and in the output's factor 1 - diff), q and k
  RMS-normed per head and map with a weight, no rotation, keys visible within blocks of ``mask.size`` positions;
* ``mamba2``: the selective state-space mixer (``heads``, ``vdim``, ``state``, ``groups``, ``conv`` taps,
  ``norm_groups``).

``layers[i].mlp`` is null, ``{"kind": "dense", "ff"}`` (down(gelu(up))) or ``{"kind": "moe", "expert": {"ff"},
"router": {"experts", "identity", "top", "scale"}, "shared": {"ff"}}``.  The embedding is multiplied by
``embedding.scale`` and gets sinusoidal positions.  ``loop`` {start, stop, times}: the layers start .. stop - 1 run
``times`` times in a row with the same weights and a cache of their own each time; before the first layer of each
pass x <- W [x; x0] with x0 the embedding's output.  Tensor names: ``embed``, ``loop.in``, ``final.norm``, ``head``,
and per layer ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass

from .spec import ConfigError, LayerSpec, ModelSpec, PartSpec, ScheduleEntry, SubLayerSpec

_DTYPES = ("float32", "float16", "bfloat16")
POSITION_BASE = 10000.0          # the design fixes the sinusoid's base


def _need(d, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json: {where} lacks '{key}'")
    return d[key]


@dataclass(frozen=True)
class RisonexConfig:
    width: int
    vocab: int
    norm_eps: float
    embedding_scale: float
    layers: tuple                   # the layers as config.json lists them (plain dicts)
    loop: dict | None = None        # {"start", "stop", "times"} or None
    max_positions: int = 0          # the design sets no bound; an optional key may
    torch_dtype: str | None = None
    eos_token_ids: tuple = ()
    architecture: str = "Risonex"

    context_key = "max_positions"

    @classmethod
    def from_dict(cls, c: dict) -> "RisonexConfig":
        layers = _need(c, "layers", "the model")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        eos = c.get("eos_token_id")
        loop = c.get("loop")
        cfg = cls(width=int(_need(c, "width", "the model")), vocab=int(_need(c, "vocab", "the model")),
                  norm_eps=float(_need(_need(c, "norm", "the model"), "eps", "norm")),
                  embedding_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                  layers=tuple(copy.deepcopy(layers)), loop=copy.deepcopy(loop) if loop else None,
                  max_positions=int(c.get("max_positions") or 0), torch_dtype=c.get("torch_dtype"),
                  eos_token_ids=() if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos])),
                  architecture=c.get("architecture") or (c.get("architectures") or ["Risonex"])[0])
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
            kind, m = _need(layer, "type", where), _need(layer, "mixer", where)
            if kind == "attention":
                for k in ("heads", "kv_heads", "dim", "vdim", "scale", "diff"):
                    _need(m, k, where + " mixer")
                if int(m["heads"]) <= 0 or int(m["kv_heads"]) <= 0 or int(m["heads"]) % int(m["kv_heads"]):
                    raise ConfigError(f"{where}: heads must be a positive multiple of kv_heads")
                if int(_need(_need(m, "mask", where + " mixer"), "size", where + " mask")) < 1:
                    raise ConfigError(f"{where}: mask.size must be positive")
            elif kind == "mamba2":
                for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups"):
                    _need(m, k, where + " mixer")
                if int(m["heads"]) % int(m["groups"]) or (int(m["heads"]) * int(m["vdim"])) % int(m["norm_groups"]):
                    raise ConfigError(f"{where}: groups must divide heads, norm_groups heads * vdim")
            else:
                raise ConfigError(f"{where}: mixer type {kind!r} is not built ('attention' and 'mamba2' are)")
            mlp = layer.get("mlp")
            if mlp is not None:
                ff_kind = _need(mlp, "kind", where + " mlp")
                if ff_kind == "dense":
                    if int(_need(mlp, "ff", where + " mlp")) <= 0:
                        raise ConfigError(f"{where} mlp: ff must be positive")
                elif ff_kind == "moe":
                    r = _need(mlp, "router", where + " mlp")
                    for k in ("experts", "top"):
                        _need(r, k, where + " router")
                    _need(_need(mlp, "expert", where + " mlp"), "ff", where + " expert")
                    if not 1 <= int(r["top"]) <= int(r["experts"]) + int(r.get("identity", 0)):
                        raise ConfigError(f"{where} router: top between 1 and experts + identity")
                    if mlp.get("shared"):
                        _need(mlp["shared"], "ff", where + " shared")
                else:
                    raise ConfigError(f"{where}: feed-forward kind {ff_kind!r} is not built ('dense' and 'moe' are)")
        if self.loop:
            lo, hi, times = (int(_need(self.loop, k, "loop")) for k in ("start", "stop", "times"))
            if not (0 <= lo < hi <= len(self.layers)) or times < 1:
                raise ConfigError("loop: 0 <= start < stop <= number of layers, times at least 1")

    def runs(self) -> list:
        """The order in which layers run: (layer, whether this run begins a pass of the loop)."""
        n = len(self.layers)
        if not self.loop:
            return [(i, False) for i in range(n)]
        lo, hi, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        out = [(i, False) for i in range(lo)]
        for _ in range(times):
            out += [(i, i == lo) for i in range(lo, hi)]
        return out + [(i, False) for i in range(hi, n)]

    def summary(self) -> list:
        """(label, value) lines for the command line's report."""
        kinds = [layer["type"] for layer in self.layers]
        heads = [int(layer["mixer"]["heads"]) for layer in self.layers]
        span = lambda xs: str(xs[0]) if len(set(xs)) == 1 else f"{min(xs)}..{max(xs)}"
        return [("Layers", f"{len(self.layers)} ({len(self.runs())} runs; " + ", ".join(
                    f"{kinds.count(k)} {k}" for k in sorted(set(kinds))) + ")"),
                ("Dimensions", self.width), ("Heads", span(heads)), ("Vocab size", self.vocab)]

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        out = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
               "layers": copy.deepcopy(list(self.layers)), "norm": {"eps": self.norm_eps}, "vocab": self.vocab,
               "width": self.width}
        if self.loop:
            out["loop"] = copy.deepcopy(self.loop)
        if self.max_positions:
            out["max_positions"] = self.max_positions
        if self.torch_dtype is not None:
            out["torch_dtype"] = self.torch_dtype
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    # ------------------------------------------------------------------ the model as data
    def _norm(self, prefix: str, name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": self.width, "eps": self.norm_eps, "name": name, "one_plus": True}, prefix)

    def _mixer(self, p: str, layer: dict) -> PartSpec:
        m, w, eps = layer["mixer"], self.width, self.norm_eps
        if layer["type"] == "attention":
            diff = float(m["diff"])
            return PartSpec("diff_attention", {
                "hidden_size": w, "n_heads": int(m["heads"]), "n_kv_heads": int(m["kv_heads"]), "head_dim": int(m["dim"]),
                "v_head_dim": int(m["vdim"]), "scale": float(m["scale"]), "maps": 2, "lambda_init": diff,
                "qk_norm_eps": eps, "out_norm_eps": eps, "out_scale": 1.0 - diff, "block": int(m["mask"]["size"]),
                "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm",
                          "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2"}}, p + "mix.")
        return PartSpec("state_space", {
            "hidden_size": w, "n_heads": int(m["heads"]), "head_dim": int(m["vdim"]), "n_state": int(m["state"]),
            "n_groups": int(m["groups"]), "conv_taps": int(m["conv"]), "norm_groups": int(m["norm_groups"]), "norm_eps": eps,
            "names": {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "a_log": "A_log", "d": "D",
                      "norm": "norm", "o": "o"}}, p + "mix.")

    def _feed_forward(self, p: str, mlp: dict) -> PartSpec:
        if mlp["kind"] == "dense":
            return PartSpec("dense_mlp", {"hidden_size": self.width, "intermediate_size": int(mlp["ff"]), "activation": "gelu",
                                          "names": {"up": "up", "down": "down"}}, p + "mlp.")
        r, shared = mlp["router"], mlp.get("shared") or {}
        return PartSpec("routed_experts", {
            "hidden_size": self.width, "n_experts": int(r["experts"]), "expert_ff": int(mlp["expert"]["ff"]),
            "top": int(r["top"]), "n_identity": int(r.get("identity", 0)), "route_scale": float(r.get("scale", 1.0)),
            "correction": True, "shared_ff": int(shared.get("ff", 0)), "shared_gate": True,
            "names": {"router": "router", "correction": "correction", "expert": "e{}.", "shared": "shared.",
                      "shared_gate": "shared.sg"}}, p + "mlp.")

    def _layer_spec(self, i: int, layer: dict) -> LayerSpec:
        p = f"l{i}."
        subs = [SubLayerSpec("mixer", self._mixer(p, layer), self._norm(p, "norm1"))]
        if layer.get("mlp") is not None:
            subs.append(SubLayerSpec("feed_forward", self._feed_forward(p, layer["mlp"]), self._norm(p, "norm2")))
        return LayerSpec("pre_norm", tuple(subs), None)

    def model_spec(self) -> ModelSpec:
        reinject = PartSpec("reinject", {"hidden_size": self.width, "name": "in"}, "loop.")
        spec = ModelSpec(
            hidden_size=self.width, vocab_size=self.vocab, max_positions=self.max_positions,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab, "hidden_size": self.width, "name": "embed",
                                             "scale": self.embedding_scale, "positions": "sinusoidal",
                                             "position_base": POSITION_BASE}, ""),
            layers=tuple(self._layer_spec(i, layer) for i, layer in enumerate(self.layers)),
            schedule=tuple(ScheduleEntry(i, None, reinject if starts else None) for i, starts in self.runs()),
            final_norm=self._norm("final.", "norm"),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "hidden_size": self.width, "tied": False, "name": "head"}, ""),
            stop_token_ids=self.eos_token_ids)
        spec.validate()
        return spec
