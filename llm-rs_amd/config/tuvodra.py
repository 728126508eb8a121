"""Typed configuration of the Tuvodra decoder, read from config.json.

A decoder whose layers are listed one by one, each with a mixer of one of three types and an optional gated
feed-forward; the residual stream is kept in `streams` copies joined by hyper-connections; every norm is an RMS norm
in `norm.groups` groups; the token table (scaled by `embedding.scale` on the way in) is also the output matrix.
Every size and every constant that the file gives is read here; nothing about the design lives in the engine.

config.json keys: architecture ("Tuvodra"), vocab, width, streams, embedding.scale, norm.eps, norm.groups and
layers[i] = {type: "mingru" | "mamba1" | "attention", mixer: {...}, mlp: null | {kind: "dense", ff}} with
  mingru:    width
  mamba1:    inner, state, conv, dt_rank
  attention: heads, kv_heads, dim, vdim, scale, mask.size
Tensors: embed, final.norm, and for layer i under "l<i>.": norm1, norm2, mix.*, mlp.{gate,up,down}, hc1.*, hc2.*.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, List

from .llama import ConfigError
from .spec import ExtraPart, LayerSpec, ModelSpec, PartSpec, RunSpec

MIXER_TYPES = ("mingru", "mamba1", "attention")
# The file gives no longest sequence: positions enter only through distances and state.
UNBOUNDED_POSITIONS = 1 << 24


def _need(d: Dict[str, Any], key: str, where: str):
    if not isinstance(d, dict) or d.get(key) is None:
        raise ConfigError(f"missing config key: {where}{key}")
    return d[key]


class TuvodraConfig:
    architecture = "Tuvodra"

    def __init__(self, d: Dict[str, Any]):
        self.raw = copy.deepcopy(d)
        self.vocab = int(_need(d, "vocab", ""))
        self.width = int(_need(d, "width", ""))
        self.streams = int(_need(d, "streams", ""))
        self.embedding_scale = float(_need(_need(d, "embedding", ""), "scale", "embedding."))
        norm = _need(d, "norm", "")
        self.eps = float(_need(norm, "eps", "norm."))
        self.groups = int(_need(norm, "groups", "norm."))
        self.layers: List[Dict[str, Any]] = list(_need(d, "layers", ""))
        self.validate()

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "TuvodraConfig":
        return cls(d)

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not 1 <= self.streams <= 16:
            raise ConfigError(f"streams must be 1 to 16, got {self.streams}")
        if self.groups <= 0 or self.width % self.groups:
            raise ConfigError(f"width {self.width} does not fall into norm.groups = {self.groups} equal parts")
        if not self.eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {self.eps}")
        if not self.layers:
            raise ConfigError("layers is empty")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]."
            kind = _need(layer, "type", where)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}type: unknown mixer {kind!r} (known: {', '.join(MIXER_TYPES)})")
            m = _need(layer, "mixer", where)
            keys = {"mingru": ("width",), "mamba1": ("inner", "state", "conv", "dt_rank"),
                    "attention": ("heads", "kv_heads", "dim", "vdim", "scale", "mask")}[kind]
            for key in keys:
                _need(m, key, where + "mixer.")
            if kind == "attention":
                if int(_need(m["mask"], "size", where + "mixer.mask.")) <= 0:
                    raise ConfigError(f"{where}mixer.mask.size must be positive")
                if int(m["heads"]) % int(m["kv_heads"]):
                    raise ConfigError(f"{where}mixer: {m['heads']} heads are no multiple of {m['kv_heads']} kv_heads")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{where}mlp.kind: unknown feed-forward {mlp.get('kind')!r} (known: dense)")
                _need(mlp, "ff", where + "mlp.")

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)

    # -- what the engine builds from -----------------------------------------------------------------------------
    def _mixer(self, i: int, kind: str, m: Dict[str, Any]) -> PartSpec:
        prefix = f"l{i}.mix"
        if kind == "mingru":
            return PartSpec("mingru", prefix, {"hidden_size": self.width, "width": int(m["width"])})
        if kind == "mamba1":
            return PartSpec("mamba1", prefix, {"hidden_size": self.width, "inner": int(m["inner"]), "state": int(m["state"]),
                                               "conv": int(m["conv"]), "dt_rank": int(m["dt_rank"])})
        names = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b", "r1": "r1", "r2": "r2"}
        return PartSpec("attention", prefix, {
            "hidden_size": self.width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]), "head_dim": int(m["dim"]),
            "value_dim": int(m["vdim"]), "window": int(m["mask"]["size"]), "position": None, "scale": float(m["scale"]),
            "bias": True, "qk_norm_eps": self.eps, "distance": "log", "names": names})

    def model_spec(self) -> ModelSpec:
        norm = lambda name: PartSpec("group_rmsnorm", name, {"size": self.width, "eps": self.eps, "groups": self.groups, "tensor": ""})
        link = lambda prefix: PartSpec("hyper", prefix, {"streams": self.streams})
        layers = []
        for i, layer in enumerate(self.layers):
            extra = [ExtraPart("mixer_connection", "connection", link(f"l{i}.hc1"))]
            ff = ff_norm = None
            mlp = layer.get("mlp")
            if mlp is not None:
                ff = PartSpec("swiglu", f"l{i}.mlp", {"hidden_size": self.width, "intermediate_size": int(mlp["ff"]),
                                                      "names": {"gate": "gate", "up": "up", "down": "down"}})
                ff_norm = norm(f"l{i}.norm2")
                extra.append(ExtraPart("feed_forward_connection", "connection", link(f"l{i}.hc2")))
            layers.append(LayerSpec("hyper", self._mixer(i, layer["type"], layer["mixer"]), ff, norm(f"l{i}.norm1"), ff_norm, tuple(extra)))
        return ModelSpec(hidden_size=self.width, vocab_size=self.vocab, max_positions=UNBOUNDED_POSITIONS, layers=layers,
                         schedule=[RunSpec(i) for i in range(len(layers))], final_norm=norm("final.norm"),
                         embedding_name="embed", head_name=None, embedding_scale=self.embedding_scale, streams=self.streams)
