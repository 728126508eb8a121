"""Typed configuration of the Lilatar decoder, read from config.json.

A decoder whose layers are listed one by one.  Every sublayer stands between two RMS norms (one before, one after,
x <- x + norm_b(f(norm(x)))).  A layer's mixer is "lightning" (linear attention with a fixed decay per head) or
"parallel" (softmax attention with biases, a partial interleaved rotation with scaled frequencies, soft-capped scores
and a sliding window that keeps the first tokens, beside a gated delta rule with short convolutions; the mean of the
two outputs, each RMS-normed with a weight of its own).  Its feed-forward, if any, is Wdown relu(Wup x)^2, dense or as
a mixture of experts chosen by the largest softmax scores, which weigh them as they are.  Final norm, an output matrix
of its own, logits times `logit_scale`.  Every size and every constant that the file gives is read here.

config.json keys: architecture ("Lilatar"), vocab, width, logit_scale, norm.eps and
layers[i] = {type: "lightning" | "parallel", mixer: {...}, mlp: null | {kind: "dense", ff} | {kind: "moe", expert.ff,
router.experts, router.top}} with
  lightning: heads, dim, vdim, decay[heads]
  parallel:  left  = heads, kv_heads, dim, vdim, scale, softcap, mask.size, mask.keep_first, rot.dims, rot.base,
                     rot.scaling = null | {factor, low, high, original}
             right = heads, kv_heads, dim, vdim, conv; the ranks of its two low-rank projections are the shapes of the
                     tensors a1 and g1 (a file's tensors give them; `decay_rank` and `gate_rank` name them where no
                     file is at hand, as for random weights)
Tensors: embed, head, final.norm, and for layer i under "l<i>.": norm1, norm1b, norm2, norm2b, mix.*, mlp.*.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, List, Mapping, Tuple

from .llama import ConfigError
from .spec import ExtraPart, LayerSpec, ModelSpec, PartSpec, RunSpec

MIXER_TYPES = ("lightning", "parallel")
FF_KINDS = ("dense", "moe")
UNIT_EPS = 1e-6             # of the unit norm of the delta rule's q and k: the design fixes it
# The file gives no longest sequence: positions enter through rotation angles, distances and state only.
UNBOUNDED_POSITIONS = 1 << 24


def _need(d: Dict[str, Any], key: str, where: str):
    if not isinstance(d, dict) or d.get(key) is None:
        raise ConfigError(f"missing config key: {where}{key}")
    return d[key]


class LilatarConfig:
    architecture = "Lilatar"

    def __init__(self, d: Dict[str, Any]):
        self.raw = copy.deepcopy(d)
        self.vocab = int(_need(d, "vocab", ""))
        self.width = int(_need(d, "width", ""))
        self.logit_scale = float(d.get("logit_scale", 1.0))
        self.eps = float(_need(_need(d, "norm", ""), "eps", "norm."))
        self.layers: List[Dict[str, Any]] = copy.deepcopy(list(_need(d, "layers", "")))
        for layer in self.layers:           # what a file may leave out: as many key heads as heads; one decay for all heads
            m = layer.get("mixer") if isinstance(layer, dict) else None
            if not isinstance(m, dict):
                continue
            for side in (m.get("left"), m.get("right")):
                if isinstance(side, dict) and side.get("kv_heads") is None and side.get("heads") is not None:
                    side["kv_heads"] = side["heads"]
            if isinstance(m.get("decay"), (int, float)) and m.get("heads") is not None:
                m["decay"] = [float(m["decay"])] * int(m["heads"])
        self.validate()

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LilatarConfig":
        return cls(d)

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
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
            if kind == "lightning":
                for key in ("heads", "dim", "vdim", "decay"):
                    _need(m, key, where + "mixer.")
                if len(m["decay"]) != int(m["heads"]):
                    raise ConfigError(f"{where}mixer.decay lists {len(m['decay'])} numbers for {m['heads']} heads")
            else:
                left, right = _need(m, "left", where + "mixer."), _need(m, "right", where + "mixer.")
                for key in ("heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot"):
                    _need(left, key, where + "mixer.left.")
                for key in ("heads", "kv_heads", "dim", "vdim", "conv"):
                    _need(right, key, where + "mixer.right.")
                for side, s in (("left", left), ("right", right)):
                    if int(s["heads"]) % int(s["kv_heads"]):
                        raise ConfigError(f"{where}mixer.{side}: {s['heads']} heads are no multiple of {s['kv_heads']} kv_heads")
                if int(_need(left["mask"], "size", where + "mixer.left.mask.")) <= 0:
                    raise ConfigError(f"{where}mixer.left.mask.size must be positive")
                rot = left["rot"]
                dims = int(_need(rot, "dims", where + "mixer.left.rot."))
                _need(rot, "base", where + "mixer.left.rot.")
                if dims % 2 or not 0 <= dims <= int(left["dim"]):
                    raise ConfigError(f"{where}mixer.left.rot.dims = {dims} does not fit heads of {left['dim']}")
                if rot.get("scaling") is not None:
                    for key in ("factor", "low", "high", "original"):
                        _need(rot["scaling"], key, where + "mixer.left.rot.scaling.")
                if int(right["conv"]) < 1:
                    raise ConfigError(f"{where}mixer.right.conv must be at least 1")
            mlp = layer.get("mlp")
            if mlp is not None:
                ff_kind = mlp.get("kind", "dense")
                if ff_kind not in FF_KINDS:
                    raise ConfigError(f"{where}mlp.kind: unknown feed-forward {ff_kind!r} (known: {', '.join(FF_KINDS)})")
                if ff_kind == "dense":
                    _need(mlp, "ff", where + "mlp.")
                else:
                    _need(_need(mlp, "expert", where + "mlp."), "ff", where + "mlp.expert.")
                    router = _need(mlp, "router", where + "mlp.")
                    if not 1 <= int(_need(router, "top", where + "mlp.router.")) <= int(_need(router, "experts", where + "mlp.router.")):
                        raise ConfigError(f"{where}mlp.router: top must be between 1 and experts")

    def sizes_from_tensors(self, shapes: Mapping[str, Tuple[int, ...]]) -> None:
        """Sizes that only the tensors' shapes give: the ranks of the delta rule's low-rank projections."""
        for i, layer in enumerate(self.layers):
            if layer["type"] != "parallel":
                continue
            right = layer["mixer"]["right"]
            for key, leaf in (("decay_rank", "a1"), ("gate_rank", "g1")):
                shape = shapes.get(f"l{i}.mix.right.{leaf}")
                if shape is not None and len(shape) == 2:
                    right[key] = int(shape[0])

    def to_dict(self) -> Dict[str, Any]:
        d = copy.deepcopy(self.raw)
        d["layers"] = copy.deepcopy(self.layers)
        return d

    # -- what the engine builds from -----------------------------------------------------------------------------
    def _mixer(self, i: int, kind: str, m: Dict[str, Any]) -> PartSpec:
        prefix = f"l{i}.mix"
        if kind == "lightning":
            return PartSpec("lightning", prefix, {"hidden_size": self.width, "heads": int(m["heads"]), "dim": int(m["dim"]),
                                                  "vdim": int(m["vdim"]), "decay": [float(x) for x in m["decay"]], "eps": self.eps})
        left, right = m["left"], m["right"]
        rot = left["rot"]
        scaling = rot.get("scaling")
        position = None
        if int(rot["dims"]) > 0:
            position = {"kind": "rope", "head_dim": int(left["dim"]), "rotary_dim": int(rot["dims"]), "theta": float(rot["base"]),
                        "layout": "interleaved",
                        "scaling": None if scaling is None else {
                            "rope_type": "llama3", "factor": float(scaling["factor"]), "low_freq_factor": float(scaling["low"]),
                            "high_freq_factor": float(scaling["high"]), "original_max_position_embeddings": float(scaling["original"])}}
        names = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b", "o_bias": "o.b"}
        attention = PartSpec("attention", prefix + ".left", {
            "hidden_size": self.width, "num_heads": int(left["heads"]), "num_kv_heads": int(left["kv_heads"]), "head_dim": int(left["dim"]),
            "value_dim": int(left["vdim"]), "window": int(left["mask"]["size"]), "keep_first": int(left["mask"].get("keep_first", 0)),
            "position": position, "scale": float(left["scale"]), "softcap": float(left.get("softcap") or 0.0),
            "bias": True, "o_bias": True, "names": names})
        for key in ("decay_rank", "gate_rank"):
            if right.get(key) is None:
                raise ConfigError(f"layers[{i}].mixer.right.{key}: given by the shape of the model's tensors, or by this key where there are none")
        delta = PartSpec("delta_rule", prefix + ".right", {
            "hidden_size": self.width, "heads": int(right["heads"]), "kv_heads": int(right["kv_heads"]), "dim": int(right["dim"]),
            "vdim": int(right["vdim"]), "conv": int(right["conv"]), "eps": self.eps, "unit_eps": UNIT_EPS,
            "decay_rank": int(right["decay_rank"]), "gate_rank": int(right["gate_rank"])})
        return PartSpec("parallel", prefix, {"hidden_size": self.width, "eps": self.eps,
                                             "branches": [{"mixer": attention, "out": "left.out"}, {"mixer": delta, "out": "right.out"}]})

    def _feed_forward(self, i: int, mlp: Dict[str, Any]) -> PartSpec:
        prefix = f"l{i}.mlp"
        if mlp.get("kind", "dense") == "dense":
            return PartSpec("plain_ff", prefix, {"hidden_size": self.width, "intermediate_size": int(mlp["ff"]), "activation": "relu2",
                                                 "names": {"up": "up", "down": "down"}})
        return PartSpec("routed_ff", prefix, {"hidden_size": self.width, "intermediate_size": int(mlp["expert"]["ff"]),
                                              "experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"]),
                                              "activation": "relu2", "renormalize": False,
                                              "names": {"router": "router", "expert": "e{}", "up": "up", "down": "down"}})

    def model_spec(self) -> ModelSpec:
        norm = lambda name: PartSpec("rmsnorm", name, {"size": self.width, "eps": self.eps, "tensor": ""})
        layers = []
        unused = []         # a layer without a feed-forward reads no second pair of norms, whether or not its file holds them
        for i, layer in enumerate(self.layers):
            extra = [ExtraPart("post_mixer_norm", "norm", norm(f"l{i}.norm1b"))]
            ff = ff_norm = None
            mlp = layer.get("mlp")
            if mlp is None:
                unused += [f"l{i}.norm2", f"l{i}.norm2b"]
            else:
                ff = self._feed_forward(i, mlp)
                ff_norm = norm(f"l{i}.norm2")
                extra.append(ExtraPart("post_feed_forward_norm", "norm", norm(f"l{i}.norm2b")))
            layers.append(LayerSpec("sandwich", self._mixer(i, layer["type"], layer["mixer"]), ff, norm(f"l{i}.norm1"), ff_norm, tuple(extra)))
        return ModelSpec(hidden_size=self.width, vocab_size=self.vocab, max_positions=UNBOUNDED_POSITIONS, layers=layers,
                         schedule=[RunSpec(i) for i in range(len(layers))], final_norm=norm("final.norm"),
                         embedding_name="embed", head_name="head", logit_scale=self.logit_scale, ignorable_tensors=tuple(unused))
