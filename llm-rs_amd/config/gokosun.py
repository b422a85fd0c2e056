"""Typed configuration of the Gokosun decoder, read from config.json.

A decoder whose layers are listed one by one.  A layer has one layer norm (weight and bias) whose output both of its
halves read: x <- x + (mixer(n) + ff(n)), n = norm1(x).  A layer's mixer is "mlstm" (a matrix memory with exponential
gates: per head a matrix S and a vector n, decayed by a forget gate and written under an input gate, both gates'
logarithms bent into (-gate_cap, gate_cap) and a running maximum of them keeping the exponentials in range; each head's
read-out RMS-normed, the heads under a sigmoid gate), "latent_attention" (queries through a small RMS-normed vector of
q_rank numbers; keys and values of all heads are matrices times another RMS-normed vector of kv_rank numbers per token,
cached beside one rotated key part of rot_dim features that all heads share; rotation in neighbouring pairs with
frequencies bent between two wavelengths and an enlarged cosine and sine; a learned sink per head in the softmax's
denominator) or "attention" (grouped-query attention: q and k RMS-normed over the whole projection, the first rot.dims
features of each head rotated in the half-split layout, and, in layers that say v_mix, the values mixed with those of
the first such layer: v <- (1 - lambda) v + lambda v_first).  The feed-forward, if any, is
Wdown (g sigmoid(1.702 g) (u + 1)) with g = min(Wgate n, limit), u = clamp(Wup n, -limit, limit), dense or as a mixture
of such experts: scores sigmoid(Wrouter n), the `top` experts with the largest score + correction, weighed by their
scores over the chosen scores' sum times router.scale, beside a shared expert that every token passes.  Final layer
norm, an output matrix of its own.  Every size and every constant that the file gives is read here.

config.json keys: architecture ("Gokosun"), vocab, width, norm.eps and
layers[i] = {type: "mlstm" | "latent_attention" | "attention", mixer: {...}, mlp: null | {...}} with
  mlstm:            heads, dim, vdim, gate_cap
  latent_attention: heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rot = {dims (= rot_dim), base, scaling = null |
                    {factor, original, fast, slow}}
  attention:        heads, kv_heads (absent: heads), dim, vdim, scale, v_mix (absent: false),
                    rot = null | {dims, base, scaling = null | {...}}
  mlp:              {kind: "dense", ff, limit} | {kind: "moe", expert: {ff, limit}, router: {experts, top, scale},
                    shared: null | {ff, limit}}
Tensors: embed, head, final.norm, final.norm.b, and for layer i under "l<i>.": norm1, norm1.b, mix.*, mlp.*
(mlp.{gate, up, down}; or mlp.e<j>.{gate, up, down}, mlp.router, mlp.correction, mlp.shared.{gate, up, down}).
"""
from __future__ import annotations

import copy
from typing import Any, Dict, List, Optional

from .llama import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec, RunSpec

MIXER_TYPES = ("mlstm", "latent_attention", "attention")
FF_KINDS = ("dense", "moe")
GLU_ALPHA = 1.702       # the design's own: what the gate is multiplied by inside the sigmoid
# The file gives no longest sequence: positions enter through rotation angles only.
UNBOUNDED_POSITIONS = 1 << 24


def _need(d: Dict[str, Any], key: str, where: str):
    if not isinstance(d, dict) or d.get(key) is None:
        raise ConfigError(f"missing config key: {where}{key}")
    return d[key]


def _positive(d: Dict[str, Any], keys, where: str) -> None:
    for key in keys:
        if not float(_need(d, key, where)) > 0:
            raise ConfigError(f"{where}{key} must be positive, got {d[key]}")


class GokosunConfig:
    architecture = "Gokosun"

    def __init__(self, d: Dict[str, Any]):
        self.raw = copy.deepcopy(d)
        self.vocab = int(_need(d, "vocab", ""))
        self.width = int(_need(d, "width", ""))
        self.eps = float(_need(_need(d, "norm", ""), "eps", "norm."))
        self.layers: List[Dict[str, Any]] = copy.deepcopy(list(_need(d, "layers", "")))
        for layer in self.layers:           # what a file may leave out: as many key heads as heads
            m = layer.get("mixer") if isinstance(layer, dict) else None
            if isinstance(m, dict) and layer.get("type") == "attention" and m.get("kv_heads") is None and m.get("heads") is not None:
                m["kv_heads"] = m["heads"]
        self.validate()

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "GokosunConfig":
        return cls(d)

    def _check_rot(self, rot: Optional[Dict[str, Any]], limit: int, where: str) -> int:
        if rot is None:
            return 0
        dims = int(_need(rot, "dims", where))
        if dims % 2 or not 0 <= dims <= limit:
            raise ConfigError(f"{where}dims = {dims} does not fit {limit} features")
        if dims > 0:
            if not float(_need(rot, "base", where)) > 0:
                raise ConfigError(f"{where}base must be positive")
            if rot.get("scaling") is not None:
                _positive(rot["scaling"], ("factor", "original", "fast", "slow"), where + "scaling.")
        return dims

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {self.eps}")
        if not self.layers:
            raise ConfigError("layers is empty")
        mixed = None            # (kv_heads, vdim) of the layers whose values are mixed: they must agree
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]."
            kind = _need(layer, "type", where)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}type: unknown mixer {kind!r} (known: {', '.join(MIXER_TYPES)})")
            m = _need(layer, "mixer", where)
            mw = where + "mixer."
            for key in ("heads", "dim", "vdim"):
                if int(_need(m, key, mw)) <= 0:
                    raise ConfigError(f"{mw}{key} must be positive")
            if kind == "mlstm":
                _positive(m, ("gate_cap",), mw)
            elif kind == "latent_attention":
                for key in ("kv_rank", "q_rank", "rot_dim"):
                    if int(_need(m, key, mw)) <= 0:
                        raise ConfigError(f"{mw}{key} must be positive")
                _need(m, "scale", mw)
                dims = self._check_rot(_need(m, "rot", mw), int(m["rot_dim"]), mw + "rot.")
                if dims != int(m["rot_dim"]):
                    raise ConfigError(f"{mw}rot.dims = {dims} is not rot_dim = {m['rot_dim']}: the rotated part is rotated whole")
            else:
                _need(m, "scale", mw)
                if int(m["kv_heads"]) <= 0 or int(m["heads"]) % int(m["kv_heads"]):
                    raise ConfigError(f"{mw}: {m['heads']} heads are no multiple of {m['kv_heads']} kv_heads")
                self._check_rot(m.get("rot"), int(m["dim"]), mw + "rot.")
                if m.get("v_mix"):
                    shape = (int(m["kv_heads"]), int(m["vdim"]))
                    if mixed is not None and shape != mixed:
                        raise ConfigError(f"{mw}: values of {shape[0]} heads of {shape[1]} cannot be mixed with the first such layer's "
                                          f"{mixed[0]} heads of {mixed[1]}")
                    mixed = shape
            mlp = layer.get("mlp")
            if mlp is not None:
                lw = where + "mlp."
                ff_kind = mlp.get("kind", "dense")
                if ff_kind not in FF_KINDS:
                    raise ConfigError(f"{lw}kind: unknown feed-forward {ff_kind!r} (known: {', '.join(FF_KINDS)})")
                if ff_kind == "dense":
                    _positive(mlp, ("ff", "limit"), lw)
                else:
                    _positive(_need(mlp, "expert", lw), ("ff", "limit"), lw + "expert.")
                    r = _need(mlp, "router", lw)
                    _positive(r, ("experts", "top"), lw + "router.")
                    _need(r, "scale", lw + "router.")
                    if int(r["top"]) > int(r["experts"]):
                        raise ConfigError(f"{lw}router: top = {r['top']} of {r['experts']} experts")
                    if mlp.get("shared") is not None:
                        _positive(mlp["shared"], ("ff", "limit"), lw + "shared.")

    def to_dict(self) -> Dict[str, Any]:
        d = copy.deepcopy(self.raw)
        d["layers"] = copy.deepcopy(self.layers)
        return d

    # -- what the engine builds from -----------------------------------------------------------------------------
    @staticmethod
    def _position(rot: Optional[Dict[str, Any]], head_dim: int, layout: str) -> Optional[Dict[str, Any]]:
        if rot is None or int(rot["dims"]) <= 0:
            return None
        scaling = rot.get("scaling")
        return {"kind": "rope", "head_dim": head_dim, "rotary_dim": int(rot["dims"]), "theta": float(rot["base"]), "layout": layout,
                "scaling": None if scaling is None else {
                    "rope_type": "ramp", "factor": float(scaling["factor"]), "original": float(scaling["original"]),
                    "fast": float(scaling["fast"]), "slow": float(scaling["slow"])}}

    def _mixer(self, i: int, kind: str, m: Dict[str, Any], value_mix: Optional[str]) -> PartSpec:
        prefix = f"l{i}.mix"
        if kind == "mlstm":
            return PartSpec("mlstm", prefix, {"hidden_size": self.width, "heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
                                              "gate_cap": float(m["gate_cap"]), "eps": self.eps})
        if kind == "latent_attention":
            return PartSpec("latent_attention", prefix, {
                "hidden_size": self.width, "heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
                "kv_rank": int(m["kv_rank"]), "q_rank": int(m["q_rank"]), "rot_dim": int(m["rot_dim"]), "scale": float(m["scale"]),
                "eps": self.eps, "sink": True, "gate": None,
                "position": self._position(m["rot"], int(m["rot_dim"]), "interleaved")})
        names = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "value_mix": "vmix"}
        return PartSpec("attention", prefix, {
            "hidden_size": self.width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]), "head_dim": int(m["dim"]),
            "value_dim": int(m["vdim"]), "position": self._position(m.get("rot"), int(m["dim"]), "split_half"), "scale": float(m["scale"]),
            "qk_norm_eps": self.eps, "qk_norm_weight": True, "qk_norm_scope": "projection", "value_mix": value_mix, "names": names})

    def _feed_forward(self, i: int, mlp: Dict[str, Any]) -> PartSpec:
        prefix = f"l{i}.mlp"
        names = {"gate": "gate", "up": "up", "down": "down"}
        glu = lambda part: {"hidden_size": self.width, "intermediate_size": int(part["ff"]), "limit": float(part["limit"]),
                            "alpha": GLU_ALPHA, "names": names}
        if mlp.get("kind", "dense") == "dense":
            return PartSpec("clamped_glu", prefix, glu(mlp))
        r, expert, shared = mlp["router"], mlp["expert"], mlp.get("shared")
        return PartSpec("routed_ff", prefix, {
            "hidden_size": self.width, "intermediate_size": int(expert["ff"]), "experts": int(r["experts"]), "top": int(r["top"]),
            "activation": "clamped_glu", "limit": float(expert["limit"]), "alpha": GLU_ALPHA, "score": "sigmoid", "correction": True,
            "renormalize": True, "scale": float(r["scale"]),
            "shared": None if shared is None else {"kind": "clamped_glu", "prefix": "shared", "params": glu(shared)},
            "names": {"router": "router", "expert": "e{}", "correction": "correction", **names}})

    def model_spec(self) -> ModelSpec:
        norm = lambda name: PartSpec("layernorm", name, {"size": self.width, "eps": self.eps})
        layers = []
        unused = []             # an attention layer that mixes nothing reads no lambda, whether or not its file holds one
        mixing = False          # whether a layer before this one mixes values: the first that does gives, the others take
        for i, layer in enumerate(self.layers):
            value_mix = None
            if layer["type"] == "attention" and layer["mixer"].get("v_mix"):
                value_mix = "later" if mixing else "first"
                mixing = True
            elif layer["type"] == "attention":
                unused.append(f"l{i}.mix.vmix")
            mlp = layer.get("mlp")
            layers.append(LayerSpec("parallel", self._mixer(i, layer["type"], layer["mixer"], value_mix),
                                    None if mlp is None else self._feed_forward(i, mlp), norm(f"l{i}.norm1"), None))
        return ModelSpec(hidden_size=self.width, vocab_size=self.vocab, max_positions=UNBOUNDED_POSITIONS, layers=layers,
                         schedule=[RunSpec(i) for i in range(len(layers))], final_norm=norm("final.norm"), embedding_name="embed",
                         head_name="head", ignorable_tensors=tuple(unused))
