"""Typed configuration of the Vivisun decoder, read from config.json.

A decoder whose layers are listed one by one.  A layer's two halves read the same stream,
x <- x + mixer(norm1(x)) + ff(norm2(x)); every norm is a dynamic tanh, tanh(alpha x) w + b (no mean, no variance).
A layer's mixer is "attention" (softmax attention over every earlier key: short causal convolutions on q, k and v, an
RMS norm of q and k per head with a weight, a rotation of the first `rot.dims` features of each head in the half-split
layout whose frequencies are bent between two wavelengths and whose cosine and sine are enlarged, a sigmoid gate on the
heads' outputs) or "latent_attention" (keys and values of all heads are matrices times one small RMS-normed vector per
token, the only thing cached; no positions; a learned sink per head in the softmax's denominator; a sigmoid gate per
head).  The feed-forward, if any, is Wdown (silu(Wgate x) * Wup x).  A stretch of layers (`loop`) runs several times in a
row with the same weights, each pass with a cache of its own, the token embeddings added to the stream again before
every pass but the first.  Final norm, an output matrix of its own.  Every size and every constant that the file gives
is read here.

config.json keys: architecture ("Vivisun"), vocab, width, norm.eps, loop = null | {start, stop, times} and
layers[i] = {type: "attention" | "latent_attention", mixer: {...}, mlp: null | {kind: "dense", ff}} with
  attention:        heads, kv_heads (absent: heads), dim, vdim, scale, conv (taps; absent or 0: none),
                    rot = null | {dims, base, scaling = null | {factor, original, fast, slow}}
  latent_attention: heads, dim, vdim, kv_rank, scale
Tensors: embed, head, final.norm(.b, .alpha), and for layer i under "l<i>.": norm1, norm2 (each with .b and .alpha),
mix.*, mlp.{gate, up, down}.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, List

from .llama import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec, RunSpec

MIXER_TYPES = ("attention", "latent_attention")
FF_KINDS = ("dense",)
# The file gives no longest sequence: positions enter through rotation angles only.
UNBOUNDED_POSITIONS = 1 << 24


def _need(d: Dict[str, Any], key: str, where: str):
    if not isinstance(d, dict) or d.get(key) is None:
        raise ConfigError(f"missing config key: {where}{key}")
    return d[key]


class VivisunConfig:
    architecture = "Vivisun"

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
        loop = d.get("loop")
        self.loop = None if loop is None else {k: int(_need(loop, k, "loop.")) for k in ("start", "stop", "times")}
        self.validate()

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "VivisunConfig":
        return cls(d)

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {self.eps}")
        if not self.layers:
            raise ConfigError("layers is empty")
        if self.loop is not None:
            a, b, n = self.loop["start"], self.loop["stop"], self.loop["times"]
            if not (0 <= a <= b <= len(self.layers)) or n < 1:
                raise ConfigError(f"loop: layers {a} to {b} (of {len(self.layers)}) cannot run {n} times")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]."
            kind = _need(layer, "type", where)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}type: unknown mixer {kind!r} (known: {', '.join(MIXER_TYPES)})")
            m = _need(layer, "mixer", where)
            for key in ("heads", "dim", "vdim", "scale"):
                _need(m, key, where + "mixer.")
            if min(int(m["heads"]), int(m["dim"]), int(m["vdim"])) <= 0:
                raise ConfigError(f"{where}mixer: heads, dim and vdim must be positive")
            if kind == "attention":
                if int(m["kv_heads"]) <= 0 or int(m["heads"]) % int(m["kv_heads"]):
                    raise ConfigError(f"{where}mixer: {m['heads']} heads are no multiple of {m['kv_heads']} kv_heads")
                if int(m.get("conv") or 0) < 0:
                    raise ConfigError(f"{where}mixer.conv must not be negative")
                rot = m.get("rot")
                if rot is not None:
                    dims = int(_need(rot, "dims", where + "mixer.rot."))
                    if dims % 2 or not 0 <= dims <= int(m["dim"]):
                        raise ConfigError(f"{where}mixer.rot.dims = {dims} does not fit heads of {m['dim']}")
                    if dims > 0:
                        _need(rot, "base", where + "mixer.rot.")
                    if rot.get("scaling") is not None:
                        for key in ("factor", "original", "fast", "slow"):
                            _need(rot["scaling"], key, where + "mixer.rot.scaling.")
            else:
                if int(_need(m, "kv_rank", where + "mixer.")) <= 0:
                    raise ConfigError(f"{where}mixer.kv_rank must be positive")
            mlp = layer.get("mlp")
            if mlp is not None:
                ff_kind = mlp.get("kind", "dense")
                if ff_kind not in FF_KINDS:
                    raise ConfigError(f"{where}mlp.kind: unknown feed-forward {ff_kind!r} (known: {', '.join(FF_KINDS)})")
                if int(_need(mlp, "ff", where + "mlp.")) <= 0:
                    raise ConfigError(f"{where}mlp.ff must be positive")

    def to_dict(self) -> Dict[str, Any]:
        d = copy.deepcopy(self.raw)
        d["layers"] = copy.deepcopy(self.layers)
        return d

    # -- what the engine builds from -----------------------------------------------------------------------------
    def _mixer(self, i: int, kind: str, m: Dict[str, Any]) -> PartSpec:
        prefix = f"l{i}.mix"
        if kind == "latent_attention":
            return PartSpec("latent_attention", prefix, {
                "hidden_size": self.width, "heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
                "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"]), "eps": self.eps, "sink": True, "gate": "head"})
        rot = m.get("rot")
        position = None
        if rot is not None and int(rot["dims"]) > 0:
            scaling = rot.get("scaling")
            position = {"kind": "rope", "head_dim": int(m["dim"]), "rotary_dim": int(rot["dims"]), "theta": float(rot["base"]),
                        "layout": "split_half",
                        "scaling": None if scaling is None else {
                            "rope_type": "ramp", "factor": float(scaling["factor"]), "original": float(scaling["original"]),
                            "fast": float(scaling["fast"]), "slow": float(scaling["slow"])}}
        names = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "q_conv": "q.conv",
                 "k_conv": "k.conv", "v_conv": "v.conv", "gate": "g"}
        return PartSpec("attention", prefix, {
            "hidden_size": self.width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]), "head_dim": int(m["dim"]),
            "value_dim": int(m["vdim"]), "position": position, "scale": float(m["scale"]), "conv": int(m.get("conv") or 0),
            "qk_norm_eps": self.eps, "qk_norm_weight": True, "gate": "feature", "names": names})

    def _feed_forward(self, i: int, mlp: Dict[str, Any]) -> PartSpec:
        return PartSpec("swiglu", f"l{i}.mlp", {"hidden_size": self.width, "intermediate_size": int(mlp["ff"]),
                                                "names": {"gate": "gate", "up": "up", "down": "down"}})

    def schedule(self) -> List[RunSpec]:
        n = len(self.layers)
        loop = self.loop
        if loop is None or loop["times"] <= 1 or loop["stop"] <= loop["start"]:
            return [RunSpec(i) for i in range(n)]
        a, b = loop["start"], loop["stop"]
        runs = [RunSpec(i) for i in range(a)]
        for p in range(loop["times"]):          # each pass owns its caches; every pass but the first sees the embeddings again
            runs += [RunSpec(i, add_embedding=(p > 0 and i == a)) for i in range(a, b)]
        return runs + [RunSpec(i) for i in range(b, n)]

    def model_spec(self) -> ModelSpec:
        norm = lambda name: PartSpec("dyt", name, {"size": self.width})
        layers = []
        unused = []         # a layer without a feed-forward reads no second norm, whether or not its file holds one
        for i, layer in enumerate(self.layers):
            ff = ff_norm = None
            mlp = layer.get("mlp")
            if mlp is None:
                unused += [f"l{i}.norm2", f"l{i}.norm2.b", f"l{i}.norm2.alpha"]
            else:
                ff = self._feed_forward(i, mlp)
                ff_norm = norm(f"l{i}.norm2")
            layers.append(LayerSpec("parallel", self._mixer(i, layer["type"], layer["mixer"]), ff, norm(f"l{i}.norm1"), ff_norm))
        return ModelSpec(hidden_size=self.width, vocab_size=self.vocab, max_positions=UNBOUNDED_POSITIONS, layers=layers,
                         schedule=self.schedule(), final_norm=norm("final.norm"), embedding_name="embed", head_name="head",
                         ignorable_tensors=tuple(unused))
