"""Typed configuration of the Tigutar decoder, read from config.json.

A decoder whose layers are "parallel" layers: one layer norm (weight and bias) that the mixer and the feed-forward both
read, x <- x + residual_mult * (mixer(h) + feed_forward(h)).  The order of layers is the file's; each has one of three
mixers:
  "attention"  grouped-query causal softmax attention with rotary positions on the first `rot.dims` numbers of a head
               (i paired with i + dims / 2), key and value heads of their own sizes, a sink per head in the softmax's
               denominator, a sigmoid gate per head on the output; `kv_from: j` reads layer j's keys and values;
  "delta"      the gated delta rule with one decay per head, short convolutions on q, k, v, a silu gate on the read-out;
  "parallel"   sliding-window attention (`left`, no sink, no gate) beside gated linear attention with a decay per key
               channel (`right`), each output RMS-normed over the width, and their mean;
and a feed-forward that is dense (silu-gated), a mixture of experts (sigmoid scores, the `top` largest, the score
multiplying the expert's input, clamped gated units), or absent.  Final layer norm and output matrix.

Keys: architecture, vocab, width, residual_mult, norm.eps, layers: [{"type", "mixer": {...}, "mlp": {...} or null}].
The inner size of the right mixer's decay projections is not in the file: it is the first size of
`l<i>.mix.right.a1` (`with_tensor_shapes`); a model made without a file names it itself (`decay_rank`).

Tensor names: embed, head, final.norm(.b), and per layer i under `l<i>.`: norm1(.b), mix.*, mlp.*.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..errors import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec

MAX_POSITIONS = 1 << 20        # config.json gives no limit; this bounds a sequence where nothing else does
TYPES = ("attention", "delta", "parallel")


def _int(d: Dict[str, Any], key: str, where: str, default: Any = None, zero_ok: bool = False) -> int:
    v = d.get(key, default)
    if isinstance(v, bool) or not isinstance(v, int) or v < 0 or (v == 0 and not zero_ok):
        raise ConfigError(f"{where}: {key} must be a positive integer, found {v!r}")
    return v


def _float(d: Dict[str, Any], key: str, where: str) -> float:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"{where}: {key} must be a number, found {v!r}")
    return float(v)


def _obj(d: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: '{key}' must be an object")
    return v


@dataclass
class TigutarConfig:
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    layers: List[Dict[str, Any]] = field(default_factory=list)
    max_positions: int = MAX_POSITIONS

    architecture = "Tigutar"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "TigutarConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config: 'layers' must be a list with at least one layer")
        cfg = cls(vocab=_int(d, "vocab", "config"), width=_int(d, "width", "config"),
                  norm_eps=_float(_obj(d, "norm", "config"), "eps", "norm"), residual_mult=_float(d, "residual_mult", "config"),
                  layers=copy.deepcopy(layers), max_positions=_int(d, "max_positions", "config", MAX_POSITIONS))
        cfg.check()
        return cfg

    # ------------------------------------------------------------------ checks
    @staticmethod
    def _check_softmax(m: Dict[str, Any], where: str) -> None:
        for key in ("heads", "kv_heads", "dim", "vdim"):
            _int(m, key, where)
        if m["heads"] % m["kv_heads"] != 0:
            raise ConfigError(f"{where}: {m['heads']} heads cannot share {m['kv_heads']} key/value heads")
        _float(m, "scale", where)
        rot = _obj(m, "rot", where)
        dims = _int(rot, "dims", f"{where} rot", zero_ok=True)
        _float(rot, "base", f"{where} rot")
        if dims % 2 != 0 or dims > m["dim"]:
            raise ConfigError(f"{where}: rot.dims must be even and at most dim, found {dims}")
        if m.get("mask") is not None:
            _int(_obj(m, "mask", where), "size", f"{where} mask")

    def check(self) -> None:
        for i, layer in enumerate(self.layers):
            where = f"layer {i}"
            if not isinstance(layer, dict) or layer.get("type") not in TYPES:
                raise ConfigError(f"{where}: type must be one of {', '.join(TYPES)}, found "
                                  f"{layer.get('type') if isinstance(layer, dict) else layer!r}")
            m = _obj(layer, "mixer", where)
            kind = layer["type"]
            if kind == "attention":
                self._check_softmax(m, where)
                j = m.get("kv_from")
                if j is not None:
                    if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < i:
                        raise ConfigError(f"{where}: kv_from must name an earlier layer, found {j!r}")
                    other = self.layers[j]
                    if other.get("type") != "attention" or other["mixer"].get("kv_from") is not None:
                        raise ConfigError(f"{where}: kv_from = {j}, but layer {j} keeps no keys and values of its own")
                    for key in ("kv_heads", "dim", "vdim"):
                        if other["mixer"].get(key) != m[key]:
                            raise ConfigError(f"{where}: {key} {m[key]} differs from layer {j}'s {other['mixer'].get(key)}")
                    if other["mixer"].get("rot") != m["rot"]:
                        raise ConfigError(f"{where}: its rotation differs from layer {j}'s, whose keys it reads")
            elif kind == "delta":
                for key in ("heads", "dim", "vdim", "conv"):
                    _int(m, key, where)
                if m["heads"] % _int(m, "kv_heads", where, m["heads"]) != 0:
                    raise ConfigError(f"{where}: {m['heads']} heads cannot share {m['kv_heads']} q/k heads")
            else:
                left, right = _obj(m, "left", where), _obj(m, "right", where)
                self._check_softmax(left, f"{where} left")
                for key in ("heads", "dim", "vdim"):
                    _int(right, key, f"{where} right")
                if not _float(right, "tau", f"{where} right") > 0:
                    raise ConfigError(f"{where} right: tau must be positive")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
                raise ConfigError(f"{where}: mlp must be null or of kind 'dense' or 'moe', found {mlp!r}")
            if mlp["kind"] == "dense":
                _int(mlp, "ff", where)
            else:
                expert, router = _obj(mlp, "expert", f"{where} mlp"), _obj(mlp, "router", f"{where} mlp")
                _int(expert, "ff", f"{where} expert")
                if not _float(expert, "limit", f"{where} expert") > 0:
                    raise ConfigError(f"{where} expert: limit must be positive")
                if _int(router, "top", f"{where} router") > _int(router, "experts", f"{where} router"):
                    raise ConfigError(f"{where} router: top {router['top']} of {router['experts']} experts")

    def to_dict(self) -> Dict[str, Any]:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "residual_mult": self.residual_mult,
               "norm": {"eps": self.norm_eps}, "layers": copy.deepcopy(self.layers)}
        if self.max_positions != MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out

    # ------------------------------------------------------------------ sizes only the weights know
    def with_tensor_shapes(self, shapes: Dict[str, Any]) -> "TigutarConfig":
        out = copy.deepcopy(self)
        for i, layer in enumerate(out.layers):
            name = f"l{i}.mix.right.a1"
            if layer["type"] == "parallel" and name in shapes and len(shapes[name]) == 2:
                layer["mixer"]["right"]["decay_rank"] = int(shapes[name][0])
        return out

    # ------------------------------------------------------------------ the spec
    def _softmax(self, m: Dict[str, Any], gated: bool) -> PartSpec:
        rot = m["rot"]
        if rot["dims"]:
            position = PartSpec("rope", {"head_dim": rot["dims"], "theta": rot["base"], "style": "half",
                                         "max_positions": self.max_positions})
        else:
            position = PartSpec("none", {"max_positions": self.max_positions})
        mask = m.get("mask")
        return PartSpec("attention", {
            "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"], "value_dim": m["vdim"],
            "scale": m["scale"], "window": None if mask is None else mask["size"], "cache_from": m.get("kv_from"),
            "sink": gated, "head_gate": gated, "position": position,
            "names": {"q": "q", "k": "k", "v": "v", "o": "o", "sink": "sink", "gate": "g"}})

    def to_spec(self) -> ModelSpec:
        def norm() -> PartSpec:
            return PartSpec("layernorm", {"size": self.width, "eps": self.norm_eps, "bias": True,
                                          "names": {"weight": "", "bias": "b"}})
        layers = []
        for i, layer in enumerate(self.layers):
            m, kind = layer["mixer"], layer["type"]
            if kind == "attention":
                mixer = self._softmax(m, gated=True)
            elif kind == "delta":
                mixer = PartSpec("gated_delta", {"heads": m["heads"], "kv_heads": m.get("kv_heads", m["heads"]), "dim": m["dim"],
                                                 "vdim": m["vdim"], "conv": m["conv"], "eps": self.norm_eps, "unit_eps": 1e-6})
            else:
                right = m["right"]
                if "decay_rank" not in right:
                    raise ConfigError(f"layer {i}: decay_rank is neither in the configuration nor given by a weight file")
                mixer = PartSpec("pair", {
                    "eps": self.norm_eps, "left": self._softmax(m["left"], gated=False),
                    "right": PartSpec("decay_attention", {"heads": right["heads"], "dim": right["dim"], "vdim": right["vdim"],
                                                          "tau": right["tau"], "decay_rank": right["decay_rank"],
                                                          "eps": self.norm_eps})})
            mlp = layer.get("mlp")
            if mlp is None:
                ff = None
            elif mlp["kind"] == "dense":
                ff = PartSpec("swiglu", {"intermediate_size": mlp["ff"], "names": {"gate": "gate", "up": "up", "down": "down"}})
            else:
                ff = PartSpec("routed_experts", {"experts": mlp["router"]["experts"], "top": mlp["router"]["top"],
                                                 "intermediate_size": mlp["expert"]["ff"], "limit": mlp["expert"]["limit"],
                                                 "alpha": 1.702})
            layers.append(LayerSpec(prefix=f"l{i}", block="parallel", mixer=mixer, feed_forward=ff, norm1=norm(), norm2=None,
                                    segments={"norm1": "norm1", "mixer": "mix", "feed_forward": "mlp"},
                                    params={"residual_scale": self.residual_mult}))
        return ModelSpec(
            architecture=self.architecture, hidden_size=self.width, vocab_size=self.vocab, max_positions=self.max_positions,
            layers=layers, embedding=PartSpec("table", {"name": "embed", "vocab_size": self.vocab}),
            head=PartSpec("linear", {"norm": norm(), "norm_name": "final.norm", "name": "head", "vocab_size": self.vocab}))
