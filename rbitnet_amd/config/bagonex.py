"""Typed configuration of the Bagonex decoder, read from config.json.

A decoder without positions whose layers alternate, in an order the file gives, between two mixers: a gated delta
rule with a decay per key channel ("channel_delta", a recurrent state per head) and causal attention through a
cached latent with a sink in the softmax ("latent_attention"; a layer may read the latents of an earlier one,
`kv_from`).  Every layer: layer norm with weight and bias, a short causal convolution in front of the mixer, a scale per
channel on each sublayer's result, the residual stream in `streams` copies (hyper-connections); dense feed-forward
with the xIELU activation, or none.  Final layer norm, output matrix, logits capped by a tanh.

Keys: architecture, vocab, width, streams, norm.eps, canon.taps, logit_softcap, and `layers`: a list of
{"type", "mixer": {sizes}, "mlp": {"kind": "dense", "ff": n} or null}.  Sizes that the file does not give (the ranks of
the delta rule's two low-rank projections) are read off the weight file's shapes (`with_tensor_shapes`); a model
made without a file names them itself (`decay_rank`, `gate_rank` in the mixer's sizes).

Tensor names: embed, head, final.norm(.b), and per layer i under `l<i>.`: norm1(.b), norm2(.b), ls1, ls2,
hc1.{in,out,mix}, hc2.{in,out,mix}, canon1, mix.* and mlp.*.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..errors import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec

MAX_POSITIONS = 1 << 20        # the design has no positions; this bounds a sequence where nothing else does
MIXERS = ("channel_delta", "latent_attention")


def _int(d: Dict[str, Any], key: str, where: str, default: Any = None) -> int:
    v = d.get(key, default)
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"{where}: {key} must be a positive integer, found {v!r}")
    return v


def _float(d: Dict[str, Any], key: str, where: str) -> float:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"{where}: {key} must be a number, found {v!r}")
    return float(v)


@dataclass
class BagonexConfig:
    vocab: int
    width: int
    streams: int
    norm_eps: float
    canon_taps: int
    logit_softcap: Optional[float]
    layers: List[Dict[str, Any]] = field(default_factory=list)
    max_positions: int = MAX_POSITIONS

    architecture = "Bagonex"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "BagonexConfig":
        norm, canon = d.get("norm"), d.get("canon")
        if not isinstance(norm, dict) or not isinstance(canon, dict):
            raise ConfigError("config: 'norm' and 'canon' must be objects")
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config: 'layers' must be a list with at least one layer")
        cap = d.get("logit_softcap")
        cfg = cls(vocab=_int(d, "vocab", "config"), width=_int(d, "width", "config"),
                  streams=_int(d, "streams", "config", 1), norm_eps=_float(norm, "eps", "norm"),
                  canon_taps=_int(canon, "taps", "canon"), logit_softcap=None if cap is None else _float(d, "logit_softcap", "config"),
                  layers=copy.deepcopy(layers), max_positions=_int(d, "max_positions", "config", MAX_POSITIONS))
        cfg.check()
        return cfg

    def check(self) -> None:
        for i, layer in enumerate(self.layers):
            where = f"layer {i}"
            if not isinstance(layer, dict) or layer.get("type") not in MIXERS:
                raise ConfigError(f"{where}: type must be one of {', '.join(MIXERS)}, found {layer.get('type') if isinstance(layer, dict) else layer!r}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"{where}: 'mixer' must be an object")
            for key in ("heads", "dim", "vdim"):
                _int(m, key, where)
            if layer["type"] == "channel_delta":
                _int(m, "conv", where)
                kv = _int(m, "kv_heads", where, m["heads"])
                if m["heads"] % kv != 0:
                    raise ConfigError(f"{where}: {m['heads']} heads cannot share {kv} q/k heads")
            else:
                _int(m, "q_rank", where)
                _int(m, "kv_rank", where)
                _float(m, "scale", where)
                j = m.get("kv_from")
                if j is not None:
                    if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < i:
                        raise ConfigError(f"{where}: kv_from must name an earlier layer, found {j!r}")
                    other = self.layers[j]
                    if other.get("type") != "latent_attention" or other["mixer"].get("kv_from") is not None:
                        raise ConfigError(f"{where}: kv_from = {j}, but layer {j} stores no latents of its own")
                    if other["mixer"].get("kv_rank") != m["kv_rank"]:
                        raise ConfigError(f"{where}: kv_rank {m['kv_rank']} differs from layer {j}'s {other['mixer'].get('kv_rank')}")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError(f"{where}: mlp must be null or of kind 'dense', found {mlp!r}")
                _int(mlp, "ff", where)

    def to_dict(self) -> Dict[str, Any]:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "streams": self.streams,
               "norm": {"eps": self.norm_eps}, "canon": {"taps": self.canon_taps}, "logit_softcap": self.logit_softcap,
               "layers": copy.deepcopy(self.layers)}
        if self.max_positions != MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out

    # ------------------------------------------------------------------ sizes only the weights know
    def with_tensor_shapes(self, shapes: Dict[str, Any]) -> "BagonexConfig":
        """The ranks of the delta rule's low-rank projections are not in config.json: they are the first sizes of
        `l<i>.mix.a1` and `l<i>.mix.g1`."""
        out = copy.deepcopy(self)
        for i, layer in enumerate(out.layers):
            if layer["type"] != "channel_delta":
                continue
            for key, name in (("decay_rank", f"l{i}.mix.a1"), ("gate_rank", f"l{i}.mix.g1")):
                if name in shapes and len(shapes[name]) == 2:
                    layer["mixer"][key] = int(shapes[name][0])
        return out

    # ------------------------------------------------------------------ the spec
    def to_spec(self) -> ModelSpec:
        def norm(bias_name: str = "b") -> PartSpec:
            return PartSpec("layernorm", {"size": self.width, "eps": self.norm_eps, "bias": True,
                                          "names": {"weight": "", "bias": bias_name}})
        layers = []
        for i, layer in enumerate(self.layers):
            m = layer["mixer"]
            if layer["type"] == "channel_delta":
                for key in ("decay_rank", "gate_rank"):
                    if key not in m:
                        raise ConfigError(f"layer {i}: {key} is neither in the configuration nor given by a weight file")
                mixer = PartSpec("channel_delta", {
                    "heads": m["heads"], "kv_heads": m.get("kv_heads", m["heads"]), "dim": m["dim"], "vdim": m["vdim"],
                    "conv": m["conv"], "eps": self.norm_eps, "unit_eps": 1e-6, "decay_rank": m["decay_rank"],
                    "gate_rank": m["gate_rank"]})
            else:
                mixer = PartSpec("latent_attention", {
                    "heads": m["heads"], "dim": m["dim"], "vdim": m["vdim"], "q_rank": m["q_rank"], "kv_rank": m["kv_rank"],
                    "scale": m["scale"], "eps": self.norm_eps, "cache_from": m.get("kv_from")})
            mlp = layer.get("mlp")
            ff = None if mlp is None else PartSpec("dense_xielu", {"intermediate_size": mlp["ff"]})
            layers.append(LayerSpec(prefix=f"l{i}", block="hyper", mixer=mixer, feed_forward=ff, norm1=norm(),
                                    norm2=None if ff is None else norm(),
                                    segments={"norm1": "norm1", "mixer": "mix", "norm2": "norm2", "feed_forward": "mlp"},
                                    params={"streams": self.streams, "input_conv": {"taps": self.canon_taps, "name": "canon1"}}))
        return ModelSpec(
            architecture=self.architecture, hidden_size=self.width, vocab_size=self.vocab, max_positions=self.max_positions,
            layers=layers,
            embedding=PartSpec("table", {"name": "embed", "vocab_size": self.vocab, "streams": self.streams}),
            head=PartSpec("linear", {"norm": norm(), "norm_name": "final.norm", "name": "head", "vocab_size": self.vocab,
                                     "softcap": self.logit_softcap}))
