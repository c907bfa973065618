"""A pre-norm layer whose residual stream is kept in several copies (hyper-connections), with a scale per channel
on every sublayer's result and, optionally, a short causal convolution in front of the mixer.

The stream is x [S, T, E] float32, all copies equal to the embedding at the start.  For sublayer p (1: the mixer,
2: the feed-forward, if the layer has one), with the layer's own tensors hc<p>.in [S], hc<p>.out [S], hc<p>.mix [S, S]
(from, to) and ls<p> [E]:
    u = sum_s in[s] x_s;   h = norm<p>(u);   (p = 1, with a convolution: h <- h + conv(h), causal, per channel)
    y = ls<p> * sublayer(h);   x_j <- sum_s mix[s, j] x_s + out[j] * y   for all j at once
The update of the copies is left to the norm that reads the stream next (`StreamsUpdate`: the layer's own second
norm, the next layer's first, the head's), which does it in its own pass over the rows.
What reads the stream after the last layer takes the sum of the copies (the head's norm does).  One copy with
in = out = mix = 1 is the plain pre-norm layer.  Norms, mixtures and sums in float32.

The convolution's last taps - 1 inputs are part of a sequence's state (`view.states["input_conv"]`), beside
whatever the mixer keeps.

Block parameters (`LayerSpec.params`): streams, input_conv (None, or {"taps": n, "name": tensor}), names (the
tensors above, with "{p}" for the sublayer's number).
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..errors import ConfigError
from .base import BuildEnv, CacheRequest, Part, TensorSpec, build_part, register_block
from .short_conv import ACT_NONE, ShortConv
from .stream import StreamsUpdate

DEFAULT_SEGMENTS = {"norm1": "norm1", "mixer": "mix", "norm2": "norm2", "feed_forward": "mlp"}
DEFAULT_NAMES = {"in": "hc{p}.in", "out": "hc{p}.out", "mix": "hc{p}.mix", "scale": "ls{p}"}
MAX_STREAMS = 16


class _OwnTensors(Part):
    """The layer's own tensors (mixtures, scales, the convolution), loaded under the layer's prefix."""

    def __init__(self, block: "HyperBlock"):
        self.block = block

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        b, s = self.block, self.block.streams
        out = {}
        for p in b.sublayers:
            out[b.name("in", p)] = TensorSpec((s,), role="gain", init="ones_normal")
            out[b.name("out", p)] = TensorSpec((s,), role="gain", init="ones_normal")
            out[b.name("mix", p)] = TensorSpec((s, s), role="gain", init="eye_normal")
            out[b.name("scale", p)] = TensorSpec((b.hidden,), role="gain", init="ones_normal")
        if b.conv is not None:
            out[b.conv_name] = b.conv.tensor_spec()
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        b = self.block
        b.coef = {p: {k: tensors[b.name(k, p)].contiguous() for k in ("in", "out", "mix", "scale")} for p in b.sublayers}
        if b.conv is not None:
            b.conv.load(tensors[b.conv_name])


class HyperBlock:
    def __init__(self, layer_spec, env: BuildEnv):
        params = dict(getattr(layer_spec, "params", None) or {})
        self.env = env
        self.hidden = env.hidden_size
        self.streams = int(params.get("streams", 1))
        if not 1 <= self.streams <= MAX_STREAMS:
            raise ConfigError(f"a stream in {self.streams} copies is not supported (1 to {MAX_STREAMS})")
        self.names = dict(DEFAULT_NAMES, **(params.get("names") or {}))
        self.segments = dict(DEFAULT_SEGMENTS, **(getattr(layer_spec, "segments", None) or {}))
        self.norm1 = build_part("norm", layer_spec.norm1, env)
        self.mixer = build_part("mixer", layer_spec.mixer, env)
        self.feed_forward = self.norm2 = None
        if layer_spec.feed_forward is not None:
            self.norm2 = build_part("norm", layer_spec.norm2, env)
            self.feed_forward = build_part("feed_forward", layer_spec.feed_forward, env)
        self.sublayers = (1, 2) if self.feed_forward is not None else (1,)
        conv = params.get("input_conv")
        self.conv = ShortConv(self.hidden, int(conv["taps"]), env, residual=True, act=ACT_NONE) if conv else None
        self.conv_name = str(conv.get("name", "input_conv")) if conv else None
        self.own = _OwnTensors(self)
        self.coef: Dict[int, Dict[str, torch.Tensor]] = {}
        for norm in (self.norm1, self.norm2):
            if norm is not None and not hasattr(norm, "forward"):
                raise ConfigError("a layer's norm needs a forward")

    def name(self, what: str, p: int) -> str:
        return self.names[what].format(p=p)

    def _all(self):
        return [x for x in (self.norm1, self.mixer, self.norm2, self.feed_forward) if x is not None]

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in self._all())

    @property
    def plan_safe(self) -> bool:
        return all(getattr(p, "plan_safe", False) for p in self._all())

    def parts(self) -> Dict[str, object]:
        out = {self.segments["norm1"]: self.norm1, self.segments["mixer"]: self.mixer, "": self.own}
        if self.feed_forward is not None:
            out[self.segments["norm2"]] = self.norm2
            out[self.segments["feed_forward"]] = self.feed_forward
        return out

    def cache_requests(self) -> List[CacheRequest]:
        many = getattr(self.mixer, "cache_requests", None)
        one = getattr(self.mixer, "cache_request", None)
        out = list(many()) if many else ([one()] if one and one() is not None else [])
        if self.conv is not None:
            req = self.conv.cache_request("input_conv")
            if req is not None:
                out.append(req)
        return out

    def _norm(self, norm, x: torch.Tensor, pending, coef: torch.Tensor, out_dtype) -> torch.Tensor:
        """norm(sum_s coef[s] x_s), after the update that the sublayer before left to be done (in the same pass)."""
        if x.dim() == 3 and hasattr(norm, "names"):           # a norm that reads the mixture of the copies itself
            return norm.forward(x, pending, None, coef=coef, out_dtype=out_dtype)
        raise ConfigError("this arrangement needs a norm that reads a stream in several copies (layernorm)")

    def forward(self, x: torch.Tensor, pending, ctx, view, next_norm=None):
        if x.dim() != 3 or x.shape[0] != self.streams:
            raise ConfigError(f"the stream must come in {self.streams} copies [S, T, E] (the embedding's `streams`)")
        if pending is not None and not isinstance(pending, StreamsUpdate):
            raise ConfigError("a layer with the stream in several copies cannot follow one that leaves a plain term to be added")
        lib, dt = self.env.lib, self.env.dtype
        c = self.coef[1]
        if self.conv is not None:
            hn = self._norm(self.norm1, x, pending, c["in"], torch.float32)
            h = self.conv.forward(hn, ctx, view.states.get("input_conv"), dt)
        else:
            h = self._norm(self.norm1, x, pending, c["in"], dt)
        y = self.mixer.forward(h, ctx, view)
        pending = StreamsUpdate(lib, c["mix"], c["out"], y, c["scale"])
        if self.feed_forward is not None:
            c = self.coef[2]
            h = self._norm(self.norm2, x, pending, c["in"], dt)
            y = self.feed_forward.forward(h, ctx)
            pending = StreamsUpdate(lib, c["mix"], c["out"], y, c["scale"])
        return pending                                        # done by whichever norm reads the stream next


register_block("hyper", HyperBlock)
