"""A plain, slow float64 implementation of the Tigutar decoder, one function per mechanism, whole sequences only
(no cache, no state, no batches): the oracle of the tests.  It shares no code with the package.

Notation: T tokens, E width; weights are [out, in] and applied as x @ W.T.  A layer is
    h = layer_norm(x);  x <- x + m * (mixer(h) + feed_forward(h))
with one norm that both sublayers read.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch

F64 = torch.float64


# ---------------------------------------------------------------- small things
def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def causal_conv(x, w):
    """x [T, C], w [C, taps], the last column is the current token's; zeros before the start."""
    t_len, c = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, c, dtype=x.dtype), x])
    out = torch.zeros_like(x)
    for j in range(taps):
        out = out + padded[j:j + t_len] * w[:, j]
    return out


def rotate(x, base: float, dims: int, first_pos: int = 0):
    """x [T, H, D]: the first `dims` numbers of every head are rotated, i paired with i + dims/2; the rest pass."""
    t_len = x.shape[0]
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = (torch.arange(t_len, dtype=F64) + first_pos)[:, None] * f[None, :]
    cos, sin = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# ---------------------------------------------------------------- softmax attention
def attention_weights(q, k, scale: float, window: Optional[int], sink: Optional[torch.Tensor]):
    """q [T, H, D], k [T, G, D] -> weights [H, T, T]; a sink adds exp(sink_h) to the denominator only."""
    t_len, h, _ = q.shape
    g = k.shape[1]
    kk = k.repeat_interleave(h // g, 1)
    s = torch.einsum("ihd,jhd->hij", q, kk) * scale
    i = torch.arange(t_len)[:, None]
    j = torch.arange(t_len)[None, :]
    seen = j <= i
    if window is not None:
        seen = seen & (i - j < window)
    s = s.masked_fill(~seen, -math.inf)
    top = s.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink.view(h, 1, 1))
    e = torch.exp(s - top)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink.view(h, 1, 1) - top)
    return e / den


def softmax_attention(h, w: Dict[str, torch.Tensor], p: Dict, kv=None):
    """The attention mixer.  p: heads, kv_heads, dim, vdim, rot {base, dims}, scale, optional mask {size}.  Tensors
    q, k, v, o and optionally sink [heads], g [heads, E].  kv: (k after rotation, v) of another layer to use instead
    of own projections.  Returns (out [T, E], (k, v))."""
    t_len = h.shape[0]
    heads, groups, dim, vdim = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    rot = p["rot"]
    q = rotate((h @ w["q"].T).view(t_len, heads, dim), rot["base"], rot["dims"])
    if kv is None:
        k = rotate((h @ w["k"].T).view(t_len, groups, dim), rot["base"], rot["dims"])
        v = (h @ w["v"].T).view(t_len, groups, vdim)
    else:
        k, v = kv
    window = (p.get("mask") or {}).get("size")
    a = attention_weights(q, k, p["scale"], window, w.get("sink"))
    o = torch.einsum("hij,jhd->ihd", a, v.repeat_interleave(heads // groups, 1))
    if "g" in w:
        o = o * torch.sigmoid(h @ w["g"].T)[:, :, None]
    return o.reshape(t_len, heads * vdim) @ w["o"].T, (k, v)


# ---------------------------------------------------------------- recurrences
def delta_recurrence(q, k, v, g, beta):
    """q, k [T, H, dk], v [T, H, dv], g [T, H] (one decay per head), beta [T, H] -> o [T, H, dv]:
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    t_len, h, dk = q.shape
    dv = v.shape[-1]
    s = torch.zeros(h, dk, dv, dtype=q.dtype)
    o = torch.zeros(t_len, h, dv, dtype=q.dtype)
    for t in range(t_len):
        s = g[t][:, None, None] * s
        u = beta[t][:, None] * (v[t] - torch.einsum("hkv,hk->hv", s, k[t]))
        s = s + torch.einsum("hk,hv->hkv", k[t], u)
        o[t] = torch.einsum("hkv,hk->hv", s, q[t])
    return o


def decay_recurrence(q, k, v, alpha):
    """q, k, alpha [T, H, dk], v [T, H, dv] -> o [T, H, dv]:  S <- diag(alpha) S + k v^T;  o = S^T q."""
    t_len, h, dk = q.shape
    dv = v.shape[-1]
    s = torch.zeros(h, dk, dv, dtype=q.dtype)
    o = torch.zeros(t_len, h, dv, dtype=q.dtype)
    for t in range(t_len):
        s = alpha[t][:, :, None] * s + torch.einsum("hk,hv->hkv", k[t], v[t])
        o[t] = torch.einsum("hkv,hk->hv", s, q[t])
    return o


def delta_mixer(h, w: Dict[str, torch.Tensor], p: Dict, eps: float):
    """p: heads, kv_heads, dim, vdim, conv.  Tensors q, k, v (+ .conv), b, a, A_log, dt_bias, norm, g, o."""
    t_len = h.shape[0]
    heads, groups, dim, vdim = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    q = silu(causal_conv(h @ w["q"].T, w["q.conv"])).view(t_len, groups, dim)
    k = silu(causal_conv(h @ w["k"].T, w["k.conv"])).view(t_len, groups, dim)
    v = silu(causal_conv(h @ w["v"].T, w["v.conv"])).view(t_len, heads, vdim)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q = q.repeat_interleave(heads // groups, 1)
    k = k.repeat_interleave(heads // groups, 1)
    beta = torch.sigmoid(h @ w["b"].T)
    g = torch.exp(-torch.exp(w["A_log"]) * softplus(h @ w["a"].T + w["dt_bias"]))
    o = delta_recurrence(q, k, v, g, beta)
    o = rms_norm(o, w["norm"], eps) * silu(h @ w["g"].T).view(t_len, heads, vdim)
    return o.reshape(t_len, heads * vdim) @ w["o"].T


def decay_mixer(h, w: Dict[str, torch.Tensor], p: Dict, eps: float):
    """Gated linear attention.  p: heads, dim, vdim, tau.  Tensors q, k, v, g, o, norm, a1, a2, a2.b."""
    t_len = h.shape[0]
    heads, dim, vdim = p["heads"], p["dim"], p["vdim"]
    q = (h @ w["q"].T).view(t_len, heads, dim) * dim ** -0.5
    k = (h @ w["k"].T).view(t_len, heads, dim)
    v = (h @ w["v"].T).view(t_len, heads, vdim)
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / p["tau"]).view(t_len, heads, dim)
    o = rms_norm(decay_recurrence(q, k, v, alpha), w["norm"], eps)
    return (o.reshape(t_len, heads * vdim) * silu(h @ w["g"].T)) @ w["o"].T


def side_by_side(h, w: Dict[str, torch.Tensor], p: Dict, eps: float):
    """The 'parallel' mixer: windowed attention (left.*) and gated linear attention (right.*) on the same input, each
    RMS-normed over the width with its own weight, and the mean of the two."""
    left = {n[5:]: t for n, t in w.items() if n.startswith("left.") and n != "left.out"}
    right = {n[6:]: t for n, t in w.items() if n.startswith("right.") and n != "right.out"}
    a, _ = softmax_attention(h, left, p["left"])
    b = decay_mixer(h, right, p["right"], eps)
    return 0.5 * (rms_norm(a, w["left.out"], eps) + rms_norm(b, w["right.out"], eps))


# ---------------------------------------------------------------- feed-forward
def dense_ff(h, w: Dict[str, torch.Tensor]):
    return (silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def expert(x, gate, up, down, limit: float):
    g = torch.clamp(x @ gate.T, max=limit)
    u = torch.clamp(x @ up.T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ down.T


def routed_ff(h, w: Dict[str, torch.Tensor], n_experts: int, top: int, limit: float):
    """Scores sigmoid(router h); the `top` largest are chosen and weigh each expert's INPUT, not renormalised."""
    s = torch.sigmoid(h @ w["router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(n_experts), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in order:
            out[t] = out[t] + expert(s[t, e] * h[t], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], limit)
    return out


# ---------------------------------------------------------------- the model
class PlainTigutar:
    def __init__(self, config: Dict, tensors: Dict[str, torch.Tensor]):
        self.cfg = config
        self.w = {n: t.to(F64) for n, t in tensors.items()}

    @classmethod
    def from_folder(cls, folder: str) -> "PlainTigutar":
        from safetensors import safe_open
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        tensors = {}
        with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
            for name in f.keys():
                tensors[name] = f.get_tensor(name)
        return cls(cfg, tensors)

    def _sub(self, prefix: str) -> Dict[str, torch.Tensor]:
        return {n[len(prefix):]: t for n, t in self.w.items() if n.startswith(prefix)}

    def logits(self, tokens: List[int], layers_out: Optional[list] = None) -> torch.Tensor:
        cfg, eps, m = self.cfg, self.cfg["norm"]["eps"], self.cfg["residual_mult"]
        x = self.w["embed"][torch.tensor(tokens)]
        kept = {}
        for i, layer in enumerate(cfg["layers"]):
            h = layer_norm(x, self.w[f"l{i}.norm1"], self.w[f"l{i}.norm1.b"], eps)
            mw, p = self._sub(f"l{i}.mix."), layer["mixer"]
            if layer["type"] == "attention":
                src = p.get("kv_from")
                y, kept[i] = softmax_attention(h, mw, p, None if src is None else kept[src])
            elif layer["type"] == "delta":
                y = delta_mixer(h, mw, p, eps)
            elif layer["type"] == "parallel":
                y = side_by_side(h, mw, p, eps)
            else:
                raise ValueError(layer["type"])
            mlp = layer.get("mlp")
            if mlp is not None:
                fw = self._sub(f"l{i}.mlp.")
                if mlp["kind"] == "dense":
                    y = y + dense_ff(h, fw)
                else:
                    y = y + routed_ff(h, fw, mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["limit"])
            x = x + m * y
            if layers_out is not None:
                layers_out.append(x.clone())
        x = layer_norm(x, self.w["final.norm"], self.w["final.norm.b"], eps)
        return x @ self.w["head"].T


# ---------------------------------------------------------------- random weights for a configuration
def random_tigutar_tensors(cfg: Dict, seed: int, decay_rank: int = 8) -> Dict[str, torch.Tensor]:
    """Every tensor of a model of this configuration, float64 values that bfloat16 holds exactly.  Projections are
    scaled so that scores, gates, decays and routers move with the input (a wrong mask, state or sink shows)."""
    g = torch.Generator().manual_seed(seed)
    e = cfg["width"]

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g, dtype=F64) * std + mean).to(torch.bfloat16).to(F64)

    def lin(n, k, gain=1.0):
        return rnd(n, k, std=gain * k ** -0.5)

    def softmax_tensors(p, prefix, gated):
        out = {f"{prefix}q": lin(p["heads"] * p["dim"], e, 2.0), f"{prefix}o": lin(e, p["heads"] * p["vdim"])}
        if p.get("kv_from") is None:
            out[f"{prefix}k"] = lin(p["kv_heads"] * p["dim"], e, 2.0)
            out[f"{prefix}v"] = lin(p["kv_heads"] * p["vdim"], e)
        if gated:
            out[f"{prefix}sink"] = rnd(p["heads"], std=1.5)
            out[f"{prefix}g"] = lin(p["heads"], e, 2.0)
        return out

    t = {"embed": rnd(cfg["vocab"], e), "head": lin(cfg["vocab"], e), "final.norm": rnd(e, std=0.1, mean=1.0),
         "final.norm.b": rnd(e, std=0.1)}
    for i, layer in enumerate(cfg["layers"]):
        pre, p = f"l{i}.", layer["mixer"]
        t[pre + "norm1"], t[pre + "norm1.b"] = rnd(e, std=0.1, mean=1.0), rnd(e, std=0.1)
        mx = pre + "mix."
        if layer["type"] == "attention":
            t.update(softmax_tensors(p, mx, True))
        elif layer["type"] == "delta":
            nqk, nv = p["kv_heads"] * p["dim"], p["heads"] * p["vdim"]
            for name, n in (("q", nqk), ("k", nqk), ("v", nv)):
                t[mx + name] = lin(n, e, 2.0)
                t[mx + name + ".conv"] = rnd(n, p["conv"], std=0.6)
            t[mx + "b"], t[mx + "a"] = lin(p["heads"], e, 2.0), lin(p["heads"], e, 2.0)
            t[mx + "A_log"], t[mx + "dt_bias"] = rnd(p["heads"], std=0.5, mean=-1.0), rnd(p["heads"], std=0.5)
            t[mx + "norm"] = rnd(p["vdim"], std=0.1, mean=1.0)
            t[mx + "g"], t[mx + "o"] = lin(nv, e, 2.0), lin(e, nv)
        else:
            t.update(softmax_tensors(p["left"], mx + "left.", False))
            r = p["right"]
            rank = r.get("decay_rank", decay_rank)
            nqk, nv = r["heads"] * r["dim"], r["heads"] * r["vdim"]
            t[mx + "right.q"], t[mx + "right.k"], t[mx + "right.v"] = lin(nqk, e, 2.0), lin(nqk, e), lin(nv, e)
            t[mx + "right.g"], t[mx + "right.o"] = lin(nv, e, 2.0), lin(e, nv)
            t[mx + "right.norm"] = rnd(r["vdim"], std=0.1, mean=1.0)
            t[mx + "right.a1"], t[mx + "right.a2"] = lin(rank, e, 2.0), lin(nqk, rank, 2.0)
            t[mx + "right.a2.b"] = rnd(nqk, std=1.0, mean=2.0)
            t[mx + "left.out"], t[mx + "right.out"] = rnd(e, std=0.1, mean=1.0), rnd(e, std=0.1, mean=1.0)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        fp = pre + "mlp."
        if mlp["kind"] == "dense":
            t[fp + "gate"], t[fp + "up"], t[fp + "down"] = lin(mlp["ff"], e, 2.0), lin(mlp["ff"], e), lin(e, mlp["ff"])
        else:
            ff = mlp["expert"]["ff"]
            t[fp + "router"] = lin(mlp["router"]["experts"], e, 3.0)
            for x in range(mlp["router"]["experts"]):
                # large enough that the clamps of the gated unit are reached now and then
                t[f"{fp}e{x}.gate"], t[f"{fp}e{x}.up"] = lin(ff, e, 3.0), lin(ff, e, 3.0)
                t[f"{fp}e{x}.down"] = lin(e, ff)
    return t
