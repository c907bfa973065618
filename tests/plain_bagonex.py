"""A plain, slow float64 implementation of the Bagonex decoder, one function per mechanism, whole sequences only
(no cache, no state, no batches): the oracle of the tests.  It shares no code with the package.

Notation: T tokens, E width, S copies of the stream; weights are [out, in] and applied as x @ W.T.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    y = (x - mu) / torch.sqrt(var + eps) * w
    return y if b is None else y + b


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def causal_conv(x, w):
    """x [T, C], w [C, taps]: out_t = sum_j w[:, j] x_(t - taps + 1 + j), zeros before the start."""
    t_len, c = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, c, dtype=x.dtype), x])
    out = torch.zeros_like(x)
    for j in range(taps):
        out = out + padded[j:j + t_len] * w[:, j]
    return out


def silu(x):
    return x / (1 + torch.exp(-x))


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def xielu(z, p, q):
    pos = softplus(p) * z * z + z / 2
    neg = (0.5 + softplus(q)) * (torch.expm1(torch.clamp(z, max=0)) - z) + z / 2
    return torch.where(z > 0, pos, neg)


def tanh_cap(x, cap):
    return cap * torch.tanh(x / cap)


def delta_recurrence(q, k, v, g, beta, state=None):
    """q, k, g [T, H, dk], v [T, H, dv], beta [T, H] -> o [T, H, dv] and the last state [H, dk, dv]."""
    t_len, h, dk = q.shape
    dv = v.shape[-1]
    s = torch.zeros(h, dk, dv, dtype=q.dtype) if state is None else state.clone()
    o = torch.zeros(t_len, h, dv, dtype=q.dtype)
    for t in range(t_len):
        s = g[t].unsqueeze(-1) * s
        u = beta[t].unsqueeze(-1) * (v[t] - torch.einsum("hkv,hk->hv", s, k[t]))
        s = s + torch.einsum("hk,hv->hkv", k[t], u)
        o[t] = torch.einsum("hkv,hk->hv", s, q[t])
    return o, s


def channel_delta(h, w: Dict[str, torch.Tensor], heads, kv_heads, dim, vdim, eps, unit_eps=1e-6):
    t_len = h.shape[0]
    q = silu(causal_conv(h @ w["q"].T, w["q.conv"])).view(t_len, kv_heads, dim)
    k = silu(causal_conv(h @ w["k"].T, w["k.conv"])).view(t_len, kv_heads, dim)
    v = silu(causal_conv(h @ w["v"].T, w["v.conv"])).view(t_len, heads, vdim)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + unit_eps) * dim ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + unit_eps)
    q = q.repeat_interleave(heads // kv_heads, 1)
    k = k.repeat_interleave(heads // kv_heads, 1)
    beta = torch.sigmoid(h @ w["b"].T)
    a = (h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]
    g = torch.exp(-torch.exp(w["A_log"]).view(1, heads, 1) * softplus(a).view(t_len, heads, dim))
    o, _ = delta_recurrence(q, k, v, g, beta)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * w["norm"]
    gate = torch.sigmoid((h @ w["g1"].T) @ w["g2"].T).view(t_len, heads, vdim)
    return (o * gate).reshape(t_len, heads * vdim) @ w["o"].T


def sink_softmax(scores, sink):
    """scores [..., J] with -inf where masked, sink broadcastable to [..., 1]: the weights of the J keys."""
    mx = torch.maximum(scores.max(-1, keepdim=True).values, sink)
    e = torch.exp(scores - mx)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink - mx))


def latent_of(h, w, eps):
    return rms_norm(h @ w["dkv"].T, w["dkv.norm"], eps)


def latent_attention(h, c, w, heads, dim, vdim, scale, eps):
    """h [T, E] the layer's input, c [T, R] the latents it attends to (its own or another layer's)."""
    t_len = h.shape[0]
    q = (rms_norm(h @ w["dq"].T, w["dq.norm"], eps) @ w["uq"].T).view(t_len, heads, dim)
    k = (c @ w["uk"].T).view(t_len, heads, dim)
    v = (c @ w["uv"].T).view(t_len, heads, vdim)
    s = torch.einsum("thd,jhd->htj", q, k) * scale
    s = s.masked_fill(~torch.ones(t_len, t_len, dtype=torch.bool).tril(), -math.inf)
    p = sink_softmax(s, w["sink"].view(heads, 1, 1))
    return torch.einsum("htj,jhd->thd", p, v).reshape(t_len, heads * vdim) @ w["o"].T


def dense_ff(h, w):
    return xielu(h @ w["up"].T, w["act"][0], w["act"][1]) @ w["down"].T


def streams_update(xs: List[torch.Tensor], mix, out, y):
    n = len(xs)
    return [sum(mix[s, j] * xs[s] for s in range(n)) + out[j] * y for j in range(n)]


class PlainBagonex:
    def __init__(self, config: Dict, tensors: Dict[str, torch.Tensor]):
        self.cfg = config
        self.w = {k: v.to(F64) for k, v in tensors.items()}

    def sub(self, prefix: str) -> Dict[str, torch.Tensor]:
        return {k[len(prefix):]: v for k, v in self.w.items() if k.startswith(prefix)}

    def logits(self, tokens, layers_out: Optional[list] = None) -> torch.Tensor:
        cfg, w = self.cfg, self.w
        eps, n = cfg["norm"]["eps"], cfg["streams"]
        xs = [w["embed"][list(tokens)].clone() for _ in range(n)]
        latents = {}
        for i, layer in enumerate(cfg["layers"]):
            own = self.sub(f"l{i}.")
            m = layer["mixer"]
            for p in (1, 2):
                if p == 2 and layer["mlp"] is None:
                    continue
                u = sum(own[f"hc{p}.in"][s] * xs[s] for s in range(n))
                h = layer_norm(u, own[f"norm{p}"], own[f"norm{p}.b"], eps)
                if p == 1:
                    h = h + causal_conv(h, own["canon1"])
                    mw = self.sub(f"l{i}.mix.")
                    if layer["type"] == "channel_delta":
                        y = channel_delta(h, mw, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"], eps)
                    else:
                        if m.get("kv_from") is None:
                            latents[i] = latent_of(h, mw, eps)
                        y = latent_attention(h, latents[i if m.get("kv_from") is None else m["kv_from"]], mw, m["heads"],
                                             m["dim"], m["vdim"], m["scale"], eps)
                else:
                    y = dense_ff(h, self.sub(f"l{i}.mlp."))
                xs = streams_update(xs, own[f"hc{p}.mix"], own[f"hc{p}.out"], y * own[f"ls{p}"])
            if layers_out is not None:
                layers_out.append(sum(xs))
        x = layer_norm(sum(xs), w["final.norm"], w["final.norm.b"], eps)
        out = x @ w["head"].T
        cap = cfg.get("logit_softcap")
        return out if cap is None else tanh_cap(out, cap)


def random_bagonex_tensors(config: Dict, seed: int, ranks=(6, 10)) -> Dict[str, torch.Tensor]:
    """Weights for a configuration, large enough that every mechanism matters in the logits; values that are
    exact in bfloat16, so that a bfloat16 weight file holds the same model."""
    gen = torch.Generator().manual_seed(seed)
    e, n = config["width"], config["streams"]
    r = lambda *shape, std=1.0, mean=0.0: (mean + std * torch.randn(*shape, generator=gen)).to(torch.bfloat16).to(F64)
    t: Dict[str, torch.Tensor] = {"embed": r(config["vocab"], e), "head": r(config["vocab"], e, std=e ** -0.5),
                                  "final.norm": r(e, std=0.1, mean=1.0), "final.norm.b": r(e, std=0.1)}
    for i, layer in enumerate(config["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        for p in (1, 2):
            if p == 2 and layer["mlp"] is None:
                continue
            t[pre + f"norm{p}"], t[pre + f"norm{p}.b"] = r(e, std=0.1, mean=1.0), r(e, std=0.1)
            t[pre + f"ls{p}"] = r(e, std=0.1, mean=0.7)
            t[pre + f"hc{p}.in"], t[pre + f"hc{p}.out"] = r(n, std=0.3, mean=1.0 / n), r(n, std=0.3, mean=1.0)
            t[pre + f"hc{p}.mix"] = (torch.eye(n, dtype=F64) + r(n, n, std=0.2)).to(torch.bfloat16).to(F64)
        t[pre + "canon1"] = r(e, config["canon"]["taps"], std=0.4)
        mp = pre + "mix."
        h = m["heads"]
        if layer["type"] == "channel_delta":
            kv, dk, dv, taps = m.get("kv_heads", h), m["dim"], m["vdim"], m["conv"]
            dr, gr = m.get("decay_rank", ranks[0]), m.get("gate_rank", ranks[1])
            for name, rows in (("q", kv * dk), ("k", kv * dk), ("v", h * dv)):
                t[mp + name], t[mp + name + ".conv"] = r(rows, e, std=e ** -0.5 * 2), r(rows, taps, std=0.5)
            t[mp + "b"], t[mp + "A_log"], t[mp + "norm"] = r(h, e, std=e ** -0.5), r(h, std=0.5, mean=-1.0), r(dv, std=0.1, mean=1.0)
            t[mp + "a1"], t[mp + "a2"] = r(dr, e, std=e ** -0.5), r(h * dk, dr, std=dr ** -0.5 * 2)
            t[mp + "dt_bias"] = r(h * dk, std=1.0, mean=-1.0)
            t[mp + "g1"], t[mp + "g2"] = r(gr, e, std=e ** -0.5), r(h * dv, gr, std=gr ** -0.5 * 2)
            t[mp + "o"] = r(e, h * dv, std=(h * dv) ** -0.5)
        else:
            dk, dv, qr, kr = m["dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            t[mp + "dq"], t[mp + "dq.norm"], t[mp + "uq"] = r(qr, e, std=e ** -0.5), r(qr, std=0.1, mean=1.0), r(h * dk, qr, std=qr ** -0.5 * 2)
            if m.get("kv_from") is None:
                t[mp + "dkv"], t[mp + "dkv.norm"] = r(kr, e, std=e ** -0.5), r(kr, std=0.1, mean=1.0)
            t[mp + "uk"], t[mp + "uv"] = r(h * dk, kr, std=kr ** -0.5 * 2), r(h * dv, kr, std=kr ** -0.5)
            t[mp + "sink"], t[mp + "o"] = r(h, std=1.0), r(e, h * dv, std=(h * dv) ** -0.5)
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            t[pre + "mlp.up"], t[pre + "mlp.down"] = r(ff, e, std=e ** -0.5), r(e, ff, std=ff ** -0.5)
            t[pre + "mlp.act"] = r(2, std=0.5)
    return t
