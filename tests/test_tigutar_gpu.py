"""The Tigutar parts and whole models on the GPU against the plain implementation of `plain_tigutar.py`: each mechanism
alone; a prompt whole, in pieces down to two tokens and token by token; batches of unequal requests against each alone;
slots and pages used again; keys far away, at page borders and just inside and outside a window, in prompts and in
decoding; the sink; the first tokens of a sequence; long decoding; sizes that differ in everything (and values that a
model may happen to make equal or 1); greedy generation through `Engine.generate`.  Configurations and weights are made
here."""
import copy
import io
import json
import os
import tempfile

import pytest
import torch

import plain_tigutar as P
from rbitnet_amd.cache import Cache
from rbitnet_amd.config.spec import PartSpec
from rbitnet_amd.engine.context import StepBatch, StepContext
from rbitnet_amd.parts import BuildEnv, build_part
from rbitnet_amd.parts.stream import ScaledSum

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64


@pytest.fixture(autouse=True)
def _same_numbers_every_run():
    torch.manual_seed(20240607)


@pytest.fixture(scope="module")
def lib():
    from rbitnet_amd.csrc.lib import kernels
    return kernels()


def _env(lib, hidden, dtype):
    return BuildEnv(hidden_size=hidden, dtype=dtype, device=torch.device(DEV), lib=lib)


def _rel(got, want):
    want = want.double().cpu()
    return float((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-30))


def _rms(got, want):
    want = want.double().cpu()
    return float(((got.double().cpu() - want) ** 2).mean().sqrt() / want.abs().max().clamp_min(1e-30))


def _close(got, want, dtype) -> bool:
    """float32: every value within 2e-5 of the largest.  bfloat16 rounds activations at every product's input, and a
    recurrent state carries such errors on for hundreds of tokens: the root mean square error is bounded tightly (a
    wrong formula, window, state or sink moves it by far more), the largest single error loosely."""
    if dtype in (torch.float32, "float32"):
        return _rel(got, want) < 2e-5
    return _rms(got, want) < 1e-2 and _rel(got, want) < 1e-1


def _close_rows(got, want, dtype) -> bool:
    """Whole models with routed experts: in bfloat16 a router's close call may go the other way for a token now and
    then (its input is rounded), which moves that token's logits and little else.  So the bound is on the rows: the
    median row as close as bfloat16 allows, and at most one row in ten further off.  A wrong mechanism moves every row."""
    if dtype in (torch.float32, "float32"):
        return _rel(got, want) < 2e-5
    want = want.double().cpu()
    err = ((got.double().cpu() - want) ** 2).mean(-1).sqrt() / want.abs().max()
    return float(err.median()) < 6e-3 and float((err > 3e-2).double().mean()) <= 0.1


def _bf(t):
    return t.to(torch.bfloat16).to(F64)


def _step(lib, cache, slots, q_lens):
    past = [cache.length(s) for s in slots]
    cache.reserve(slots, q_lens)
    return StepContext.for_batch(DEV, StepBatch(slots, past, [[0] * q for q in q_lens], [], cache.block_tables(slots)),
                                 n_compute_units=lib.n_compute_units)


def _place(part, w, dtype):
    specs = part.tensor_specs()
    return {n: w[n].to(DEV, torch.float32 if specs[n].role == "gain" else dtype).contiguous() for n in specs}


def _requests(part):
    many = getattr(part, "cache_requests", None)
    return [many()] if many else [part.cache_request()]


def _run_mixer(lib, part, x, cuts, dtype, pages=8):
    """The mixer on x [T, E] fed in pieces of the given sizes, through a cache of its own."""
    cache = Cache(_requests(part), 2, 64 * pages, dtype, DEV)
    cache.alloc_slot()                                    # slot 0 stays idle: the sequence lives in slot 1
    slot = cache.alloc_slot()
    outs, at = [], 0
    for n in cuts:
        ctx = _step(lib, cache, [slot], [n])
        outs.append(part.forward(x[at:at + n].to(DEV, dtype).contiguous(), ctx, cache.view(0, ctx.block_tables)))
        cache.commit([slot], [n])
        at += n
    return torch.cat(outs)


def _mixer_weights(kind, hidden, p, seed):
    cfg = {"vocab": 4, "width": hidden, "layers": [{"type": kind, "mixer": p, "mlp": None}]}
    t = P.random_tigutar_tensors(cfg, seed)
    return {k[len("l0.mix."):]: v for k, v in t.items() if k.startswith("l0.mix.")}


def _softmax_spec(p, gated, cache_from=None):
    rot = p["rot"]
    position = (PartSpec("rope", {"head_dim": rot["dims"], "theta": rot["base"], "style": "half", "max_positions": 4096})
                if rot["dims"] else PartSpec("none", {}))
    return PartSpec("attention", {
        "num_heads": p["heads"], "num_kv_heads": p["kv_heads"], "head_dim": p["dim"], "value_dim": p["vdim"], "scale": p["scale"],
        "window": (p.get("mask") or {}).get("size"), "cache_from": cache_from, "sink": gated, "head_gate": gated,
        "position": position, "names": {"q": "q", "k": "k", "v": "v", "o": "o", "sink": "sink", "gate": "g"}})


# ---------------------------------------------------------------------------- small kernels
def test_layer_norm_with_the_scaled_sum_of_two_terms(lib):
    for e, dtype in ((40, torch.float32), (256, torch.bfloat16), (50, torch.float32)):
        x, a, b = (torch.randn(9, e, dtype=F64) for _ in range(3))
        w, bias = 1 + 0.2 * torch.randn(e, dtype=F64), torch.randn(e, dtype=F64)
        part = build_part("norm", PartSpec("layernorm", {"size": e, "eps": 1e-4, "names": {"weight": "", "bias": "b"}}),
                          _env(lib, e, dtype))
        part.load({"": w.float().to(DEV), "b": bias.float().to(DEV)})
        tol = 5e-6 if dtype == torch.float32 else 8e-3
        for second in (b, None):
            xd = x.float().to(DEV)
            s = x + 0.3 * (a + (second if second is not None else 0))
            pending = ScaledSum(a.float().to(DEV), None if second is None else second.float().to(DEV), 0.3)
            assert _rel(part.forward(xd, pending), P.layer_norm(s, w, bias, 1e-4)) < tol
            assert _rel(xd, s) < 1e-6                      # the sum went into the stream
            xd = x.float().to(DEV)
            rows = torch.tensor([7, 0, 7], dtype=torch.int32, device=DEV)
            assert _rel(part.forward(xd, pending, rows), P.layer_norm(s[[7, 0, 7]], w, bias, 1e-4)) < tol
            assert torch.equal(xd.cpu(), x.float())        # only some rows asked for: the stream is left as it is


def test_rotation_of_a_part_of_a_head_and_padded_heads(lib):
    """rope_store alone: first positions, a page's border, rotated part smaller than the head, keys and values of
    different sizes laid out with the larger one."""
    hq, hk, dim, vdim, rot, pad, n = 3, 1, 12, 20, 8, 20, 70
    from rbitnet_amd.parts import CacheRequest
    cache = Cache([CacheRequest("kv", heads=hk, head_dim=pad)], 1, 128, torch.float32, DEV)
    slot = cache.alloc_slot()
    ctx = _step(lib, cache, [slot], [n])
    view = cache.view(0, ctx.block_tables)
    qkv = torch.randn(n, hq * dim + hk * dim + hk * vdim, dtype=F64)
    f = torch.tensor([77.0 ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=F64)
    ang = torch.arange(n, dtype=F64)[:, None] * f
    q_out = torch.empty(n, hq, pad, dtype=torch.float32, device=DEV)
    lib.rope_store(qkv.float().to(DEV), torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV), rot, q_out,
                   view.k_pages, view.v_pages, ctx.tok_pos, ctx.tok_seq, view.block_table, hq, hk, dim, vdim, pad)
    want_q = P.rotate(qkv[:, :hq * dim].view(n, hq, dim), 77.0, rot)
    want_k = P.rotate(qkv[:, hq * dim:(hq + hk) * dim].view(n, hk, dim), 77.0, rot)
    assert _rel(q_out[:, :, :dim], want_q) < 1e-6 and float(q_out[:, :, dim:].abs().max()) == 0.0
    pages = view.block_table[0].tolist()
    for t in (0, 1, 63, 64, 69):
        kp = view.k_pages[pages[t // 64], :, t % 64]
        vp = view.v_pages[pages[t // 64], :, t % 64]
        assert _rel(kp[:, :dim], want_k[t]) < 1e-6 and float(kp[:, dim:].abs().max()) == 0.0
        assert _rel(vp[:, :vdim], qkv[t, (hq + hk) * dim:].view(hk, vdim)) < 1e-6


# ---------------------------------------------------------------------------- softmax attention
ATTENTIONS = [
    dict(heads=4, kv_heads=2, dim=16, vdim=24, rot={"base": 100.0, "dims": 8}, scale=0.3),                   # values larger, part rotated
    dict(heads=3, kv_heads=3, dim=24, vdim=8, rot={"base": 5000.0, "dims": 24}, scale=0.2),                  # values smaller, no sharing
    dict(heads=8, kv_heads=2, dim=64, vdim=64, rot={"base": 10000.0, "dims": 64}, scale=0.125),              # the matrix cores' own sizes
    dict(heads=6, kv_heads=3, dim=64, vdim=128, rot={"base": 1e6, "dims": 32}, scale=0.1, mask={"size": 70}),  # padded to 128, window
    dict(heads=1, kv_heads=1, dim=6, vdim=5, rot={"base": 10.0, "dims": 0}, scale=1.0, mask={"size": 1}),      # no rotation, sees itself only
    dict(heads=2, kv_heads=1, dim=128, vdim=64, rot={"base": 300.0, "dims": 128}, scale=0.05, mask={"size": 64}),
    dict(heads=2, kv_heads=1, dim=7, vdim=9, rot={"base": 20.0, "dims": 6}, scale=0.4, mask={"size": 129}),       # odd sizes
    dict(heads=34, kv_heads=2, dim=64, vdim=64, rot={"base": 1e4, "dims": 64}, scale=0.125),                    # 17 heads on one
    dict(heads=2, kv_heads=2, dim=5, vdim=5, rot={"base": 20.0, "dims": 0}, scale=0.5),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("gated", [True, False])
@pytest.mark.parametrize("p", ATTENTIONS)
def test_attention_whole_in_pieces_and_token_by_token(lib, p, gated, dtype):
    hidden, t_len = 64, 200
    part = build_part("mixer", _softmax_spec(p, gated), _env(lib, hidden, dtype))
    w = _mixer_weights("attention", hidden, p, seed=p["heads"] + p["dim"])
    if not gated:
        del w["sink"], w["g"]
    part.load(_place(part, w, dtype))
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want, _ = P.softmax_attention(x, w, p)
    for cuts in ([t_len], [63, 1, 1, 2, 61, 72], [130] + [1] * 70, [2] * 5 + [190]):
        assert _close(_run_mixer(lib, part, x, cuts, dtype), want, dtype), cuts


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,dim,vdim", [(80, 64, 128), (64, 64, 64), (65, 16, 16), (7, 8, 12)])
def test_a_key_that_stands_out_just_inside_and_just_outside_the_window(lib, dtype, window, dim, vdim):
    """One token's input is scaled so that its key takes the softmax of the query at the window's last position: that
    output holds its value, the next position's does not.  In a prompt and in decoding, the key in the first page and
    at a page's border."""
    hidden = 64
    p = dict(heads=2, kv_heads=1, dim=dim, vdim=vdim, rot={"base": 1000.0, "dims": 0}, scale=1.0 / (8 * dim ** 0.5), mask={"size": window})
    part = build_part("mixer", _softmax_spec(p, False), _env(lib, hidden, dtype))
    w = _mixer_weights("attention", hidden, p, seed=window)
    del w["sink"], w["g"]
    part.load(_place(part, w, dtype))
    for at in (3, 63, 64):
        t_len = at + window + 5
        inside, outside = at + window - 1, at + window
        # the key's input scaled so that its score with the query at the edge is +20 for the head that sees it best; inputs
        # are drawn again until a factor of at most 30 does that (a larger one makes scores that bfloat16 cannot hold)
        for _ in range(50):
            x = _bf(torch.randn(t_len, hidden, dtype=F64))
            raw = torch.einsum("hd,d->h", (x[inside] @ w["q"].T).view(2, dim), x[at] @ w["k"].T) * p["scale"]
            best = int(raw.abs().argmax())
            if abs(20.0 / float(raw[best])) <= 30:
                break
        x[at] = _bf(x[at] * (20.0 / float(raw[best])))
        q, k = (x @ w["q"].T).view(t_len, 2, dim), (x @ w["k"].T).view(t_len, 1, dim)
        a = P.attention_weights(q, k, p["scale"], window, None)
        assert float(a[best, inside, at]) > 0.9 and float(a[:, outside, at].max()) == 0.0       # the edge shows in the plain weights
        want, _ = P.softmax_attention(x, w, p)
        for cuts in ([t_len], [at + 1] + [1] * (t_len - at - 1), [inside, 1, 1, t_len - inside - 2]):
            got = _run_mixer(lib, part, x, cuts, dtype)
            assert _close(got, want, dtype), (at, cuts)
            assert _close(got[[inside, outside]], want[[inside, outside]], dtype), (at, cuts)


def test_a_far_key_among_hundreds_and_the_sink(lib):
    """Position 2's input is made large: queries 600 tokens later still find it (fp32 and the matrix cores' kernels); a
    sink far above every score empties the output, one far below leaves plain softmax."""
    hidden, t_len = 64, 640
    p = dict(heads=4, kv_heads=1, dim=64, vdim=64, rot={"base": 10000.0, "dims": 64}, scale=0.125)
    w = _mixer_weights("attention", hidden, p, seed=5)
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    x[2] = x[2] * 5
    for sink in (None, 400.0, -400.0):
        ws = dict(w)
        if sink is not None:
            ws["sink"] = torch.full((4,), sink, dtype=F64)
        want, _ = P.softmax_attention(x, ws, p)
        if sink == 400.0:
            assert float(want.abs().max()) < 1e-6 * float(P.softmax_attention(x, w, p)[0].abs().max())
        for dtype in (torch.float32, torch.bfloat16):
            part = build_part("mixer", _softmax_spec(p, True), _env(lib, hidden, dtype))
            part.load(_place(part, ws, dtype))
            for cuts in ([t_len], [600] + [1] * 40):
                got = _run_mixer(lib, part, x, cuts, dtype, pages=11)
                if sink == 400.0:
                    assert float(got.abs().max()) < 1e-5
                else:
                    assert _close(got, want, dtype), (sink, dtype, cuts)


# ---------------------------------------------------------------------------- recurrences
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("p", [dict(heads=4, kv_heads=2, dim=16, vdim=24, conv=3), dict(heads=2, kv_heads=1, dim=64, vdim=16, conv=5),
                               dict(heads=1, kv_heads=1, dim=8, vdim=8, conv=1), dict(heads=3, kv_heads=3, dim=40, vdim=12, conv=7),
                               dict(heads=2, kv_heads=2, dim=128, vdim=128, conv=2)])
def test_delta_rule_with_a_decay_per_head(lib, p, dtype):
    hidden, t_len = 48, 150
    part = build_part("mixer", PartSpec("gated_delta", dict(p, eps=1e-5)), _env(lib, hidden, dtype))
    w = _mixer_weights("delta", hidden, p, seed=p["dim"])
    part.load(_place(part, w, dtype))
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want = P.delta_mixer(x, w, p, 1e-5)
    for cuts in ([t_len], [63, 1, 1, 2, 61, 22], [100] + [1] * 50, [2, 3, 145]):
        assert _close(_run_mixer(lib, part, x, cuts, dtype), want, dtype), cuts


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("p", [dict(heads=2, dim=32, vdim=48, tau=12.0, decay_rank=16), dict(heads=3, dim=12, vdim=20, tau=2.5, decay_rank=8),
                               dict(heads=1, dim=128, vdim=16, tau=1.0, decay_rank=24), dict(heads=5, dim=8, vdim=8, tau=40.0, decay_rank=8)])
def test_gated_linear_attention(lib, p, dtype):
    hidden, t_len = 48, 150
    part = build_part("mixer", PartSpec("decay_attention", dict(p, eps=1e-5)), _env(lib, hidden, dtype))
    cfg = {"vocab": 4, "width": hidden, "layers": [{"type": "parallel", "mlp": None, "mixer": {
        "left": dict(heads=1, kv_heads=1, dim=8, vdim=8, rot={"base": 10.0, "dims": 8}, scale=1.0, mask={"size": 4}), "right": p}}]}
    t = P.random_tigutar_tensors(cfg, p["dim"])
    w = {k[len("l0.mix.right."):]: v for k, v in t.items() if k.startswith("l0.mix.right.") and k != "l0.mix.right.out"}
    part.load(_place(part, w, dtype))
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want = P.decay_mixer(x, w, p, 1e-5)
    for cuts in ([t_len], [63, 1, 1, 2, 61, 22], [100] + [1] * 50):
        assert _close(_run_mixer(lib, part, x, cuts, dtype), want, dtype), cuts


def test_a_value_written_at_the_first_token_is_read_much_later(lib):
    """The plain rule with decays of exactly 1 (the decay's bias far above zero) keeps the first token's k v^T for good:
    a state that is lost or cleared between steps shows at once.  A second sequence in another slot does not disturb it."""
    hidden, p = 32, dict(heads=2, dim=16, vdim=8, tau=1.0, decay_rank=8)
    part = build_part("mixer", PartSpec("decay_attention", dict(p, eps=1e-5)), _env(lib, hidden, torch.float32))
    cfg = {"vocab": 4, "width": hidden, "layers": [{"type": "parallel", "mlp": None, "mixer": {
        "left": dict(heads=1, kv_heads=1, dim=8, vdim=8, rot={"base": 10.0, "dims": 8}, scale=1.0, mask={"size": 4}), "right": p}}]}
    t = P.random_tigutar_tensors(cfg, 3)
    w = {k[len("l0.mix.right."):]: v for k, v in t.items() if k.startswith("l0.mix.right.") and k != "l0.mix.right.out"}
    w["a2.b"] = torch.full_like(w["a2.b"], 60.0)
    part.load(_place(part, w, torch.float32))
    x = _bf(torch.randn(260, hidden, dtype=F64))
    x[1:] = x[1:] * 0.05
    want = P.decay_mixer(x, w, p, 1e-5)
    cache = Cache(_requests(part), 2, 64, torch.float32, DEV)
    a, b = cache.alloc_slot(), cache.alloc_slot()
    other = _bf(torch.randn(260, hidden, dtype=F64))
    outs, at = [], 0
    for n in [1, 2, 61, 64, 1, 1, 130]:
        ctx = _step(lib, cache, [b, a], [n, n])                     # the other sequence first, in the same steps
        both = torch.cat([other[at:at + n], x[at:at + n]]).float().to(DEV).contiguous()
        outs.append(part.forward(both, ctx, cache.view(0, ctx.block_tables))[n:])
        cache.commit([b, a], [n, n])
        at += n
    assert _close(torch.cat(outs), want, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_two_mixers_side_by_side(lib, dtype):
    hidden, t_len = 64, 170
    p = {"left": dict(heads=4, kv_heads=2, dim=16, vdim=32, rot={"base": 1000.0, "dims": 16}, scale=0.25, mask={"size": 33}),
         "right": dict(heads=2, dim=16, vdim=24, tau=8.0, decay_rank=8)}
    spec = PartSpec("pair", {"eps": 1e-5, "left": _softmax_spec(p["left"], False),
                             "right": PartSpec("decay_attention", dict(p["right"], eps=1e-5))})
    part = build_part("mixer", spec, _env(lib, hidden, dtype))
    w = _mixer_weights("parallel", hidden, p, seed=9)
    part.load(_place(part, w, dtype))
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want = P.side_by_side(x, w, p, 1e-5)
    for cuts in ([t_len], [63, 1, 1, 2, 61, 42], [120] + [1] * 50):
        assert _close(_run_mixer(lib, part, x, cuts, dtype), want, dtype), cuts


# ---------------------------------------------------------------------------- routed experts
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden,ff,experts,top,limit", [(64, 32, 12, 1, 1.7), (64, 64, 5, 2, 1.0), (48, 20, 3, 3, 0.7),
                                                         (96, 96, 40, 4, 3.0), (32, 32, 1, 1, 2.0), (128, 64, 130, 2, 2.0)])
def test_routed_experts(lib, dtype, hidden, ff, experts, top, limit):
    cfg = {"vocab": 4, "width": hidden, "layers": [{"type": "delta", "mixer": dict(heads=1, kv_heads=1, dim=8, vdim=8, conv=2),
           "mlp": {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}}]}
    t = P.random_tigutar_tensors(cfg, experts + top)
    w = {k[len("l0.mlp."):]: v for k, v in t.items() if k.startswith("l0.mlp.")}
    part = build_part("feed_forward", PartSpec("routed_experts", {"experts": experts, "top": top, "intermediate_size": ff,
                                                                  "limit": limit}), _env(lib, hidden, dtype))
    part.load(_place(part, w, dtype))
    for n in (1, 7, 16, 150):
        x = _bf(torch.randn(n, hidden, dtype=F64))
        want = P.routed_ff(x, w, experts, top, limit)
        got = part.forward(x.to(DEV, dtype).contiguous(), None)
        if dtype == torch.float32:
            assert _rel(got, want) < 2e-5, n
        else:
            # a score that differs in its last bits may choose another expert where two are as good as equal: rows
            # whose two best unchosen and chosen scores lie close are left out
            z = (x @ w["router"].T).sort(dim=-1, descending=True).values
            clear = (z[:, top - 1] - z[:, top]) > 1e-3 if top < experts else torch.ones(n, dtype=torch.bool)
            assert int(clear.sum()) >= 0.9 * n - 1
            assert _rms(got[clear], want[clear]) < 1e-2 and _rel(got[clear], want[clear]) < 1e-1, n
        # a token's result does not depend on what else the step holds, beyond the rounding of the router's product
        # (whose kernel follows the number of tokens) and of the scaled input
        alone = part.forward(x[n // 2:n // 2 + 1].to(DEV, dtype).contiguous(), None)
        assert _rel(alone[0], got[n // 2]) < (1e-5 if dtype == torch.float32 else 2e-2)


# ---------------------------------------------------------------------------- whole models
def _soft(heads, kv_heads, dim, vdim, rot_dims, base, scale, **more):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, rot={"base": base, "dims": rot_dims}, scale=scale, **more)


def _moe(ff, limit, experts, top):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


# everything different: head sizes that differ between keys and values both ways, heads rotated in part, windows that
# end inside a page, several experts a token, a layer without a feed-forward, a reader of another layer's keys
MODEL_A = {"architecture": "Tigutar", "vocab": 70, "width": 48, "residual_mult": 0.4, "norm": {"eps": 1e-5}, "layers": [
    {"type": "delta", "mixer": dict(heads=4, kv_heads=2, dim=12, vdim=20, conv=3), "mlp": _moe(24, 1.0, 6, 2)},
    {"type": "attention", "mixer": _soft(4, 2, 16, 24, 8, 100.0, 0.3), "mlp": _dense(64)},
    {"type": "parallel", "mixer": {"left": _soft(2, 1, 24, 8, 24, 5000.0, 0.25, mask={"size": 37}),
                                   "right": dict(heads=3, dim=8, vdim=12, tau=4.0, decay_rank=8)}, "mlp": None},
    {"type": "attention", "mixer": _soft(6, 2, 16, 24, 8, 100.0, 0.2, kv_from=1), "mlp": _moe(16, 2.5, 3, 3)},
    {"type": "parallel", "mixer": {"left": _soft(3, 3, 8, 8, 4, 50.0, 0.5, mask={"size": 64}),
                                   "right": dict(heads=1, dim=16, vdim=16, tau=30.0, decay_rank=16)}, "mlp": _dense(40)}]}
# what a model may happen to have: one head, one expert, one tap, sizes equal everywhere, factor 1, a window of 1
MODEL_B = {"architecture": "Tigutar", "vocab": 33, "width": 32, "residual_mult": 1.0, "norm": {"eps": 1e-6}, "layers": [
    {"type": "parallel", "mixer": {"left": _soft(1, 1, 32, 32, 32, 10000.0, 1.0, mask={"size": 1}),
                                   "right": dict(heads=1, dim=32, vdim=32, tau=1.0, decay_rank=32)}, "mlp": _moe(32, 2.0, 1, 1)},
    {"type": "delta", "mixer": dict(heads=1, kv_heads=1, dim=32, vdim=32, conv=1), "mlp": _dense(32)},
    {"type": "attention", "mixer": _soft(1, 1, 32, 32, 32, 10000.0, 1.0), "mlp": None}]}
# sizes on the matrix cores' grid: heads of 64 and 128, keys of 64 beside values of 128 and the other way round, experts
# on the matrix cores
MODEL_C = {"architecture": "Tigutar", "vocab": 320, "width": 128, "residual_mult": 0.45, "norm": {"eps": 1e-5}, "layers": [
    {"type": "attention", "mixer": _soft(4, 1, 128, 128, 128, 10000.0, 0.09), "mlp": _dense(256)},
    {"type": "delta", "mixer": dict(heads=4, kv_heads=2, dim=32, vdim=64, conv=3), "mlp": _moe(96, 1.5, 8, 2)},
    {"type": "parallel", "mixer": {"left": _soft(4, 2, 64, 128, 32, 2e5, 0.11, mask={"size": 80}),
                                   "right": dict(heads=1, dim=64, vdim=32, tau=5.0, decay_rank=16)}, "mlp": _moe(32, 3.0, 24, 1)},
    {"type": "attention", "mixer": _soft(8, 1, 128, 128, 128, 10000.0, 0.07, kv_from=0), "mlp": _dense(128)},
    {"type": "parallel", "mixer": {"left": _soft(2, 2, 128, 64, 64, 1e4, 0.09, mask={"size": 130}),
                                   "right": dict(heads=4, dim=16, vdim=16, tau=8.0, decay_rank=8)}, "mlp": _dense(256)}]}
# sizes off every grid: a width that is no multiple of 4, odd heads, seven experts of ten channels, one tap and nine
MODEL_D = {"architecture": "Tigutar", "vocab": 37, "width": 50, "residual_mult": 0.7, "norm": {"eps": 1e-4}, "layers": [
    {"type": "parallel", "mixer": {"left": _soft(3, 1, 10, 14, 6, 33.0, 0.3, mask={"size": 3}),
                                   "right": dict(heads=3, dim=5, vdim=7, tau=3.0, decay_rank=3)}, "mlp": _moe(10, 0.8, 7, 3)},
    {"type": "attention", "mixer": _soft(5, 5, 6, 6, 2, 7.0, 0.4), "mlp": None},
    {"type": "delta", "mixer": dict(heads=6, kv_heads=2, dim=9, vdim=3, conv=9), "mlp": _dense(31)},
    {"type": "attention", "mixer": _soft(5, 5, 6, 6, 2, 7.0, 0.6, kv_from=1), "mlp": _moe(9, 5.0, 2, 1)},
    {"type": "delta", "mixer": dict(heads=1, kv_heads=1, dim=3, vdim=11, conv=1), "mlp": None}]}
MODELS = {"A": (MODEL_A, 21), "B": (MODEL_B, 22), "C": (MODEL_C, 23), "D": (MODEL_D, 24)}
_TMP = tempfile.TemporaryDirectory(prefix="tigutar_models_")
_MADE = {}


def _model(name):
    """(folder, oracle) of a model written once per session: config.json (without the sizes that only the weights
    know) and bfloat16 weights."""
    if name not in _MADE:
        from rbitnet_amd.weights.safetensors_io import save_file
        cfg, seed = MODELS[name]
        tensors = P.random_tigutar_tensors(cfg, seed)
        stored = copy.deepcopy(cfg)
        for layer in stored["layers"]:
            if layer["type"] == "parallel":
                layer["mixer"]["right"].pop("decay_rank")
        folder = os.path.join(_TMP.name, name)
        os.makedirs(folder)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(stored, f)
        save_file(os.path.join(folder, "model.safetensors"), [(k, v.to(torch.bfloat16)) for k, v in tensors.items()])
        _MADE[name] = (folder, P.PlainTigutar(copy.deepcopy(cfg), tensors))
    return _MADE[name]


def _tokens(name, n, seed):
    g = torch.Generator().manual_seed(100 * seed + n)
    return torch.randint(0, MODELS[name][0]["vocab"], (n,), generator=g).tolist()


def _engine(name, dtype, **kw):
    import rbitnet_amd
    return rbitnet_amd.Engine.load_path(_model(name)[0], dtype=dtype, max_seq_len=1024, **kw)


def test_every_layer_of_a_model_against_the_plain_stream():
    """The residual stream after every layer (float32), so that a fault names its layer."""
    import rbitnet_amd.engine.model as M
    eng = _engine("A", "float32", max_tokens=64 * 4, max_batch=1)
    toks = _tokens("A", 90, 4)
    want = []
    _model("A")[1].logits(toks, want)
    seen = []
    orig = M.run_blocks

    def traced(blocks, schedule, x, ctx, cache, last_norm=None):
        pending = None
        for place, i in enumerate(schedule):
            pending = blocks[i].forward(x, pending, ctx, cache.view(place, ctx.block_tables), next_norm=None)
            a, b, scale = pending.parts()
            seen.append((x + scale * (a + (b if b is not None else 0))).cpu())
        return pending

    M.run_blocks = traced
    try:
        slot = eng.alloc_slot()
        eng.use_plans = False
        eng.step([(slot, toks)], "last")
    finally:
        M.run_blocks = orig
    assert len(seen) == len(want)
    for i, (g, w) in enumerate(zip(seen, want)):
        assert _rel(g, w) < 2e-5, i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_model_whole_in_pieces_and_decoded(name, dtype):
    eng = _engine(name, dtype, max_tokens=64 * 12, max_batch=3)
    toks = _tokens(name, 200, 1)
    want = _model(name)[1].logits(toks)
    for cuts in ([200], [130] + [1] * 70, [2, 2, 3, 57, 64, 1, 65, 6], [1] * 5 + [195]):
        slot = eng.alloc_slot()
        out, at = [], 0
        for n in cuts:
            out.append(eng.step([(slot, toks[at:at + n])], "all"))
            at += n
        eng.free_slot(slot)
        assert _close_rows(torch.cat(out), want, dtype), cuts


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C", "D"])
def test_batches_of_unequal_requests_and_slots_used_again(name, dtype):
    """Four requests of 1 to 150 tokens start together and are decoded together, the short ones leaving early; then two
    new requests take the freed slots and pages.  Every request's logits are those it has alone."""
    eng = _engine(name, dtype, max_tokens=64 * 8, max_batch=4)
    oracle = _model(name)[1]
    for wave, lens in enumerate(([1, 150, 67, 30], [64, 129])):
        seqs = [_tokens(name, n + 12, 7 + wave) for n in lens]
        want = [oracle.logits(s) for s in seqs]
        slots = [eng.alloc_slot() for _ in seqs]
        got = [[] for _ in seqs]
        logits = eng.step([(sl, s[:n]) for sl, s, n in zip(slots, seqs, lens)], "all")
        off = 0
        for i, n in enumerate(lens):
            got[i].append(logits[off:off + n])
            off += n
        ends = [n + (3 + 4 * i if i < 3 else 12) for i, n in enumerate(lens)]       # they leave at different steps
        at = list(lens)
        live = list(range(len(seqs)))
        while live:
            logits = eng.step([(slots[i], [seqs[i][at[i]]]) for i in live], "last")
            for row, i in enumerate(live):
                got[i].append(logits[row:row + 1])
                at[i] += 1
            for i in [i for i in live if at[i] >= min(ends[i], len(seqs[i]))]:
                eng.free_slot(slots[i])
                live.remove(i)
        for i in range(len(seqs)):
            g = torch.cat(got[i])
            assert _close_rows(g, want[i][:g.shape[0]], dtype), (wave, i)
        eng.cache.check()


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("C", "bfloat16")])
def test_long_decoding_and_greedy_generation_through_the_engine(name, dtype):
    """Greedy generation through `Engine.generate` (its scheduler, its captured decode step) gives the plain
    implementation's greedy tokens for a batch of unequal prompts, past every window of the model."""
    eng = _engine(name, dtype, max_tokens=64 * 16, max_batch=5)
    oracle = _model(name)[1]
    limits = (150, 40, 90, 12, 25)
    prompts = [_tokens(name, n, 3) for n in (5, 70, 1, 33, 64)]
    results = eng.generate(prompts, max_tokens=list(limits), temperature=0.0)
    margin = 1e-4 if dtype == "float32" else 0.15
    for p, r, n in zip(prompts, results, limits):
        assert len(r.tokens) == n and r.finish_reason == "length"
        seq = list(p) + r.tokens
        logits = oracle.logits(seq[:-1])
        top2 = logits[len(p) - 1:].topk(2, dim=-1)
        greedy = top2.indices[:, 0].tolist()
        clear = (top2.values[:, 0] - top2.values[:, 1]) > margin          # a tie within rounding may go either way
        same = sum(1 for g, t, c in zip(greedy, r.tokens, clear.tolist()) if c and g == t)
        # bfloat16: a router's close call that goes the other way moves a token's logits by more than the margin
        assert same >= (1.0 if dtype == "float32" else 0.9) * int(clear.sum())
        assert int(clear.sum()) > (0.9 if dtype == "float32" else 0.5) * n
    assert eng.stats["decode_tokens"] > 0 and eng.model.graph_safe and eng.model.plan_safe


def test_replay_and_command_line_on_a_model_of_this_design(tmp_path, capsys):
    import numpy as np
    from rbitnet_amd import cli
    from rbitnet_amd.replay import replay
    folder, oracle = _model("B")
    eng = _engine("B", "float32", max_tokens=64 * 6, max_batch=4)
    a, b = _tokens("B", 70, 5), _tokens("B", 9, 6)
    lines = [json.dumps({"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 65]},
                                                {"id": "b", "tokens": b[:8], "want": []}], "end": []}),
             json.dumps({"step": 1, "entries": [{"id": "a", "tokens": a[66:67], "want": [0]},
                                                {"id": "b", "tokens": b[8:9], "want": [0]}], "end": ["b"]}),
             json.dumps({"step": 2, "entries": [{"id": "a", "tokens": a[67:], "want": [2]}], "end": ["a"]})]
    log = io.StringIO()
    assert replay(eng, io.StringIO("\n".join(lines) + "\n"), str(tmp_path / "out"), log=log) == 3
    wa, wb = oracle.logits(a), oracle.logits(b)
    vocab = MODELS["B"][0]["vocab"]
    got = [np.fromfile(tmp_path / "out" / f"{i}.f32", dtype="<f4").reshape(-1, vocab) for i in range(3)]
    assert _close(torch.from_numpy(got[0]), wa[[0, 65]], "float32")
    assert _close(torch.from_numpy(got[1]), torch.stack([wa[66], wb[8]]), "float32")
    assert _close(torch.from_numpy(got[2]), wa[[69]], "float32")
    assert eng.cache.live_slots == []
    del eng
    capsys.readouterr()
    assert cli.main(["generate", "--model", folder, "--dtype", "float32", "--prompt-ids", ",".join(str(t) for t in b),
                     "--max-tokens", "5", "--temperature", "0"]) == 0
    rec = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert len(rec["tokens"]) == 5 and rec["tokens"][0] == int(oracle.logits(b)[-1].argmax())
