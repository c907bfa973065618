"""The Bagonex parts and whole models on the GPU against the plain implementation of `plain_bagonex.py`: each
mechanism alone; a prompt whole, in pieces down to two tokens and token by token; batches of unequal requests against
each alone; slots and pages used again; keys far away and at page borders; the sink; the first tokens of a sequence;
long decoding; sizes that differ in everything (and values that a model may happen to make equal or 1); greedy
generation through `Engine.generate`.  Configurations and weights are made here."""
import copy
import json
import math
import os
import tempfile

import pytest
import torch

import plain_bagonex as P
from rbitnet_amd.cache import Cache
from rbitnet_amd.config.spec import PartSpec
from rbitnet_amd.engine.context import StepBatch, StepContext
from rbitnet_amd.parts import BuildEnv, build_part
from rbitnet_amd.parts.short_conv import ACT_NONE, ACT_SILU, ShortConv

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64


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
    wrong formula, window or state moves it by far more), the largest single error loosely."""
    if dtype in (torch.float32, "float32"):
        return _rel(got, want) < 2e-5
    return _rms(got, want) < 1e-2 and _rel(got, want) < 1e-1


def _bf(t):
    """Values that bfloat16 holds exactly, in float64."""
    return t.to(torch.bfloat16).to(F64)


def _step(lib, cache, slots, q_lens):
    past = [cache.length(s) for s in slots]
    cache.reserve(slots, q_lens)
    return StepContext.for_batch(DEV, StepBatch(slots, past, [[0] * q for q in q_lens], [], cache.block_tables(slots)),
                                 n_compute_units=lib.n_compute_units)


def _place(part, w, dtype):
    """The oracle's tensors as the model would hand them to a part: matrices in the compute dtype, the rest float32."""
    specs = part.tensor_specs()
    return {n: w[n].to(DEV, torch.float32 if specs[n].role == "gain" else dtype).contiguous() for n in specs}


# ---------------------------------------------------------------------------- element-wise and norms
def test_layer_norm_of_a_mixture_of_copies(lib):
    for s_, e in ((1, 40), (3, 100), (4, 256)):
        x = torch.randn(s_, 9, e, dtype=F64) * 3 + 1
        coef, w, b = torch.randn(s_, dtype=F64), 1 + 0.2 * torch.randn(e, dtype=F64), torch.randn(e, dtype=F64)
        part = build_part("norm", PartSpec("layernorm", {"size": e, "eps": 1e-4, "names": {"weight": "", "bias": "b"}}),
                          _env(lib, e, torch.float32))
        assert set(part.tensor_specs()) == {"", "b"}
        part.load({"": w.float().to(DEV), "b": b.float().to(DEV)})
        xd = x.float().to(DEV)
        u = sum(coef[s] * x[s] for s in range(s_))
        assert _rel(part.forward(xd, coef=coef.float().to(DEV)), P.layer_norm(u, w, b, 1e-4)) < 5e-6
        rows = torch.tensor([7, 0, 7], dtype=torch.int32, device=DEV)
        assert _rel(part.forward(xd, rows=rows), P.layer_norm(x.sum(0)[[7, 0, 7]], w, b, 1e-4)) < 5e-6
    # one copy, as a plain pre-norm layer uses a norm: the pending term is added to the stream
    x, d = torch.randn(5, 40), torch.randn(5, 40)
    part = build_part("norm", PartSpec("layernorm", {"size": 40, "eps": 1e-5, "bias": False}), _env(lib, 40, torch.bfloat16))
    part.load({"weight": torch.ones(40, device=DEV)})
    xd = x.to(DEV).clone()
    got = part.forward(xd, d.to(DEV))
    assert got.dtype == torch.bfloat16 and _rel(got, P.layer_norm((x + d).double(), torch.ones(40, dtype=F64), None, 1e-5)) < 8e-3
    assert torch.equal(xd.cpu(), x + d)


def test_streams_update_xielu_and_cap(lib):
    for s_ in (1, 2, 5):
        x, y = torch.randn(s_, 7, 24, dtype=F64), torch.randn(7, 24, dtype=F64)
        mix, out, scale = torch.randn(s_, s_, dtype=F64), torch.randn(s_, dtype=F64), torch.randn(24, dtype=F64)
        xd = x.float().to(DEV)
        lib.streams_update(xd, mix.float().to(DEV), out.float().to(DEV), y.float().to(DEV), scale.float().to(DEV))
        want = torch.stack(P.streams_update([x[s] for s in range(s_)], mix, out, y * scale))
        assert _rel(xd, want) < 2e-6
    z = torch.cat([torch.linspace(-30, 30, 1001, dtype=F64), torch.tensor([0.0, -1e-4, 1e-4], dtype=F64)]).view(4, 251)
    for p, q in ((0.3, -0.7), (-5.0, 4.0), (25.0, 0.0)):
        act = torch.tensor([p, q], dtype=F64)
        got = torch.empty(z.shape, dtype=torch.float32, device=DEV)
        lib.xielu(z.float().to(DEV), act.float().to(DEV), got)
        assert _rel(got, P.xielu(z, act[0], act[1])) < 2e-6
    lg = (torch.randn(6, 77, dtype=F64) * 40).float().to(DEV)
    want = P.tanh_cap(lg.double().cpu(), 7.5)
    lib.tanh_cap(lg, 7.5)
    assert _rel(lg, want) < 2e-6


@pytest.mark.parametrize("m,n,k", [(1, 384, 256), (8, 8192, 2048), (16, 16384, 512), (40, 512, 4096), (128, 1024, 8192),
                                   (300, 2048, 1024), (2048, 4096, 1024), (100, 256, 200), (5, 40, 24), (70, 96, 100)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_xielu_in_the_products_epilogue(lib, m, n, k, out_dtype):
    """xIELU(x W^T) from the product's own epilogue, for token counts and sizes that reach each of the product kernels
    (few tokens, rows resident, tiles with and without slices of K, K that is no multiple of 64, sizes off the matrix
    cores' grid), W stored either way: the float32 sums are activated, then rounded once."""
    from rbitnet_amd.parts.linear import pack_rows, xielu_linear
    g = torch.Generator().manual_seed(m + n + k)
    x = _bf(torch.randn(m, k, generator=g, dtype=F64))
    w = _bf(torch.randn(n, k, generator=g, dtype=F64) * k ** -0.5 * 2)
    act = torch.tensor([0.4, -0.3], dtype=F64)
    want = P.xielu(x @ w.T, act[0], act[1])
    wd = w.to(DEV, torch.bfloat16)
    for frag_allowed in (True, False):
        mat = pack_rows(lib, [(wd, 0, None, None)], n, k, torch.bfloat16, torch.device(DEV), frag_allowed)
        got = xielu_linear(lib, x.to(DEV, torch.bfloat16), mat, act.float().to(DEV), out_dtype)
        assert got.dtype == out_dtype and _rel(got, want) < (6e-3 if out_dtype == torch.bfloat16 else 2e-5), frag_allowed
    if k % 8 == 0:                                   # and the plain product beside it is what it was
        plain = torch.empty(m, n, dtype=torch.float32, device=DEV)
        lib.gemm_bf16(x.to(DEV, torch.bfloat16), wd, plain, 0)
        assert _rel(plain, x @ w.T) < 2e-5


@pytest.mark.parametrize("taps", [1, 2, 4])
@pytest.mark.parametrize("residual,act", [(True, ACT_NONE), (False, ACT_SILU)])
def test_short_convolution_in_pieces_and_batches(lib, taps, residual, act):
    """Three sequences of unequal lengths as a batch in unequal pieces (down to one token, and pieces shorter than the
    taps), on columns inside a wider matrix; then a slot that is freed and used again starts from zeros."""
    c, width, col0 = 37, 64, 11
    conv = ShortConv(c, taps, _env(lib, c, torch.float32), residual=residual, act=act)
    w = torch.randn(c, taps, dtype=F64)
    conv.load(w.float().to(DEV))
    req = conv.cache_request("conv")
    assert (req is None) == (taps == 1)
    cache = Cache([req], 3, 64 * 8, torch.float32, DEV)
    lens = [23, 5, 12]
    xs = [torch.randn(n, width, dtype=F64) for n in lens]

    def want(x):
        y = P.causal_conv(x[:, col0:col0 + c], w)
        y = y + x[:, col0:col0 + c] if residual else y
        return P.silu(y) if act == ACT_SILU else y

    slots = [cache.alloc_slot() for _ in lens]
    cuts = [[9, 1, 1, 2, 10], [1, 2, 2], [3, 1, 8]]
    got = [[] for _ in lens]
    for r in range(5):
        live = [i for i in range(3) if r < len(cuts[i])]
        q = [cuts[i][r] for i in live]
        at = [sum(cuts[i][:r]) for i in live]
        ctx = _step(lib, cache, [slots[i] for i in live], q)
        x = torch.cat([xs[i][a:a + n] for i, a, n in zip(live, at, q)]).float().to(DEV)
        state = cache.view(0, ctx.block_tables).states.get("conv")
        out = conv.forward(x, ctx, state, torch.float32, col0=col0)
        cache.commit([slots[i] for i in live], q)
        off = 0
        for i, n in zip(live, q):
            got[i].append(out[off:off + n])
            off += n
    for i in range(3):
        assert _rel(torch.cat(got[i]), want(xs[i])) < 2e-6, i
    cache.free_slot(slots[0])
    s = cache.alloc_slot()
    ctx = _step(lib, cache, [s], [4])
    out = conv.forward(xs[2][:4].float().to(DEV), ctx, cache.view(0, ctx.block_tables).states.get("conv"), torch.float32, col0=col0)
    assert _rel(out, want(xs[2][:4])) < 2e-6


# ---------------------------------------------------------------------------- the gated delta rule
def _delta_weights(hidden, h, kv, dk, dv, taps, dr, gr, seed):
    cfg = {"vocab": 4, "width": hidden, "streams": 1, "canon": {"taps": 1},
           "layers": [{"type": "channel_delta", "mlp": None,
                       "mixer": {"heads": h, "kv_heads": kv, "dim": dk, "vdim": dv, "conv": taps, "decay_rank": dr, "gate_rank": gr}}]}
    t = P.random_bagonex_tensors(cfg, seed)
    return {k[len("l0.mix."):]: v for k, v in t.items() if k.startswith("l0.mix.")}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("h,kv,dk,dv,taps", [(4, 2, 24, 40, 4), (3, 3, 64, 16, 2), (1, 1, 130, 8, 3), (6, 1, 8, 72, 1),
                                             (2, 2, 16, 16, 4)])
def test_delta_rule_mixer_whole_in_pieces_and_token_by_token(lib, dtype, h, kv, dk, dv, taps):
    hidden, t_len = 48, 90
    params = {"heads": h, "kv_heads": kv, "dim": dk, "vdim": dv, "conv": taps, "eps": 1e-5, "decay_rank": 8, "gate_rank": 16}
    part = build_part("mixer", PartSpec("channel_delta", params), _env(lib, hidden, dtype))
    w = _delta_weights(hidden, h, kv, dk, dv, taps, 8, 16, seed=h * 10 + taps)
    part.load(_place(part, w, dtype))
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want = P.channel_delta(x, w, h, kv, dk, dv, 1e-5)
    for cuts in ([t_len], [50, 2, 1, 1, 3, 33], [1] * 12 + [78]):
        cache = Cache([part.cache_requests()], 2, 64 * 4, dtype, DEV)
        cache.alloc_slot()
        slot = cache.alloc_slot()                    # not slot 0: the state is found by the slot's number
        outs, at = [], 0
        for n in cuts:
            ctx = _step(lib, cache, [slot], [n])
            outs.append(part.forward(x[at:at + n].to(DEV, dtype).contiguous(), ctx, cache.view(0, ctx.block_tables)))
            cache.commit([slot], [n])
            at += n
        assert _close(torch.cat(outs), want, dtype), cuts


def test_delta_recurrence_kernel_keeps_what_was_written_long_ago(lib):
    """With decays of 1 and orthogonal unit keys a value written at the first token is read back exactly two hundred
    tokens later, in a step of its own, and a decay of 1/2 per token on one key channel halves what that channel holds;
    the state of another sequence in the batch is not touched."""
    h, dk, dv, n = 2, 32, 48, 200
    cache = Cache([P_REQ(h, dk, dv)], 3, 64, torch.float32, DEV)
    slots = [cache.alloc_slot() for _ in range(3)]
    q = torch.zeros(n, 2 * h * dk + h * dv, dtype=F64)          # q heads | k heads | v heads
    k_idx = lambda t: t % dk
    for t in range(n):
        for head in range(h):
            q[t, h * dk + head * dk + k_idx(t)] = 1.0            # k = e_(t mod dk): overwrites that row every dk tokens
            q[t, 2 * h * dk + head * dv:2 * h * dk + (head + 1) * dv] = t + 1 + head
    q[n - 1, :h * dk] = 0
    for head in range(h):
        q[n - 1, head * dk + 5] = 1.0                            # read row 5: last written at the latest t with t % dk == 5
    g = torch.ones(n, h * dk, dtype=F64)
    beta = torch.ones(n, h, dtype=F64)
    state = cache.view(0, {}).states["delta"]
    state[slots[2]] = 7.0
    got = []
    for lo, hi in ((0, n - 1), (n - 1, n)):
        ctx = _step(lib, cache, [slots[1]], [hi - lo])
        o = torch.empty(hi - lo, h * dv, dtype=torch.float32, device=DEV)
        lib.delta_rule(q[lo:hi].float().to(DEV).contiguous(), h, dk, h, dv, g[lo:hi].float().to(DEV).contiguous(),
                       beta[lo:hi].float().to(DEV).contiguous(), state, ctx, o)
        cache.commit([slots[1]], [hi - lo])
        got.append(o)
    last_write = max(t for t in range(n) if t % dk == 5)
    for head in range(h):
        assert torch.allclose(got[1][0, head * dv:(head + 1) * dv].cpu(), torch.full((dv,), float(last_write + 1 + head)))
    assert float((state[slots[2]] - 7.0).abs().max()) == 0.0 and float(state[slots[0]].abs().max()) == 0.0
    want, _ = P.delta_recurrence(q[:, :h * dk].view(n, h, dk), q[:, h * dk:2 * h * dk].view(n, h, dk),
                                 q[:, 2 * h * dk:].view(n, h, dv), g.view(n, h, dk), beta)
    assert _rel(torch.cat(got), want.reshape(n, h * dv)) < 1e-6


def P_REQ(h, dk, dv):
    from rbitnet_amd.parts import CacheRequest
    return CacheRequest("state", state_shape=(h, dv, dk), state_init=0.0, name="delta")      # S of a head, column by column


# ---------------------------------------------------------------------------- latent attention
def _latent_weights(hidden, h, dk, dv, qr, kr, seed):
    cfg = {"vocab": 4, "width": hidden, "streams": 1, "canon": {"taps": 1},
           "layers": [{"type": "latent_attention", "mlp": None,
                       "mixer": {"heads": h, "dim": dk, "vdim": dv, "q_rank": qr, "kv_rank": kr, "scale": 1.0}}]}
    t = P.random_bagonex_tensors(cfg, seed)
    return {k[len("l0.mix."):]: v for k, v in t.items() if k.startswith("l0.mix.")}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("h,dk,dv,qr,kr,scale", [(4, 16, 24, 40, 32, 0.25), (1, 64, 8, 16, 64, 0.1), (5, 8, 8, 24, 18, 0.6),
                                                 (2, 32, 32, 32, 128, 0.2), (3, 16, 8, 24, 320, 0.1), (2, 7, 5, 9, 33, 0.4)])
def test_latent_attention_whole_in_pieces_and_token_by_token(lib, dtype, h, dk, dv, qr, kr, scale):
    hidden, t_len = 48, 150
    params = {"heads": h, "dim": dk, "vdim": dv, "q_rank": qr, "kv_rank": kr, "scale": scale, "eps": 1e-5, "cache_from": None}
    part = build_part("mixer", PartSpec("latent_attention", params), _env(lib, hidden, dtype))
    w = _latent_weights(hidden, h, dk, dv, qr, kr, seed=h + kr)
    part.load(_place(part, w, dtype))
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want = P.latent_attention(x, P.latent_of(x, w, 1e-5), w, h, dk, dv, scale, 1e-5)
    for cuts in ([t_len], [63, 1, 1, 2, 61, 22], [100] + [1] * 50, [64, 64, 22]):
        cache = Cache([part.cache_request()], 1, 64 * 4, dtype, DEV)
        slot = cache.alloc_slot()
        outs, at = [], 0
        for n in cuts:
            ctx = _step(lib, cache, [slot], [n])
            outs.append(part.forward(x[at:at + n].to(DEV, dtype).contiguous(), ctx, cache.view(0, ctx.block_tables)))
            cache.commit([slot], [n])
            at += n
        assert _close(torch.cat(outs), want, dtype), cuts


def test_sink_and_a_far_key_show_in_the_output(lib):
    """Attention over latents with hand-made queries: one far key is given a score that stands out among hundreds, so
    the output must be that key's latent times what the sink leaves; a sink far above every score empties the output,
    one far below changes nothing; a key one position after the query is not seen."""
    h, r, n = 2, 32, 300
    cache = Cache([P_KV(r)], 1, 64 * 5, torch.float32, DEV)
    slot = cache.alloc_slot()
    ctx = _step(lib, cache, [slot], [n])
    view = cache.view(0, ctx.block_tables)
    c = torch.randn(n, r, dtype=F64) * 0.1
    far, late = 3, 129                               # a key in the first page; the key right after the query at 128
    c[far] = 0
    c[far, 0] = 4.0
    c[late] = 0
    c[late, 0] = 9.0
    proj = c.float().to(DEV).contiguous()
    lib.latent_norm_store(proj, 0, None, None, r, torch.full((r,), 1.0, device=DEV), view.k_pages, ctx, view.block_table,
                          0.0, torch.float32)
    stored = c / torch.sqrt((c * c).mean(-1, keepdim=True))
    q = torch.zeros(n, h, r, dtype=F64)
    q[:, :, 0] = 3.0
    for sinks in ([-50.0, 0.5], [80.0, -50.0]):
        out = torch.empty(n, h * r, dtype=torch.float32, device=DEV)
        lib.attention_sinks(q.float().to(DEV), view.k_pages, view.k_pages, out, ctx.tok_pos, ctx.tok_seq, view.block_table,
                            h, 1, r, 1.0, None, torch.tensor(sinks, device=DEV))
        for head in range(h):
            s = (q[:, head] @ stored.T).masked_fill(~torch.ones(n, n, dtype=torch.bool).tril(), -math.inf)
            want = P.sink_softmax(s, torch.tensor(sinks[head], dtype=F64)) @ stored
            got = out[:, head * r:(head + 1) * r].double().cpu()
            assert float((got - want).abs().max()) < 2e-5
        top = out[128, :r].double().cpu()            # head 0 at position 128: the far key wins, the late one is unseen
        if sinks[0] < 0:
            assert abs(float(top[0]) - float(stored[far, 0])) < 1e-2 * float(stored[far, 0])
        else:
            assert float(out[:, :r].abs().max()) < 1e-6


def P_KV(r):
    from rbitnet_amd.parts import CacheRequest
    return CacheRequest("kv", heads=1, head_dim=r, values=False, name="latent")


# ---------------------------------------------------------------------------- whole models
def _layer(kind, **m):
    mlp = m.pop("mlp", None)
    return {"type": kind, "mixer": m, "mlp": None if mlp is None else {"kind": "dense", "ff": mlp}}


MODEL_A = {"architecture": "Bagonex", "vocab": 70, "width": 48, "streams": 3, "norm": {"eps": 1e-5}, "canon": {"taps": 2},
           "logit_softcap": 6.0, "layers": [
               _layer("latent_attention", heads=3, dim=8, vdim=12, q_rank=20, kv_rank=24, scale=0.4, mlp=64),
               _layer("channel_delta", heads=4, kv_heads=2, dim=12, vdim=20, conv=3, mlp=None),
               _layer("latent_attention", heads=2, dim=16, vdim=8, q_rank=12, kv_rank=24, scale=0.3, kv_from=0, mlp=40),
               _layer("channel_delta", heads=2, kv_heads=2, dim=40, vdim=8, conv=2, mlp=56)]}
# one copy of the stream, one tap in front of the mixer, one head, equal sizes everywhere: what a model may happen to have
MODEL_B = {"architecture": "Bagonex", "vocab": 33, "width": 32, "streams": 1, "norm": {"eps": 1e-6}, "canon": {"taps": 1},
           "logit_softcap": 30.0, "layers": [
               _layer("channel_delta", heads=1, kv_heads=1, dim=32, vdim=32, conv=4, mlp=32),
               _layer("latent_attention", heads=1, dim=32, vdim=32, q_rank=32, kv_rank=32, scale=1.0, mlp=None)]}
# sizes that no kernel's fast path was made for: a width that is no multiple of 16, odd head counts, a latent of 80 and
# one of 128 under five heads, ranks that are no multiples of 8, four copies, the first layer an attention layer,
# two readers of one layer's latents, delta layers without a feed-forward
MODEL_C = {"architecture": "Bagonex", "vocab": 101, "width": 72, "streams": 4, "norm": {"eps": 1e-6}, "canon": {"taps": 4},
           "logit_softcap": 12.0, "layers": [
               _layer("latent_attention", heads=5, dim=24, vdim=40, q_rank=44, kv_rank=128, scale=0.2, mlp=100),
               _layer("channel_delta", heads=6, kv_heads=1, dim=48, vdim=20, conv=2, mlp=None),
               _layer("latent_attention", heads=7, dim=8, vdim=8, q_rank=20, kv_rank=128, scale=0.35, kv_from=0, mlp=None),
               _layer("latent_attention", heads=3, dim=40, vdim=12, q_rank=36, kv_rank=80, scale=0.15, mlp=44),
               _layer("channel_delta", heads=3, kv_heads=3, dim=100, vdim=36, conv=5, mlp=88),
               _layer("latent_attention", heads=2, dim=16, vdim=16, q_rank=12, kv_rank=128, scale=0.25, kv_from=0, mlp=36)]}
# widths and ranks on the matrix cores' grid, many heads on a latent of 64 (more than a decode kernel's group takes)
MODEL_D = {"architecture": "Bagonex", "vocab": 320, "width": 128, "streams": 2, "norm": {"eps": 1e-5}, "canon": {"taps": 3},
           "logit_softcap": 20.0, "layers": [
               _layer("channel_delta", heads=4, kv_heads=2, dim=64, vdim=64, conv=4, decay_rank=16, gate_rank=32, mlp=256),
               _layer("latent_attention", heads=20, dim=16, vdim=16, q_rank=64, kv_rank=64, scale=0.25, mlp=256),
               _layer("channel_delta", heads=2, kv_heads=2, dim=128, vdim=32, conv=4, decay_rank=8, gate_rank=8, mlp=None)]}
MODELS = {"A": (MODEL_A, 11), "B": (MODEL_B, 12), "C": (MODEL_C, 13), "D": (MODEL_D, 14)}
_TMP = tempfile.TemporaryDirectory(prefix="bagonex_models_")
_MADE = {}


def _model(name):
    """(folder, oracle) of a model written once per session: config.json and bfloat16 weights."""
    if name not in _MADE:
        from rbitnet_amd.weights.safetensors_io import save_file
        cfg, seed = MODELS[name]
        tensors = P.random_bagonex_tensors(cfg, seed)
        folder = os.path.join(_TMP.name, name)
        os.makedirs(folder)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(cfg, f)
        save_file(os.path.join(folder, "model.safetensors"), [(k, v.to(torch.bfloat16)) for k, v in tensors.items()])
        _MADE[name] = (folder, P.PlainBagonex(copy.deepcopy(cfg), tensors))
    return _MADE[name]


def _tokens(name, n, seed):
    g = torch.Generator().manual_seed(100 * seed + n)
    return torch.randint(0, MODELS[name][0]["vocab"], (n,), generator=g).tolist()


def _engine(name, dtype, **kw):
    import rbitnet_amd
    return rbitnet_amd.Engine.load_path(_model(name)[0], dtype=dtype, **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
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
        assert _close(torch.cat(out), want, dtype), cuts


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["C", "D"])
def test_models_of_other_shapes_as_a_batch_in_pieces(name, dtype):
    """Two requests of unequal lengths together: their prompts in two unequal pieces each (so that the second piece
    reads states and latents that the first left), then token by token; against each request's plain logits."""
    eng = _engine(name, dtype, max_tokens=64 * 8, max_batch=2)
    oracle = _model(name)[1]
    seqs = [_tokens(name, 150, 21), _tokens(name, 71, 22)]
    want = [oracle.logits(s) for s in seqs]
    slots = [eng.alloc_slot() for _ in seqs]
    got = [[], []]
    at = [0, 0]
    for pieces in ([67, 3], [62, 60]):
        logits = eng.step([(sl, s[a:a + n]) for sl, s, a, n in zip(slots, seqs, at, pieces)], "all")
        got[0].append(logits[:pieces[0]])
        got[1].append(logits[pieces[0]:])
        at = [a + n for a, n in zip(at, pieces)]
    live = [0, 1]
    while live:
        logits = eng.step([(slots[i], [seqs[i][at[i]]]) for i in live], "last")
        for row, i in enumerate(live):
            got[i].append(logits[row:row + 1])
            at[i] += 1
        for i in [i for i in live if at[i] >= len(seqs[i])]:
            eng.free_slot(slots[i])
            live.remove(i)
    for i in range(2):
        assert _close(torch.cat(got[i]), want[i], dtype), i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batches_of_unequal_requests_and_slots_used_again(dtype):
    """Four requests of 1 to 150 tokens start together and are decoded together, the short ones leaving early; then two
    new requests take the freed slots and pages.  Every request's logits are those it has alone."""
    eng = _engine("A", dtype, max_tokens=64 * 8, max_batch=4)
    oracle = _model("A")[1]
    for wave, lens in enumerate(([1, 150, 67, 30], [64, 129])):
        seqs = [_tokens("A", n + 12, 7 + wave) for n in lens]
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
            assert _close(g, want[i][:g.shape[0]], dtype), (wave, i)
        eng.cache.check()


def test_long_decoding_and_greedy_generation_through_the_engine():
    """Greedy generation of 150 tokens through `Engine.generate` (its scheduler, its captured decode step) gives the
    plain implementation's greedy tokens, for a batch of three unequal prompts; the logits of the last decode step are
    the plain ones."""
    eng = _engine("A", "float32", max_tokens=64 * 16, max_batch=5)
    oracle = _model("A")[1]
    # five requests: a captured step for five runs in the one made for six, whose sixth row is an idle sequence in the
    # cache's spare slot and page; as requests end, the steps for four, three, two and one follow
    limits = (150, 40, 90, 12, 25)
    prompts = [_tokens("A", n, 3) for n in (5, 70, 1, 33, 64)]
    results = eng.generate(prompts, max_tokens=list(limits), temperature=0.0)
    for p, r, n in zip(prompts, results, limits):
        assert len(r.tokens) == n and r.finish_reason == "length"
        seq = list(p) + r.tokens
        logits = oracle.logits(seq[:-1])
        top2 = logits[len(p) - 1:].topk(2, dim=-1)
        greedy = top2.indices[:, 0].tolist()
        clear = (top2.values[:, 0] - top2.values[:, 1]) > 1e-4           # a tie within rounding may go either way
        assert all(g == t for g, t, c in zip(greedy, r.tokens, clear.tolist()) if c)
        assert int(clear.sum()) > 0.9 * n
    assert eng.stats["decode_tokens"] > 0 and eng.model.graph_safe


def test_replay_and_command_line_on_a_model_of_this_design(tmp_path, capsys):
    """The trace replay (steps from a stream of JSON lines, logits to files) and `rbitnet generate` on model B:
    the replayed logits are the plain ones, whole and decoded, and the command line prints greedy tokens."""
    import io
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
    assert log.getvalue().split() == ["done", "0", "done", "1", "done", "2"]
    wa, wb = oracle.logits(a), oracle.logits(b)
    vocab = MODELS["B"][0]["vocab"]
    got0 = np.fromfile(tmp_path / "out" / "0.f32", dtype="<f4").reshape(-1, vocab)
    got1 = np.fromfile(tmp_path / "out" / "1.f32", dtype="<f4").reshape(-1, vocab)
    got2 = np.fromfile(tmp_path / "out" / "2.f32", dtype="<f4").reshape(-1, vocab)
    assert _close(torch.from_numpy(got0), wa[[0, 65]], "float32")
    assert _close(torch.from_numpy(got1), torch.stack([wa[66], wb[8]]), "float32")
    assert _close(torch.from_numpy(got2), wa[[69]], "float32")
    assert eng.cache.live_slots == []
    del eng
    capsys.readouterr()
    assert cli.main(["generate", "--model", folder, "--dtype", "float32", "--prompt-ids", ",".join(str(t) for t in b),
                     "--max-tokens", "5", "--temperature", "0"]) == 0
    out = capsys.readouterr().out
    rec = json.loads(out.strip().splitlines()[-1])
    assert len(rec["tokens"]) == 5 and rec["tokens"][0] == int(oracle.logits(b)[-1].argmax())
