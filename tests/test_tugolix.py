"""Tugolix through the framework (loader, state and latent caches, slot scheduler, ragged batches, generate loops) against the
plain float64 statement of the design in tests/tugolix_oracle.py.  Every scenario runs on the CPU (the modules' torch graph: cache,
slot and batching logic) and, marked gpu, on the HIP kernels of libgbx_mixers.so.  Configurations and weights are made here; sizes
differ between layers of one model and include the corners: grouped and ungrouped q / k heads, convolutions of 1 to 4 taps, head
sizes off every 16-lane grid, one stream, two, five and none, routers with and without groups, one expert per group, top 1, layers
without a feed-forward, two latent tables with readers of each."""
import json
import math
import subprocess
import sys

import pytest
import torch

import tugolix_oracle as O
from gbx_lm_amd.batching import BatchScheduler, StepBatch
from gbx_lm_amd.models import recurrent_mixers as RM
from gbx_lm_amd.models.cache import SequenceSlots, SlotStateCache
from gbx_lm_amd.models.feed_forward import GatedDenseFeedForward, glu_
from gbx_lm_amd.models.residual import StreamLayerNorm, hyper_step_
from gbx_lm_amd.models.switch_layers import DenseRoutedGLU
from gbx_lm_amd.utils import generate_step, load_model

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
# Whole models, worst row's rms difference relative to the reference row's rms.  fp32 is the sharp test; in bf16 the rounding of
# eight small layers adds up to a few per cent at the worst row (a median row: about one per cent).
TOL = {torch.float32: 3e-4, torch.bfloat16: 0.15}
SAME = {torch.float32: 2e-4, torch.bfloat16: 0.15}     # the same arithmetic through another schedule


def model_err(got, want, dtype):
    if dtype == torch.float32:
        return O.rel_err(got, want)
    return max(O.rel_err_most(got, want, 0.95), O.rel_err(got, want) / 5)

MIXED = O.make_config([
    O.delta_layer(4, 2, 24, 12, conv=4, mlp=O.dense(96)),                                  # grouped q / k heads, 4 taps, 24 key channels
    O.gla_layer(2, 20, 24, tau=8.0, mlp=O.moe(8, 3, 32, limit=1.5, groups=(4, 2), scale=2.0)),
    O.latent_layer(3, 16, 24, 40, scale=0.2, mlp=O.moe(6, 2, 24, limit=0.7, groups=None, scale=1.0)),
    O.delta_layer(2, 2, 32, 16, conv=2, mlp=None),                                          # no feed-forward
    O.latent_layer(2, 24, 8, 40, kv_from=2, mlp=O.dense(40)),                               # reads layer 2's table, not its neighbour's
    O.latent_layer(4, 8, 8, 16, mlp=None),                                                  # a second table
    O.latent_layer(1, 32, 16, 16, kv_from=5, mlp=O.moe(4, 1, 16, limit=1.0, groups=(4, 3), scale=0.5)),   # one expert per group, top 1
    O.gla_layer(3, 8, 6, tau=1.0, mlp=None),
], vocab=61, width=64, streams=3, logit_scale=0.7)
PLAIN = O.make_config([                                                                     # no streams: the plain pre-norm residual
    O.gla_layer(1, 130, 34, tau=32.0, mlp=O.dense(72)),                                     # 130 key channels: 9 per lane, 34 value channels
    O.delta_layer(6, 3, 16, 10, conv=1, mlp=O.moe(16, 4, 32, limit=2.0, groups=(2, 1), scale=1.5)),   # a convolution of one tap
    O.latent_layer(2, 64, 64, 128, mlp=None),
    O.delta_layer(1, 1, 64, 64, conv=3, mlp=O.dense(48)),
], vocab=40, width=136, eps=1e-6, streams=None)
PAIR = O.make_config([O.delta_layer(2, 1, 16, 16, conv=3, mlp=O.moe(4, 2, 16, groups=(2, 2))), O.gla_layer(2, 16, 16, tau=4.0, mlp=O.dense(32)),
                      O.latent_layer(2, 16, 16, 24, mlp=None), O.latent_layer(2, 16, 16, 24, kv_from=2, mlp=O.dense(32))],
                     vocab=33, width=32, streams=2, logit_scale=1.3)
FIVE = O.make_config([O.gla_layer(2, 16, 8, tau=2.0, mlp=O.dense(16)), O.delta_layer(2, 2, 8, 8, conv=2, mlp=None)], vocab=17, width=24, streams=5)
ONE = O.make_config([O.delta_layer(2, 2, 16, 8, conv=3, mlp=O.dense(16))], vocab=17, width=24, streams=1)


@pytest.fixture(scope="module")
def checkpoints(tmp_path_factory):
    out = {}
    for name, cfg, seed, ranks in (("mixed", MIXED, 3, (6, 5)), ("plain", PLAIN, 5, (16, 8)), ("pair", PAIR, 8, (4, 4)), ("five", FIVE, 9, (3, 2)),
                                   ("one", ONE, 10, (8, 8))):
        for steady in (False, True):                                                        # bf16 runs take the steady routers
            w = O.make_weights(cfg, seed, *ranks, steady_router=steady)
            out[name, steady] = (O.save_checkpoint(str(tmp_path_factory.mktemp(name)), cfg, w), cfg, w)
    return out


def ckpt(checkpoints, name, dtype):
    return checkpoints[name, dtype == torch.bfloat16]


_loaded, _memo = {}, {}


def model_for(checkpoints, name, device, dtype):
    key = (name, device, dtype)
    if key not in _loaded:
        _loaded[key] = load_model(ckpt(checkpoints, name, dtype)[0], device=device, dtype=dtype)[0]
    return _loaded[key]


def oracle(cfg, w, toks):
    key = (id(w), tuple(toks))
    if key not in _memo:
        _memo[key] = O.forward(cfg, w, toks)
    return _memo[key]


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def one_batch(n, device, pos0=0, slot=0):
    return StepBatch.build([slot], [pos0], [n], device)


# ------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_hyper_step_and_layer_norm(device, dtype):
    """Read, write with and without a weighted sum of candidates, mixing, layer norm or the plain read-out; rows wider than a
    thread's registers hold."""
    g = torch.Generator().manual_seed(2)
    for s, width, top in ((1, 24, 1), (3, 64, 1), (2, 40, 3), (5, 2100, 2), (8, 16, 1)):
        t, eps = 5, 1e-5
        X = torch.randn((t, s, width), generator=g) * 3 + 0.5
        y = torch.randn((t, top, width) if top > 1 else (t, width), generator=g).to(dtype)
        y_mix = torch.rand((t, top), generator=g) if top > 1 else None
        mix, write, read = torch.randn((s, s), generator=g), torch.randn(s, generator=g), torch.randn(s, generator=g)
        norm = StreamLayerNorm(width, eps)
        norm.weight, norm.bias = torch.rand(width, generator=g) + 0.5, torch.randn(width, generator=g)
        z = y.to(O.F64) if top == 1 else (y.to(O.F64) * y_mix.to(O.F64)[:, :, None]).sum(1)
        Xn = torch.einsum("ij,tiw->tjw", mix.to(O.F64), X.to(O.F64)) + write.to(O.F64)[None, :, None] * z[:, None, :]
        u = (read.to(O.F64)[None, :, None] * Xn).sum(1)
        want_h = O.layer_norm(u, norm.weight.to(O.F64), norm.bias.to(O.F64), eps)
        dev = lambda v: None if v is None else v.to(device)
        norm = norm.to(device)
        Xd = X.clone().to(device)
        h = hyper_step_(Xd, dev(y), dev(y_mix), dev(mix), dev(write), dev(read), norm, dtype)
        assert h.dtype == dtype and O.rel_err(Xd.reshape(t, -1), Xn.reshape(t, -1)) < 1e-6
        assert O.rel_err(h, want_h) < (1e-5 if dtype == torch.float32 else 1e-2)
        Xd = X.clone().to(device)                                                            # no update: read and norm only
        h0 = hyper_step_(Xd, None, None, None, None, dev(read), norm, dtype)
        u0 = (read.to(O.F64)[None, :, None] * X.to(O.F64)).sum(1)
        assert torch.equal(Xd.cpu(), X) and O.rel_err(h0, O.layer_norm(u0, norm.weight.to(O.F64).cpu(), norm.bias.to(O.F64).cpu(), eps)) < (1e-5 if dtype == torch.float32 else 1e-2)
        Xd = X.clone().to(device)                                                            # update, then the plain sum without a norm
        total = hyper_step_(Xd, dev(y), dev(y_mix), dev(mix), dev(write), None, None, dtype)
        assert total.dtype == torch.float32 and O.rel_err(total, Xn.sum(1)) < 1e-6
        assert O.rel_err(norm(total, dtype), O.layer_norm(Xn.sum(1), norm.weight.to(O.F64).cpu(), norm.bias.to(O.F64).cpu(), eps)) < (1e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_activations_and_dense_ff(device, dtype):
    g = torch.Generator().manual_seed(3)
    gu = (torch.randn((7, 2 * 37), generator=g) * 2).to(dtype)
    a, b = gu[:, :37].to(O.F64), gu[:, 37:].to(O.F64)
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    assert O.rel_err(glu_(gu.to(device), "silu"), O.silu(a) * b) < tol
    lim = 0.8
    ac, bc = a.clamp(max=lim), b.clamp(min=-lim, max=lim)
    assert O.rel_err(glu_(gu.to(device), "clamped_swish", lim), ac * O.sigmoid(1.702 * ac) * (bc + 1)) < tol
    ff = GatedDenseFeedForward(24, 40, bias=True)
    w = {"gate": torch.randn((40, 24), generator=g) / 4, "up": torch.randn((40, 24), generator=g) / 4, "down": torch.randn((24, 40), generator=g) / 4,
         "gate.b": torch.randn(40, generator=g), "up.b": torch.randn(40, generator=g), "down.b": torch.randn(24, generator=g)}
    w = {k: v.to(dtype) for k, v in w.items()}
    ff.gate_up.weight.data, ff.gate_up.bias.data = torch.cat([w["gate"], w["up"]]), torch.cat([w["gate.b"], w["up.b"]])
    ff.down.weight.data, ff.down.bias.data = w["down"], w["down.b"]
    h = torch.randn((9, 24), generator=g).to(dtype)
    want = O.dense_ff(h.to(O.F64), {k: v.to(O.F64) for k, v in w.items()}, "")
    assert O.rel_err(ff.to(device)(h.to(device)), want) < (1e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("device", DEVICES)
def test_grouped_sigmoid_router(device):
    """The choice against the oracle's, token by token: groups of several sizes, one expert per group, no groups, all choice scores
    negative (an expert outside the kept groups must lose to any negative score), and equal scores (the lower index wins)."""
    g = torch.Generator().manual_seed(4)
    for E, top, groups, scale in ((8, 3, (4, 2), 2.0), (12, 2, (3, 1), 1.0), (6, 3, None, 0.5), (4, 1, (4, 2), 1.0), (16, 6, (2, 2), 1.0), (70, 5, (7, 3), 1.0)):
        K, t = 16, 40
        m = DenseRoutedGLU(K, 8, E, top, renormalize=True, scoring="sigmoid", groups=groups, route_scale=scale, activation="clamped_swish", limit=1.0)
        m.router = torch.randn((E, K), generator=g)
        m.correction = torch.rand(E, generator=g) * 2 - 3.0                                  # every choice score below zero
        h = torch.randn((t, K), generator=g)
        h[3] = 0                                                                             # equal scores everywhere but for the correction
        m.correction[1] = m.correction[0]
        m = m.to(device)
        idx, wgt = m.route(h.to(device))
        s = O.sigmoid(h.to(O.F64) @ m.router.to(O.F64).cpu().T)
        for i in range(t):
            chosen = O.grouped_choice(s[i], m.correction.to(O.F64).cpu(), top, None if groups is None else {"count": groups[0], "keep": groups[1]})
            assert idx[i].tolist() == chosen, (E, top, groups, i)
            want = s[i][chosen] / (s[i][chosen].sum() + 1e-20) * scale
            assert torch.allclose(wgt[i].cpu().double(), want, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_routed_clamped_experts(device, dtype):
    """The routed feed-forward against the oracle, few rows (row kernels) and many (grouped matrix-core products)."""
    g = torch.Generator().manual_seed(5)
    for K, F_, E, top, groups, t in ((32, 48, 10, 3, (5, 2), 6), (64, 32, 8, 2, (2, 1), 300), (24, 20, 5, 2, None, 9)):
        spec = O.moe(E, top, F_, limit=0.9, groups=groups, scale=1.7)
        cfg = O.make_config([O.gla_layer(1, 8, 8, 2.0, mlp=spec)], width=K)
        w = {k[len("l0.mlp."):]: v for k, v in O.make_weights(cfg, 1).items() if k.startswith("l0.mlp.")}
        m = DenseRoutedGLU(K, F_, E, top, renormalize=True, scoring="sigmoid", groups=groups, route_scale=1.7, activation="clamped_swish", limit=0.9)
        m.router, m.correction = w["router"].float(), w["correction"].float()
        m.gate_up = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(E)]).to(dtype)
        m.down = torch.stack([w[f"e{e}.down"] for e in range(E)]).to(dtype)
        h = torch.randn((t, K), generator=g).to(dtype)
        y, mix = m.to(device)(h.to(device))
        got = (y.double() * mix.double()[:, :, None]).sum(1)
        want = O.moe_ff(h.to(O.F64), {k: v.to(O.F64) for k, v in w.items()}, "", spec)
        assert O.rel_err(got, want) < (2e-5 if dtype == torch.float32 else 4e-2)


def _prepared_reference(y, a, lay, bias, rate, sign, conv, unit, q_scale):
    """Rows of recurrent_prepare for ONE whole sequence, in float64, from the oracle's pieces."""
    t = y.shape[0]
    nq, nv = lay.nq, lay.nv
    parts = [y[:, lay.off_q:lay.off_q + nq], y[:, lay.off_k:lay.off_k + nq], y[:, lay.off_v:lay.off_v + nv]]
    if conv is not None:
        c0 = 0
        for i, p in enumerate(parts):
            parts[i] = O.silu(O.short_convolution(p, conv[c0:c0 + p.shape[1]]))
            c0 += p.shape[1]
    q, k, v = parts
    if unit:
        q = (q.view(t, -1, lay.dk) / torch.sqrt((q.view(t, -1, lay.dk) ** 2).sum(-1, keepdim=True) + 1e-6)).reshape(t, nq)
        k = (k.view(t, -1, lay.dk) / torch.sqrt((k.view(t, -1, lay.dk) ** 2).sum(-1, keepdim=True) + 1e-6)).reshape(t, nq)
    decay = torch.exp(-rate.repeat_interleave(lay.dk)[None] * O.softplus(sign * (a + bias)))
    out = [q * q_scale, k, v, decay]
    if lay.off_beta >= 0:
        out.append(O.sigmoid(y[:, lay.off_beta:lay.off_beta + lay.heads]))
    return torch.cat(out, dim=1)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [0, 1, 2, 3, 4])
def test_recurrent_prepare_and_tail(device, dtype, taps):
    """Convolution, silu, unit heads, decay and beta against the oracle: a whole sequence, and the same in portions down to one
    token (a portion shorter than the tail: old inputs shift, new ones join), on a slot another sequence used before."""
    g = torch.Generator().manual_seed(6 + taps)
    H, G, dk, dv, T = 4, 2, 12, 10, 23
    nq, nv = G * dk, H * dv
    lay = RM.RecurrentLayout(H, G, dk, dv, 0, nq, 2 * nq, 2 * nq + nv if taps else -1)
    width = 2 * nq + nv + H + 3
    y = (torch.randn((T, width), generator=g) * 1.5).to(dtype)
    a = (torch.randn((T, H * dk), generator=g) * 2).to(dtype)
    bias, rate = torch.randn(H * dk, generator=g), torch.rand(H, generator=g) + 0.1
    conv = (torch.randn((2 * nq + nv, taps), generator=g) * 0.7).to(dtype) if taps else None
    sign, unit, q_scale = (1.0, True, dk ** -0.5) if taps else (-1.0, False, 0.3)
    want = _prepared_reference(y.to(O.F64), a.to(O.F64), lay, bias.to(O.F64), rate.to(O.F64), sign, None if conv is None else conv.to(O.F64), unit, q_scale)
    tol = 2e-6 if dtype == torch.float32 else 1e-5                                           # fp32 arithmetic on the same rounded inputs either way
    for portions in ([T], [1, 1, 1, 2, 5, 1, 12], [3, 20]):
        slots = SequenceSlots(3)
        cache = SlotStateCache(H, dk, dv, 2 * nq + nv if taps else 0, taps, slots)
        cache.reserve(dtype, device)
        if cache.tail.numel():
            cache.tail.fill_(7.0)                                                            # what an earlier owner of the slot left behind
        pos = 0
        got = []
        for n in portions:
            batch = one_batch(n, device, pos, slot=2)
            yd, ad = y[pos:pos + n].to(device), a[pos:pos + n].to(device)
            got.append(RM.recurrent_prepare(yd, ad, lay, bias.to(device), rate.to(device), sign, None if conv is None else conv.to(device), cache,
                                            batch, unit, q_scale))
            if taps > 1:
                RM.conv_tail_update(yd, 2 * nq + nv, cache, batch)
            pos += n
        assert O.rel_err(torch.cat(got), want) < tol, portions


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("delta", [False, True])
def test_state_scan_sizes_and_schedules(device, delta):
    """The scan alone against the oracle's token loop: key channels 1 .. 256 (every register count of the kernel, sizes off the
    16-lane grid), value channels off the 4-column grid, grouped heads; whole, in portions and token by token; two sequences of
    unequal length in one step; a slot that held another sequence's state."""
    g = torch.Generator().manual_seed(7)
    for H, G, dk, dv, T in ((2, 1, 16, 8, 40), (1, 1, 1, 1, 9), (3, 3, 20, 6, 17), (2, 2, 48, 33, 30), (1, 1, 130, 5, 25), (4, 2, 96, 12, 12), (1, 1, 256, 4, 10),
                            (2, 2, 33, 7, 11), (1, 1, 180, 3, 8)):
        lay = RM.RecurrentLayout(H, G, dk, dv, 0, G * dk, 2 * G * dk, 2 * G * dk + H * dv if delta else -1)
        def rows(T):
            q, k = torch.randn((T, G * dk), generator=g), torch.randn((T, G * dk), generator=g) / math.sqrt(dk)
            v, d = torch.randn((T, H * dv), generator=g), torch.rand((T, H * dk), generator=g) * 0.3 + 0.7
            return torch.cat([q, k, v, d] + ([torch.rand((T, H), generator=g)] if delta else []), dim=1)
        def want_of(r):
            T = r.shape[0]
            q, k = r[:, :lay.nq].view(T, G, dk).to(O.F64), r[:, lay.nq:2 * lay.nq].view(T, G, dk).to(O.F64)
            v = r[:, 2 * lay.nq:2 * lay.nq + lay.nv].view(T, H, dv).to(O.F64)
            d = r[:, 2 * lay.nq + lay.nv:2 * lay.nq + lay.nv + lay.nd].view(T, H, dk).to(O.F64)
            b = r[:, 2 * lay.nq + lay.nv + lay.nd:].to(O.F64)
            rep = H // G
            return torch.stack([O.decayed_delta_scan(q[:, i // rep], k[:, i // rep], v[:, i], d[:, i], b[:, i]) if delta else
                                O.decayed_outer_scan(q[:, i // rep], k[:, i // rep], v[:, i], d[:, i]) for i in range(H)], dim=1).reshape(T, H * dv)
        r1, r2 = rows(T), rows(max(T // 3, 1))
        w1, w2 = want_of(r1), want_of(r2)
        for portions in ([T], [1] * T, [2, T - 2] if T > 2 else [T]):
            slots = SequenceSlots(4)
            cache = SlotStateCache(H, dk, dv, 0, 0, slots)
            cache.reserve(torch.float32, device)
            cache.state.fill_(3.0)                                                          # a new sequence must not see it
            pos, got1, got2 = 0, [], []
            for n in portions:
                n2 = min(n, r2.shape[0] - pos) if pos < r2.shape[0] else 0                   # the short sequence rides along while it lasts
                if n2 > 0:
                    batch = StepBatch.build([3, 1], [pos, pos], [n2, n], device)
                    out = RM.decayed_state_scan(torch.cat([r2[pos:pos + n2], r1[pos:pos + n]]).to(device), lay, cache, batch, delta)
                    got2.append(out[:n2])
                    got1.append(out[n2:])
                else:
                    got1.append(RM.decayed_state_scan(r1[pos:pos + n].to(device), lay, cache, one_batch(n, device, pos, slot=1), delta))
                pos += n
            assert O.rel_err(torch.cat(got1), w1) < 2e-5, (H, G, dk, dv, portions[:3])
            if got2:
                n2 = sum(x.shape[0] for x in got2)
                assert O.rel_err(torch.cat(got2), w2[:n2]) < 2e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("delta", [False, True])
def test_state_carries_a_far_token(device, delta):
    """One early token writes a large value under a key that no later token uses and that does not decay; 400 tokens later (whole,
    or decoded one by one after a prompt) a query with that key reads it back: a state that is lost, reset or decayed in the wrong
    channel shows at once."""
    g = torch.Generator().manual_seed(8)
    H, dk, dv, T, far = 2, 16, 8, 420, 5
    lay = RM.RecurrentLayout(H, H, dk, dv, 0, H * dk, 2 * H * dk, 2 * H * dk + H * dv if delta else -1)
    q, k = torch.randn((T, H, dk), generator=g) * 0.1, torch.randn((T, H, dk), generator=g) * 0.1
    v, d = torch.randn((T, H, dv), generator=g) * 0.1, torch.full((T, H, dk), 0.8)
    k[:, :, 0], q[:, :, 0], d[:, :, 0] = 0.0, 0.0, 1.0                                       # channel 0: nobody writes, nobody reads, no decay
    k[far, :, 0], v[far] = 1.0, torch.arange(H * dv, dtype=torch.float32).view(H, dv) + 10.0
    q[T - 1, :, 0] = 1.0
    r = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1), d.reshape(T, -1)] + ([torch.full((T, H), 0.9)] if delta else []), dim=1)
    scale = 0.9 if delta else 1.0
    for portions in ([T], [T - 40] + [1] * 40, [far + 1, T - far - 1]):
        cache = SlotStateCache(H, dk, dv, 0, 0, SequenceSlots(1))
        cache.reserve(torch.float32, device)
        pos, out = 0, None
        for n in portions:
            out = RM.decayed_state_scan(r[pos:pos + n].to(device), lay, cache, one_batch(n, device, pos), delta)
            pos += n
        last = out[-1].cpu().view(H, dv)
        assert (last - scale * v[far]).abs().max() < 0.5 and last.min() > 5.0, portions


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_head_norm_gate(device, dtype):
    g = torch.Generator().manual_seed(9)
    for H, dv in ((3, 10), (1, 130), (5, 64)):
        o, gate, w = torch.randn((6, H * dv), generator=g) * 5, torch.randn((6, H * dv + 8), generator=g).to(dtype), torch.rand(dv, generator=g) + 0.5
        x = O.rms(o.to(O.F64).view(6, H, dv), 1e-5, w.to(O.F64))
        gv = gate[:, 3:3 + H * dv]                                                          # a strided view, as a slice of a projection is
        for kind, fn in ((RM.GATE_SILU, O.silu), (RM.GATE_SIGMOID, O.sigmoid)):
            got = RM.head_norm_gate(o.to(device), gate.to(device)[:, 3:3 + H * dv], w.to(device), H, 1e-5, kind)
            assert got.dtype == dtype and O.rel_err(got, (x * fn(gv.to(O.F64)).view(6, H, dv)).reshape(6, -1)) < (1e-5 if dtype == torch.float32 else 1e-2)


# ------------------------------------------------------------------------------------------------ whole models
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "plain", "pair", "five", "one"])
def test_model_layers_against_oracle(checkpoints, device, dtype, name):
    """A whole prompt: the sum of the streams after every layer and the logits at every position."""
    path, cfg, w = ckpt(checkpoints, name, dtype)
    model = model_for(checkpoints, name, device, dtype)
    toks = tokens_for(cfg, 37, 1)
    want, layers = oracle(cfg, w, toks)
    model.trace_layers = []
    try:
        got = BatchScheduler(model).step([("a", toks)], [list(range(len(toks)))])
        for i, x in enumerate(model.trace_layers):
            assert model_err(x, layers[i], dtype) < TOL[dtype], (name, i)
    finally:
        model.trace_layers = None
    assert model_err(got, want, dtype) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "plain"])
def test_prefill_against_decoding(checkpoints, device, dtype, name):
    """A prompt and 70 single-token steps (the scheduler captures the step after two eager ones and replays it) against the oracle's
    whole sequence and against the same tokens as one prompt."""
    path, cfg, w = ckpt(checkpoints, name, dtype)
    model = model_for(checkpoints, name, device, dtype)
    toks = tokens_for(cfg, 90, 2)
    want, _ = oracle(cfg, w, toks)
    eng = BatchScheduler(model)
    rows = [eng.step([("a", toks[:20])], [list(range(20))])]
    for t in toks[20:]:
        rows.append(eng.step([("a", [t])]))
    got = torch.cat(rows)
    whole = BatchScheduler(model).step([("b", toks)], [list(range(len(toks)))])
    assert model_err(got, want, dtype) < TOL[dtype]
    assert model_err(got, whole, dtype) < SAME[dtype]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["mixed", "pair"])
@pytest.mark.parametrize("size", [2, 3, 16, 64])
def test_portions(checkpoints, device, name, size):
    """A prompt cut into portions of one size (the last one shorter), fp32: every position as in the whole prompt."""
    path, cfg, w = ckpt(checkpoints, name, torch.float32)
    model = model_for(checkpoints, name, device, torch.float32)
    toks = tokens_for(cfg, 75, 3)
    want, _ = oracle(cfg, w, toks)
    eng = BatchScheduler(model)
    got = torch.cat([eng.step([("a", toks[i:i + size])], [list(range(len(toks[i:i + size])))]) for i in range(0, len(toks), size)])
    assert O.rel_err(got, want) < TOL[torch.float32]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_unequal_batch_and_slot_reuse(checkpoints, device, dtype):
    """Requests of 1, 7, 33 and 140 tokens start together and decode together; the shortest leave first, a new request takes a freed
    slot while its neighbours decode (their state, tail and latent rows stay, the newcomer starts from zeros).  Every logit against
    the oracle and against the request alone."""
    path, cfg, w = ckpt(checkpoints, "mixed", dtype)
    model = model_for(checkpoints, "mixed", device, dtype)
    lens = {"a": 1, "b": 7, "c": 33, "d": 140, "e": 21}
    full = {k: tokens_for(cfg, n + 12, 10 + i) for i, (k, n) in enumerate(lens.items())}
    eng = BatchScheduler(model)
    got = {k: [] for k in lens}
    first = ["a", "b", "c", "d"]
    out = eng.step([(k, full[k][:lens[k]]) for k in first], [list(range(lens[k])) for k in first])
    at = 0
    for k in first:
        got[k].append(out[at:at + lens[k]])
        at += lens[k]
    live, done = list(first), {k: lens[k] for k in first}
    for step in range(16):
        if step == 2:
            eng.release("a")
            live.remove("a")
        if step == 4:                                                                        # "e" takes the slot "a" left, with a prompt of its own
            out = eng.step([("e", full["e"][:lens["e"]])], [list(range(lens["e"]))])
            got["e"].append(out)
            done["e"] = lens["e"]
            live.append("e")
        entries = [(k, [full[k][done[k]]]) for k in live if done[k] < len(full[k])]
        if not entries:
            break
        out = eng.step(entries)
        for i, (k, _) in enumerate(entries):
            got[k].append(out[i:i + 1])
            done[k] += 1
    assert eng.slot_of["e"] == 0                                                             # the freed slot was used again
    for k in lens:
        seen = torch.cat(got[k])
        want, _ = oracle(cfg, w, full[k][:seen.shape[0]])
        assert model_err(seen, want, dtype) < TOL[dtype], k
        alone = BatchScheduler(model).step([("x", full[k][:seen.shape[0]])], [list(range(seen.shape[0]))])
        assert model_err(seen, alone, dtype) < SAME[dtype], k


@pytest.mark.parametrize("device", DEVICES)
def test_slot_tables_grow_while_decoding(checkpoints, device):
    """One sequence decodes; later three more start, one by one: the state, tail and latent tables are re-allocated with more slots
    under the running sequence (and any captured decode step is dropped).  Every logit against the oracle."""
    path, cfg, w = ckpt(checkpoints, "mixed", torch.float32)
    model = model_for(checkpoints, "mixed", device, torch.float32)
    seqs = {k: tokens_for(cfg, 26, 40 + i) for i, k in enumerate("abcd")}
    eng = BatchScheduler(model)
    got = {k: [] for k in seqs}
    done = {}
    for step in range(24):
        if step % 6 == 0:
            k = "abcd"[step // 6]
            got[k].append(eng.step([(k, seqs[k][:2])], [[0, 1]]))
            done[k] = 2
        entries = [(k, [seqs[k][done[k]]]) for k in done if done[k] < 26]
        out = eng.step(entries)
        for i, (k, _) in enumerate(entries):
            got[k].append(out[i:i + 1])
            done[k] += 1
    assert len(set(eng.slot_of.values())) == 4
    for k in seqs:
        seen = torch.cat(got[k])
        assert O.rel_err(seen, oracle(cfg, w, seqs[k][:seen.shape[0]])[0]) < TOL[torch.float32], k


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_across_table_growth(checkpoints, device):
    """300 single-token steps from the first token: the latent tables double on the way (256 rows at first), the states recur 300
    times, the decode graph is dropped and captured again when the tables move."""
    path, cfg, w = ckpt(checkpoints, "pair", torch.float32)
    model = model_for(checkpoints, "pair", device, torch.float32)
    toks = tokens_for(cfg, 300, 4)
    want, _ = oracle(cfg, w, toks)
    eng = BatchScheduler(model)
    got = torch.cat([eng.step([("a", [t])]) for t in toks])
    assert O.rel_err(got, want) < 1e-4


@pytest.mark.parametrize("device", DEVICES)
def test_latent_reader_sees_far_rows(device):
    """A reader of another layer's latent table (its own key and value products) must find a row 300 tokens back: one query scores
    one old position far above the rest, whole, across the prompt / decode border and token by token, and the reader's output is
    that position's value."""
    from gbx_lm_amd.models.sink_attention import LatentAttention
    g = torch.Generator().manual_seed(11)
    width, rank, T, far = 32, 16, 330, 17
    own = LatentAttention(width, 2, 8, 0, 8, rank, 10000.0, None, 1.0, 1e-5, sink=False, gated=False, own_latent=True)
    reader = LatentAttention(width, 1, 16, 0, rank, rank, 10000.0, None, 1.0, 1e-5, sink=False, gated=False, own_latent=False)
    def set_fused(m, fused):
        for k, v in fused.items():
            if k.endswith(".weight"):
                getattr(m, k[:-len(".weight")]).weight.data = v
            else:
                setattr(m, k, v)

    wq, dkv = torch.randn((16, width), generator=g) / 6, torch.randn((rank, width), generator=g) / 6
    uk, uv, o = torch.randn((16, rank), generator=g) / 4, torch.randn((16, rank), generator=g) / 4, torch.randn((width, 16), generator=g) / 4
    set_fused(own, own.fuse_weights(wq, dkv, None, uk, uv))
    own.o.weight.data = o
    # the reader: q = the first 16 channels of its input, keys = values = the latent rows themselves, output = the weighted sum
    set_fused(reader, reader.fuse_weights(torch.eye(16, width), None, None, torch.eye(16, rank), torch.eye(rank)))
    reader.o.weight.data = torch.eye(width, rank)
    h = torch.randn((T, width), generator=g)
    latent = O.rms(h.double() @ dkv.double().T, 1e-5)                                       # the owner's rows (norm weight one)
    # the last token's query of the reader = 40 x the far row's latent: its score stands far above every other row's
    hq = torch.zeros((T, 16))
    hq[T - 1] = 40.0 * latent[far].float()
    own, reader = own.to(device), reader.to(device)
    for portions in ([T], [T - 30] + [1] * 30, [1] * 40 + [T - 40]):
        slots = SequenceSlots(1)
        slots.length[0] = 0
        c_own = own.make_cache(slots)
        c_reader = reader.make_cache(slots, c_own)
        pos, out = 0, None
        for n in portions:
            batch = one_batch(n, device, pos)
            own(h[pos:pos + n].to(device), batch, c_own)
            x = torch.zeros((n, width))
            x[:, :16] = hq[pos:pos + n]
            out = reader(x.to(device), batch, c_reader)
            pos += n
            slots.length[0] = pos
        assert (out[-1, :rank].cpu().double() - latent[far]).abs().max() < 2e-2, portions


# ------------------------------------------------------------------------------------------------ generation
@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_entry_points(checkpoints, device, tmp_path):
    """Greedy tokens through generate_step (one sequence), BatchScheduler.generate (a batch) and the command line agree with the
    oracle's own greedy loop."""
    path, cfg, w = ckpt(checkpoints, "pair", torch.float32)
    model = model_for(checkpoints, "pair", device, torch.float32)
    prompts = [tokens_for(cfg, 9, 20), tokens_for(cfg, 4, 21)]
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(8):
            seq.append(int(torch.argmax(O.forward(cfg, w, seq)[0][-1])))
        want.append(seq[len(p):])
    one = [t for t, _, _ in generate_step(torch.tensor(prompts[0]), model, max_tokens=8)]
    assert [int(t) for t in one] == want[0]
    assert BatchScheduler(model).generate(prompts, max_tokens=8) == want
    if device == "cpu":
        cmd = [sys.executable, "-m", "gbx_lm_amd.cli", "--model", path, "--dtype", "float32", "--max-tokens", "8"]
        for p in prompts:
            cmd += ["--prompt-ids", ",".join(map(str, p))]
        env = dict(__import__("os").environ, CUDA_VISIBLE_DEVICES="", HIP_VISIBLE_DEVICES="")
        out = subprocess.run(cmd, capture_output=True, text=True, check=True, env=env, cwd=__import__("os").path.dirname(__import__("os").path.dirname(__file__)))
        assert [json.loads(l)["tokens"] for l in out.stdout.strip().splitlines()] == want


@pytest.mark.parametrize("device", DEVICES)
def test_trace_replay_program(checkpoints, device, tmp_path):
    """bin/trace_run on a schedule with a ragged start, decoding, a request that ends and one that joins its slot."""
    import os
    path, cfg, w = ckpt(checkpoints, "pair", torch.float32)
    a, b, c = tokens_for(cfg, 12, 30), tokens_for(cfg, 5, 31), tokens_for(cfg, 6, 32)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:9], "want": [0, 8]}, {"id": "b", "tokens": b[:3], "want": [2]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[9:10], "want": [0]}, {"id": "b", "tokens": b[3:4], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[10:11], "want": []}, {"id": "b", "tokens": b[4:5], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "c", "tokens": c, "want": [5]}], "end": ["c"]},
             {"step": 4, "entries": [{"id": "a", "tokens": a[11:12], "want": [0]}], "end": ["a"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ)
    if device == "cpu":
        env.update(CUDA_VISIBLE_DEVICES="", HIP_VISIBLE_DEVICES="")
    out = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32", "--out", str(tmp_path), "--max-tokens", "64"],
                         input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, env=env, cwd=root)
    assert out.returncode == 0, out.stderr[-2000:]
    assert [l for l in out.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    la, lb, lc = oracle(cfg, w, a)[0], oracle(cfg, w, b)[0], oracle(cfg, w, c)[0]
    import numpy as np
    read = lambda i: torch.from_numpy(np.fromfile(os.path.join(str(tmp_path), f"{i}.f32"), dtype="<f4").reshape(-1, cfg["vocab"]).copy())
    assert O.rel_err(read(0), torch.stack([la[0], la[8], lb[2]])) < 3e-5
    assert O.rel_err(read(1), la[9:10]) < 3e-5 and O.rel_err(read(2), lb[4:5]) < 3e-5
    assert O.rel_err(read(3), lc[5:6]) < 3e-5 and O.rel_err(read(4), la[11:12]) < 3e-5
