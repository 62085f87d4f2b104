"""Recurrent sequence mixers over ragged step batches: a matrix-valued state per head that every token decays and writes to.

The core (``decayed_state_scan``), per head with key channels ``i`` and value channels ``j``, state ``S [dk, dv]`` (fp32, zero at a
sequence's first token, carried in a ``SlotStateCache``), per token ``t`` with decay ``g_t [dk]`` in (0, 1]:

    S <- diag(g_t) S                                   (every key channel has its own decay)
    plain:  S <- S + k_t v_t^T
    delta:  u = beta_t (v_t - S^T k_t),  S <- S + k_t u^T       (the write replaces what the state holds under k_t)
    o_t = S^T q_t                                      (the read-out sees the token's own write)

Everything that enters it is prepared in fp32 by ONE row launch (``recurrent_prepare``): optionally a short causal convolution over
time per channel followed by silu on q | k | v (its last ``taps - 1`` inputs per sequence are part of the cache), optionally q and k
scaled to unit length per head, q times a constant, the decay  g = exp(-rate_h * softplus(sign * (a + bias)))  -- which is
``sigmoid(a + bias)^(1/tau)`` for ``sign = -1, rate = 1/tau`` and ``exp(-exp(A_h) softplus(a + bias))`` for ``sign = +1, rate =
exp(A_h)`` -- and ``beta = sigmoid(b)``.  After the scan each head's read-out is RMS-normalised over its value channels, weighted
and gated (``head_norm_gate``: silu or sigmoid gate).

Mixers: ``GatedLinearAttention`` (plain write, decay from a low-rank projection, silu output gate), ``LightningAttention`` (plain
write, silu on q / k / v, a constant decay per head, all heads normalised together, sigmoid gate) and ``ChannelDeltaRule`` (delta
write with grouped q / k heads, convolution, unit q / k, low-rank decay and low-rank sigmoid gate).

GPU tensors run the HIP kernels of ``mixer_ops``; CPU tensors the plain torch graph below, which the kernels are tested against.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn

from .cache import SlotStateCache

GATE_SILU, GATE_SIGMOID = 1, 2


@dataclass
class RecurrentLayout:
    """Where a row of the input projection holds what ``recurrent_prepare`` reads (channel offsets), and the head geometry."""
    heads: int            # value / state heads
    groups: int           # q / k heads (a state head h reads group h // (heads // groups))
    dk: int
    dv: int
    off_q: int
    off_k: int
    off_v: int
    off_beta: int = -1    # one channel per head, or -1: no beta (plain write)

    @property
    def nq(self) -> int: return self.groups * self.dk
    @property
    def nv(self) -> int: return self.heads * self.dv
    @property
    def nd(self) -> int: return self.heads * self.dk
    @property
    def out_width(self) -> int: return 2 * self.nq + self.nv + self.nd + (self.heads if self.off_beta >= 0 else 0)


def recurrent_prepare(y: torch.Tensor, a: Optional[torch.Tensor], lay: RecurrentLayout, decay_bias: Optional[torch.Tensor], decay_rate: torch.Tensor,
                      sign: float, conv: Optional[torch.Tensor], cache: SlotStateCache, batch, unit: bool, q_scale: float,
                      qkv_silu: bool = False) -> torch.Tensor:
    """y [T, N] projection rows, a [T, heads * dk] decay projection rows (both activation dtype, unit inner stride) -> fp32
    [T, q | k | v | decay | beta].  ``conv`` [nq + nq + nv, taps] or None (then q | k | v must be adjacent from ``off_q`` on).
    ``a`` None: no decay projection, every key channel of head h decays by the constant ``decay_rate[h]`` itself.  ``qkv_silu``
    (without a convolution): q, k and v pass silu."""
    if y.is_cuda:
        from .. import mixer_ops as M
        return M.recurrent_prepare(y, a, lay, decay_bias, decay_rate, sign, conv, cache, batch, unit, q_scale, qkv_silu)
    t = y.shape[0]
    nq, nv = lay.nq, lay.nv
    q, k, v = y[:, lay.off_q:lay.off_q + nq].float(), y[:, lay.off_k:lay.off_k + nq].float(), y[:, lay.off_v:lay.off_v + nv].float()
    if qkv_silu and conv is None:
        q, k, v = F.silu(q), F.silu(k), F.silu(v)
    if conv is not None:
        taps = conv.shape[1]
        raw = torch.cat([q, k, v], dim=1)
        out = torch.empty_like(raw)
        r0 = 0
        for slot, pos0, n in zip(batch.slot, batch.pos0, batch.n_new):
            before = cache.tail[slot].float() if pos0 else torch.zeros((taps - 1, raw.shape[1]))
            if 0 < pos0 < taps - 1:                                   # rows of the tail older than the sequence are not its own
                before = before.clone()
                before[:taps - 1 - pos0] = 0
            ext = torch.cat([before, raw[r0:r0 + n]])                 # [taps - 1 + n, C]
            acc = torch.zeros((n, raw.shape[1]))
            for j in range(taps):
                acc += ext[j:j + n] * conv[:, j].float()
            out[r0:r0 + n] = F.silu(acc)
            r0 += n
        q, k, v = out[:, :nq], out[:, nq:2 * nq], out[:, 2 * nq:]
    if unit:
        q = q.view(t, lay.groups, lay.dk)
        k = k.view(t, lay.groups, lay.dk)
        q = (q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6)).reshape(t, nq)
        k = (k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)).reshape(t, nq)
    if a is None:
        decay = decay_rate.float().repeat_interleave(lay.dk)[None, :].expand(t, lay.nd)
    else:
        z = sign * (a.float() + decay_bias.float())
        decay = torch.exp(-decay_rate.float().repeat_interleave(lay.dk)[None, :] * F.softplus(z))
    parts = [q * q_scale, k, v, decay]
    if lay.off_beta >= 0:
        parts.append(torch.sigmoid(y[:, lay.off_beta:lay.off_beta + lay.heads].float()))
    return torch.cat(parts, dim=1)


def conv_tail_update(y: torch.Tensor, channels: int, cache: SlotStateCache, batch) -> None:
    """The last ``taps - 1`` convolution inputs of every sequence of the step (channels [0, channels) of ``y``) into the cache."""
    if y.is_cuda:
        from .. import mixer_ops as M
        M.conv_tail_update(y, channels, cache, batch)
        return
    keep = cache.taps - 1
    r0 = 0
    for slot, pos0, n in zip(batch.slot, batch.pos0, batch.n_new):
        old = cache.tail[slot] if pos0 else torch.zeros_like(cache.tail[slot])
        cache.tail[slot] = torch.cat([old, y[r0:r0 + n, :channels].to(old.dtype)])[-keep:] if keep else old
        r0 += n


def decayed_state_scan(r: torch.Tensor, lay: RecurrentLayout, cache: SlotStateCache, batch, delta: bool) -> torch.Tensor:
    """r: rows of ``recurrent_prepare``.  Runs every sequence of the step over its new tokens from the state its slot holds (zeros
    for a sequence at position 0), leaves the new state there and returns the read-outs fp32 [T, heads * dv]."""
    if r.is_cuda:
        from .. import mixer_ops as M
        return M.decayed_state_scan(r, lay, cache, batch, delta)
    t = r.shape[0]
    h, g, dk, dv, nq = lay.heads, lay.groups, lay.dk, lay.dv, lay.nq
    rep = h // g
    q = r[:, :nq].view(t, g, dk).repeat_interleave(rep, 1)
    k = r[:, nq:2 * nq].view(t, g, dk).repeat_interleave(rep, 1)
    v = r[:, 2 * nq:2 * nq + lay.nv].view(t, h, dv)
    decay = r[:, 2 * nq + lay.nv:2 * nq + lay.nv + lay.nd].view(t, h, dk)
    beta = r[:, 2 * nq + lay.nv + lay.nd:].view(t, h) if delta else None
    out = torch.empty((t, h, dv), dtype=torch.float32)
    r0 = 0
    for slot, pos0, n in zip(batch.slot, batch.pos0, batch.n_new):
        s = cache.state[slot].transpose(1, 2).clone() if pos0 else torch.zeros((h, dk, dv))       # [H, dk, dv]
        for i in range(r0, r0 + n):
            s = s * decay[i][:, :, None]
            u = v[i]
            if delta:
                u = beta[i][:, None] * (v[i] - torch.einsum("hkv,hk->hv", s, k[i]))
            s = s + k[i][:, :, None] * u[:, None, :]
            out[i] = torch.einsum("hkv,hk->hv", s, q[i])
        cache.state[slot] = s.transpose(1, 2)
        r0 += n
    return out.view(t, h * dv)


def head_norm_gate(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, heads: int, eps: float, kind: int) -> torch.Tensor:
    """o fp32 [T, heads * dv], gate [T, heads * dv] (activation dtype, unit inner stride), weight fp32 [dv] ->
    rms_norm_per_head(o) * weight * (silu | sigmoid)(gate) in the gate's dtype."""
    if o.is_cuda:
        from .. import mixer_ops as M
        return M.head_norm_gate(o, gate, weight, heads, eps, kind)
    t = o.shape[0]
    x = o.view(t, heads, -1)
    x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    g = gate.float().reshape(t, heads, -1)
    g = F.silu(g) if kind == GATE_SILU else torch.sigmoid(g)
    return (x * g).reshape(t, -1).to(gate.dtype)


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


class _RecurrentMixer(nn.Module):
    """Shared by the mixers: the cache and the order of launches of a step."""
    delta = False
    unit = False
    gate_kind = GATE_SILU
    qkv_silu = False
    norm_heads_together = False        # the read-outs of all heads are RMS-normalised as ONE vector (weight over heads * dv)

    def make_cache(self, slots) -> SlotStateCache:
        lay = self.layout
        return SlotStateCache(lay.heads, lay.dk, lay.dv, (2 * lay.nq + lay.nv) if self.taps else 0, self.taps, slots)

    def _mix(self, y: torch.Tensor, a: torch.Tensor, gate: torch.Tensor, batch, cache: SlotStateCache) -> torch.Tensor:
        lay = self.layout
        cache.reserve(y.dtype, y.device)
        r = recurrent_prepare(y, a, lay, self.decay_bias, self.decay_rate, self.decay_sign, self.conv if self.taps else None, cache, batch,
                              self.unit, self.q_scale, self.qkv_silu)
        if self.taps > 1:
            conv_tail_update(y, 2 * lay.nq + lay.nv, cache, batch)
        o = decayed_state_scan(r, lay, cache, batch, self.delta)
        return F.linear(head_norm_gate(o, gate, self.out_norm, 1 if self.norm_heads_together else lay.heads, self.eps, self.gate_kind), self.o.weight)


class GatedLinearAttention(_RecurrentMixer):
    """q = W_q h / sqrt(dk), k = W_k h, v = W_v h per head; decay  sigmoid(W_a2 (W_a1 h) + bias)^(1/tau)  per head and key channel;
    plain write; read-out RMS-normalised per head (shared weight over the value channels), times silu(W_g h); then W_o."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay_rank: int, tau: float, eps: float):
        super().__init__()
        self.width, self.eps, self.taps = width, float(eps), 0
        nq, nv = heads * dim, heads * vdim
        self.layout = RecurrentLayout(heads, heads, dim, vdim, 0, nq, 2 * nq)
        self.off_gate, self.off_a1, self.decay_rank = 2 * nq + nv, 2 * nq + 2 * nv, decay_rank
        self.inp = nn.Linear(width, _pad8(self.off_a1 + decay_rank), bias=False)          # q | k | v | g | a1 (padded with empty rows)
        self.a2 = nn.Linear(decay_rank, heads * dim, bias=False)
        self.o = nn.Linear(nv, width, bias=False)
        self.register_buffer("decay_bias", torch.zeros(heads * dim))
        self.register_buffer("decay_rate", torch.full((heads,), 1.0 / float(tau)))
        self.register_buffer("out_norm", torch.ones(vdim))
        self.decay_sign, self.q_scale = -1.0, dim ** -0.5
        for p in self.parameters():
            p.requires_grad_(False)

    def forward(self, h: torch.Tensor, batch, cache: SlotStateCache) -> torch.Tensor:
        y = F.linear(h, self.inp.weight)
        a = F.linear(y[:, self.off_a1:self.off_a1 + self.decay_rank], self.a2.weight)
        return self._mix(y, a, y[:, self.off_gate:self.off_gate + self.layout.nv], batch, cache)


class LightningAttention(_RecurrentMixer):
    """q = silu(W_q h), k = silu(W_k h), v = silu(W_v h) per head; every key channel of head h decays by the constant ``decay[h]``;
    plain write, no scale; the read-outs of all heads are RMS-normalised together (one weight over heads * vdim), times
    sigmoid(W_g h); then W_o."""
    gate_kind = GATE_SIGMOID
    qkv_silu = True
    norm_heads_together = True

    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay, eps: float):
        super().__init__()
        if len(decay) != heads:
            raise ValueError("LightningAttention: one decay per head")
        self.width, self.eps, self.taps = width, float(eps), 0
        nq, nv = heads * dim, heads * vdim
        self.layout = RecurrentLayout(heads, heads, dim, vdim, 0, nq, 2 * nq)
        self.off_gate = 2 * nq + nv
        self.inp = nn.Linear(width, _pad8(self.off_gate + nv), bias=False)                # q | k | v | g
        self.o = nn.Linear(nv, width, bias=False)
        self.decay_bias = None
        self.register_buffer("decay_rate", torch.tensor([float(d) for d in decay], dtype=torch.float64).to(torch.float32))
        self.register_buffer("out_norm", torch.ones(nv))
        self.decay_sign, self.q_scale = 0.0, 1.0
        for p in self.parameters():
            p.requires_grad_(False)

    def forward(self, h: torch.Tensor, batch, cache: SlotStateCache) -> torch.Tensor:
        y = F.linear(h, self.inp.weight)
        return self._mix(y, None, y[:, self.off_gate:self.off_gate + self.layout.nv], batch, cache)


class ChannelDeltaRule(_RecurrentMixer):
    """Grouped q / k heads (``kv_heads``) and ``heads`` value heads; q | k | v pass a short causal convolution over time per channel
    and silu; q, k unit vectors per head (q also / sqrt(dk)); beta = sigmoid(W_b h) per head; decay per head and key channel
    exp(-exp(A_h) softplus(W_a2 (W_a1 h) + dt_bias)); delta write; read-out RMS-normalised per head (shared weight), times
    sigmoid(W_g2 (W_g1 h)); then W_o."""
    delta = True
    unit = True
    gate_kind = GATE_SIGMOID

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int, decay_rank: int, gate_rank: int, eps: float):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.width, self.eps, self.taps = width, float(eps), int(taps)
        nq, nv = kv_heads * dim, heads * vdim
        self.off_a1, self.decay_rank = _pad8(2 * nq + nv + heads), decay_rank
        self.off_g1, self.gate_rank = _pad8(self.off_a1 + decay_rank), gate_rank
        self.layout = RecurrentLayout(heads, kv_heads, dim, vdim, 0, nq, 2 * nq, 2 * nq + nv)
        # q | k | v | b | a1 | g1, the low-rank parts starting at multiples of 8 rows (their rows are the inputs of further products)
        self.inp = nn.Linear(width, _pad8(self.off_g1 + gate_rank), bias=False)
        self.a2 = nn.Linear(decay_rank, heads * dim, bias=False)
        self.g2 = nn.Linear(gate_rank, nv, bias=False)
        self.o = nn.Linear(nv, width, bias=False)
        self.register_buffer("conv", torch.zeros((2 * nq + nv, max(self.taps, 1))))          # activation dtype (a matrix like the projections)
        self.register_buffer("decay_bias", torch.zeros(heads * dim))
        self.register_buffer("decay_rate", torch.ones(heads))                             # exp(A_log), formed in 32-bit at load time
        self.register_buffer("out_norm", torch.ones(vdim))
        self.decay_sign, self.q_scale = 1.0, dim ** -0.5
        for p in self.parameters():
            p.requires_grad_(False)

    def fuse_weights(self, q, k, v, b, a1, g1):
        """The input projection from the checkpoint's matrices (all [out, in]), with the empty rows between the parts."""
        w = torch.zeros((self.inp.out_features, q.shape[1]), dtype=q.dtype, device=q.device)
        lay = self.layout
        for off, part in ((0, q), (lay.off_k, k), (lay.off_v, v), (lay.off_beta, b), (self.off_a1, a1), (self.off_g1, g1)):
            w[off:off + part.shape[0]] = part
        return w

    def forward(self, h: torch.Tensor, batch, cache: SlotStateCache) -> torch.Tensor:
        y = F.linear(h, self.inp.weight)
        a = F.linear(y[:, self.off_a1:self.off_a1 + self.decay_rank], self.a2.weight)
        gate = F.linear(y[:, self.off_g1:self.off_g1 + self.gate_rank], self.g2.weight)
        return self._mix(y, a, gate, batch, cache)
