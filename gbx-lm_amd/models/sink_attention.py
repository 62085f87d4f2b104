"""Softmax attention with a sink over ragged step batches, and the two mixers built on it.

The core (``sink_attend``): per query head, scores  s_ij = scale * <q_i, k_j>  over the keys the mask shows, weights
``p_ij = exp(s_ij) / (exp(sink_h) + sum_j exp(s_ij))``: the sink is a number per head that joins the denominator and has no value
(``sink = 0`` adds one to the denominator, no sink is the plain softmax).  The mask is causal, optionally a sliding window
(``i - j < window``) that keeps the first ``keep`` positions of a sequence visible for ever.  Optionally each head's output is
multiplied by ``sigmoid(gate[t, h])``.  Keys before the step come from a ``SlotKVCache``, the step's own keys from the step.
Scores, weights and the running sums are 32-bit whatever the activation dtype is.

Mixers:

* ``GatedSinkWindowAttention``: grouped-query attention with biases; weighted q / k norm per head before a partial rotation, unit
  values, sliding window, learned sink per head, a sigmoid output gate per channel.
* ``RotatedValueWindowAttention``: grouped-query attention; q and k are rotated (rotate-half pairs over the first ``rot_dims``
  channels, any frequency table) and then set to unit root mean square per head; values are rotated by their own position over all
  of their channels and cached so, a head's output is turned back by the query's position (so a value enters rotated by the
  distance); window with kept first tokens; sink 0.
* ``LatentAttention``: keys and values of all heads are products of one small latent row per token, ``c = norm(W_dkv h)``, plus one
  rotated key part shared by all heads; only ``c | rotated part`` is cached.  Whole prompts form every head's keys and values from
  ``c`` and attend as usual; steps with history attend over the cached rows directly: the key product is moved to the query side
  (``q' = W_uk^T q``), the value product behind the weighted sum (``o = W_uv sum_j p_j c_j``) -- one shared key/value row of
  ``kv_rank + rot_dim`` channels for all heads.  Learned sink per head, sigmoid output gate from the mixer's input.

GPU tensors run the HIP kernels of ``mixer_ops``; CPU tensors the plain torch graph below, which the kernels are tested against.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import torch
import torch.nn.functional as F
from torch import nn

from .cache import SharedLatentRows, SlotKVCache
from .rope_utils import rotary_table

NORM_NONE, NORM_UNIT, NORM_WEIGHT = 0, 1, 2


@dataclass
class HeadSegment:
    """A run of ``heads`` heads of ``head_dim`` channels inside a row, starting at ``offset``: what ``rotate_norm_heads_`` does to it.
    Channels [rot_offset, rot_offset + rot_dims) of every head are rotated (pair i with i + rot_dims / 2, or 2i with 2i + 1 when
    ``interleaved``) by ``sign * position * freq[i]``, cos and sin times ``mult``; then the head is normalised to unit root mean
    square (NORM_UNIT) or RMS-normalised with a weight per channel (NORM_WEIGHT).  ``norm_first``: the norm comes before the
    rotation (the weight then meets the channels as projected)."""
    offset: int
    heads: int
    head_dim: int
    rot_offset: int = 0
    rot_dims: int = 0
    freq: Optional[torch.Tensor] = None
    mult: float = 1.0
    sign: float = 1.0
    interleaved: bool = False
    norm: int = NORM_NONE
    weight: Optional[torch.Tensor] = None
    norm_first: bool = False


def rotate_norm_heads_(rows: torch.Tensor, positions: torch.Tensor, segments: List[HeadSegment], eps: float) -> None:
    """In place on rows [T, N]; ``positions`` int32 [T]; arithmetic in fp32."""
    if rows.is_cuda:
        from .. import mixer_ops as M
        M.rotate_norm_heads_(rows, positions, segments, eps)
        return
    t = rows.shape[0]
    pos = positions.to(torch.float32)
    for s in segments:
        seg = rows[:, s.offset:s.offset + s.heads * s.head_dim].view(t, s.heads, s.head_dim)
        v = seg.float()

        def normed(v):
            v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
            return v * s.weight.float() if s.norm == NORM_WEIGHT else v
        if s.norm != NORM_NONE and s.norm_first:
            v = normed(v)
        if s.rot_dims:
            a = s.sign * (pos[:, None] * s.freq.float()[None, :])
            cos, sin = (torch.cos(a) * s.mult)[:, None, :], (torch.sin(a) * s.mult)[:, None, :]
            part = v[..., s.rot_offset:s.rot_offset + s.rot_dims]
            if s.interleaved:
                u, w = part[..., 0::2], part[..., 1::2]
                turned = torch.stack([u * cos - w * sin, w * cos + u * sin], dim=-1).flatten(-2)
            else:
                u, w = part[..., :s.rot_dims // 2], part[..., s.rot_dims // 2:]
                turned = torch.cat([u * cos - w * sin, w * cos + u * sin], dim=-1)
            v = torch.cat([v[..., :s.rot_offset], turned, v[..., s.rot_offset + s.rot_dims:]], dim=-1)
        if s.norm != NORM_NONE and not s.norm_first:
            v = normed(v)
        seg.copy_(v.to(rows.dtype))


def _attend_one(q, k, v, pos_q, pos_k, scale, window, keep, sink, gate):
    """q [n, H, dk], k [m, G, dk], v [m, G, dv] fp32 of ONE sequence with their positions -> [n, H, dv] fp32."""
    heads, groups = q.shape[1], k.shape[1]
    rep = heads // groups
    kh = k.transpose(0, 1).repeat_interleave(rep, 0)
    vh = v.transpose(0, 1).repeat_interleave(rep, 0)
    s = torch.matmul(q.transpose(0, 1), kh.transpose(1, 2)) * scale                      # [H, n, m]
    i, j = pos_q[:, None], pos_k[None, :]
    seen = j <= i
    if window is not None:
        seen = seen & ((i - j < window) | (j < keep))
    s = s.masked_fill(~seen[None], float("-inf"))
    top = s.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink.float()[:, None, None])
    e = torch.exp(s - top)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink.float()[:, None, None] - top)
    o = torch.matmul(e / den, vh).transpose(0, 1)                                         # [n, H, dv]
    if gate is not None:
        o = o * torch.sigmoid(gate.float())[:, :, None]
    return o


def sink_attend(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor, cache: Optional[SlotKVCache], batch, scale: float,
                window: Optional[int], keep: int, sink: Optional[torch.Tensor], gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [T, H, dk], k_new [T, G, dk], v_new [T, G, dv] (views with unit inner stride), gate [T, H] or None -> [T, H * dv].
    ``cache`` (or None when no sequence of the step has history) holds the positions before the step."""
    if q.is_cuda:
        from .. import mixer_ops as M
        return M.sink_attention(q, k_new, v_new, cache, batch, scale, window, keep, sink, gate)
    t, heads, _ = q.shape
    groups, dv = v_new.shape[1], v_new.shape[2]
    out = torch.empty((t, heads * dv), dtype=q.dtype, device=q.device)
    r0 = 0
    for slot, pos0, n in zip(batch.slot, batch.pos0, batch.n_new):
        k, v = k_new[r0:r0 + n].float(), v_new[r0:r0 + n].float()
        pos_k = torch.arange(pos0, pos0 + n)
        if pos0:
            old = cache.stored(pos0)
            rows = cache.row_of(old)
            k = torch.cat([cache.keys[slot, rows, :groups * k.shape[2]].float().view(-1, groups, k.shape[2]), k])
            v = torch.cat([cache.values[slot, rows, :groups * dv].float().view(-1, groups, dv), v])
            pos_k = torch.cat([old, pos_k])
        o = _attend_one(q[r0:r0 + n].float(), k, v, torch.arange(pos0, pos0 + n), pos_k, scale, window, keep, sink,
                        None if gate is None else gate[r0:r0 + n])
        out[r0:r0 + n] = o.reshape(n, heads * dv).to(q.dtype)
        r0 += n
    return out


def head_project(x: torch.Tensor, w: torch.Tensor, n_tail: int = 0) -> torch.Tensor:
    """x [T, H, n_in + n_tail], w [H, n_in, n_out] -> [T, H, n_out + n_tail]: each head's own matrix on its first n_in channels, the
    remaining channels copied through.  Few GPU rows: one HIP launch; else a batched matrix product."""
    if x.is_cuda and x.shape[0] <= 32:
        from .. import mixer_ops as M
        return M.head_project(x, w, n_tail)
    n_in = w.shape[1]
    y = torch.bmm(x[:, :, :n_in].transpose(0, 1), w).transpose(0, 1)
    return torch.cat([y, x[:, :, n_in:]], dim=-1) if n_tail else y.contiguous()


def cache_append(cache: SlotKVCache, k_rows: torch.Tensor, v_rows: Optional[torch.Tensor], batch) -> None:
    """The step's key rows [T, k_width] (and value rows) into the table, after every query of the step has attended."""
    if k_rows.is_cuda:
        from .. import mixer_ops as M
        M.slot_append(cache, k_rows, v_rows, batch)
        return
    r0 = 0
    for slot, pos0, n in zip(batch.slot, batch.pos0, batch.n_new):
        cache.append_rows(k_rows[r0:r0 + n], None if v_rows is None else v_rows[r0:r0 + n], slot, pos0)
        r0 += n


class RotatedValueWindowAttention(nn.Module):
    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, rot_dims: int, rot_base: float,
                 rot_scaling: Optional[dict], window: Optional[int], keep_first: int, scale: float, eps: float):
        super().__init__()
        if heads % kv_heads or rot_dims % 2 or rot_dims > dim or vdim % 2:
            raise ValueError("heads must be a multiple of kv_heads; rotated channel counts are even and within the head")
        self.width, self.heads, self.kv_heads, self.dim, self.vdim = width, heads, kv_heads, dim, vdim
        self.window = None if window is None else int(window)
        self.keep_first, self.scale, self.eps = int(keep_first), float(scale), float(eps)
        self.rot_dims = int(rot_dims)
        self.nq, self.nk, self.nv = heads * dim, kv_heads * dim, kv_heads * vdim
        self.qkv = nn.Linear(width, self.nq + self.nk + self.nv, bias=False)
        self.o = nn.Linear(heads * vdim, width, bias=False)
        freq, self.rot_mult = rotary_table(rot_base, rot_dims, rot_scaling)
        self.register_buffer("freq", freq)
        self.register_buffer("vfreq", rotary_table(rot_base, vdim, None)[0])     # values: plain frequencies over all their channels
        self.register_buffer("sink", torch.zeros(heads))                          # one added to the denominator
        for p in self.parameters():
            p.requires_grad_(False)

    def make_cache(self, slots) -> SlotKVCache:
        return SlotKVCache(self.nk, self.nv, self.window, self.keep_first, slots)

    def forward(self, h: torch.Tensor, batch, cache: SlotKVCache) -> torch.Tensor:
        t = h.shape[0]
        qkv = F.linear(h, self.qkv.weight)
        pos = batch.tok[:, 1]
        rotate_norm_heads_(qkv, pos, [
            HeadSegment(0, self.heads, self.dim, 0, self.rot_dims, self.freq, self.rot_mult, norm=NORM_UNIT),
            HeadSegment(self.nq, self.kv_heads, self.dim, 0, self.rot_dims, self.freq, self.rot_mult, norm=NORM_UNIT),
            HeadSegment(self.nq + self.nk, self.kv_heads, self.vdim, 0, self.vdim, self.vfreq)], self.eps)
        cache.reserve(max(p + n for p, n in zip(batch.pos0, batch.n_new)), qkv.dtype, qkv.device)
        k_rows, v_rows = qkv[:, self.nq:self.nq + self.nk], qkv[:, self.nq + self.nk:]
        ctx = sink_attend(qkv[:, :self.nq].view(t, self.heads, self.dim), k_rows.view(t, self.kv_heads, self.dim),
                          v_rows.view(t, self.kv_heads, self.vdim), cache, batch, self.scale, self.window, self.keep_first, self.sink)
        rotate_norm_heads_(ctx, pos, [HeadSegment(0, self.heads, self.vdim, 0, self.vdim, self.vfreq, sign=-1.0)], self.eps)
        cache_append(cache, k_rows, v_rows, batch)
        return F.linear(ctx, self.o.weight)


class GatedSinkWindowAttention(nn.Module):
    """Grouped-query sliding-window attention: q | k | v (and the gate) from one projection with biases; q and k RMS-normalised per
    head with a weight per channel BEFORE the rotation; rotate-half pairs over the first ``rot_dims`` channels of a head (any
    frequency table: plain, linear, YaRN); every value head scaled to unit root mean square and cached so; scores times ``scale``;
    window ``i - j < window`` (None: all earlier keys); a learned sink per head in the softmax denominator; the concatenated heads
    times sigmoid(W_g h), channel by channel; output projection with a bias."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, rot_dims: int, rot_base: float,
                 rot_scaling: Optional[dict], window: Optional[int], scale: float, eps: float, bias: bool = True):
        super().__init__()
        if heads % kv_heads or rot_dims % 2 or rot_dims > dim:
            raise ValueError("heads must be a multiple of kv_heads; the rotated channel count is even and within the head")
        self.width, self.heads, self.kv_heads, self.dim, self.vdim = width, heads, kv_heads, dim, vdim
        self.window = None if window is None else int(window)
        self.scale, self.eps, self.rot_dims = float(scale), float(eps), int(rot_dims)
        self.nq, self.nk, self.nv, self.ng = heads * dim, kv_heads * dim, kv_heads * vdim, heads * vdim
        self.off_gate = (self.nq + self.nk + self.nv + 7) // 8 * 8
        self.inp = nn.Linear(width, (self.off_gate + self.ng + 7) // 8 * 8, bias=bias)          # q | k | v | (empty rows) | g
        self.o = nn.Linear(self.ng, width, bias=bias)
        freq, self.rot_mult = rotary_table(rot_base, rot_dims, rot_scaling) if rot_dims else (torch.zeros(0), 1.0)
        self.register_buffer("freq", freq)
        self.register_buffer("q_norm", torch.ones(dim))
        self.register_buffer("k_norm", torch.ones(dim))
        self.register_buffer("sink", torch.zeros(heads))
        for p in self.parameters():
            p.requires_grad_(False)

    def make_cache(self, slots) -> SlotKVCache:
        return SlotKVCache(self.nk, self.nv, self.window, 0, slots)

    def fuse_weights(self, q, k, v, g, qb=None, kb=None, vb=None):
        """The input projection (and its bias) from the checkpoint's matrices (all [out, in]), with the empty rows in front of the gate."""
        w = torch.zeros((self.inp.out_features, q.shape[1]), dtype=q.dtype, device=q.device)
        b = torch.zeros((self.inp.out_features,), dtype=q.dtype, device=q.device)
        for off, part, bias in ((0, q, qb), (self.nq, k, kb), (self.nq + self.nk, v, vb), (self.off_gate, g, None)):
            w[off:off + part.shape[0]] = part
            if bias is not None:
                b[off:off + part.shape[0]] = bias
        return w, b

    def forward(self, h: torch.Tensor, batch, cache: SlotKVCache) -> torch.Tensor:
        from .feed_forward import gate_mul
        t = h.shape[0]
        y = F.linear(h, self.inp.weight, self.inp.bias)
        pos = batch.tok[:, 1]
        rotate_norm_heads_(y, pos, [
            HeadSegment(0, self.heads, self.dim, 0, self.rot_dims, self.freq, self.rot_mult, norm=NORM_WEIGHT, weight=self.q_norm, norm_first=True),
            HeadSegment(self.nq, self.kv_heads, self.dim, 0, self.rot_dims, self.freq, self.rot_mult, norm=NORM_WEIGHT, weight=self.k_norm, norm_first=True),
            HeadSegment(self.nq + self.nk, self.kv_heads, self.vdim, norm=NORM_UNIT)], self.eps)
        cache.reserve(max(p + n for p, n in zip(batch.pos0, batch.n_new)), y.dtype, y.device)
        k_rows, v_rows = y[:, self.nq:self.nq + self.nk], y[:, self.nq + self.nk:self.nq + self.nk + self.nv]
        ctx = sink_attend(y[:, :self.nq].view(t, self.heads, self.dim), k_rows.view(t, self.kv_heads, self.dim),
                          v_rows.view(t, self.kv_heads, self.vdim), cache, batch, self.scale, self.window, 0, self.sink)
        cache_append(cache, k_rows, v_rows, batch)
        return F.linear(gate_mul(y[:, self.off_gate:self.off_gate + self.ng], ctx, "sigmoid"), self.o.weight, self.o.bias)


class LatentAttention(nn.Module):
    """``rot_dim = 0``: no rotated key part (attention without positions).  ``sink`` / ``gated`` False: plain softmax / no output
    gate.  ``own_latent`` False: the mixer has no latent projection of its own and attends over the rows of ANOTHER latent mixer of
    the same ``kv_rank`` (and rotated part) -- the table that mixer's cache holds and the rows it formed in this step, which its
    cache hands over (``SharedLatentRows``) -- with its own queries, key and value products."""

    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, rot_base: float,
                 rot_scaling: Optional[dict], scale: float, eps: float, sink: bool = True, gated: bool = True, own_latent: bool = True):
        super().__init__()
        if rot_dim % 2:
            raise ValueError("the rotated part has an even number of channels")
        self.width, self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank = width, heads, dim, rot_dim, vdim, kv_rank
        self.scale, self.eps = float(scale), float(eps)
        self.gated, self.own_latent = bool(gated), bool(own_latent)
        self.dk = dim + rot_dim
        self.nq, self.nl = heads * self.dk, kv_rank + rot_dim
        self.n_own = self.nl if own_latent else 0
        # q | latent, rotated key part | gate, padded with empty rows to a multiple of 8 (rows of the product start 16-byte aligned)
        self.inp = nn.Linear(width, (self.nq + self.n_own + (heads if gated else 0) + 7) // 8 * 8, bias=False)
        # rows of every head's key product, padded with rot_dim empty rows per head (the shared rotated part is written there), then
        # the value product: one matrix product forms every head's keys and values of a whole prompt
        self.up = nn.Linear(kv_rank, heads * (self.dk + vdim), bias=False)
        self.register_buffer("uk_heads", torch.zeros((heads, dim, kv_rank)))      # W_uk per head, for the query side
        self.register_buffer("uv_heads_t", torch.zeros((heads, kv_rank, vdim)))   # W_uv^T per head, behind the weighted sum
        self.o = nn.Linear(heads * vdim, width, bias=False)
        freq, self.rot_mult = rotary_table(rot_base, rot_dim, rot_scaling)
        self.register_buffer("freq", freq)
        if own_latent:
            self.register_buffer("latent_norm", torch.ones(kv_rank))
        else:
            self.latent_norm = None
        if sink:
            self.register_buffer("sink", torch.zeros(heads))
        else:
            self.sink = None
        for p in self.parameters():
            p.requires_grad_(False)

    def make_cache(self, slots, source: Optional[SlotKVCache] = None):
        if self.own_latent:
            return SlotKVCache(self.nl, 0, None, 0, slots)
        if source is None or source.k_width != self.nl or source.v_width or source.window is not None:
            raise ValueError("a latent mixer without a latent projection needs the table of one with the same row width")
        return SharedLatentRows(source)

    def fuse_weights(self, q, dkv, g, uk, uv):
        """The module's matrices from the checkpoint's (all [out, in]); ``dkv`` / ``g`` None for a mixer without them."""
        h, d, r, dv, rank = self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank
        uk_pad = torch.cat([uk.view(h, d, rank), torch.zeros((h, r, rank), dtype=uk.dtype, device=uk.device)], dim=1).reshape(h * (d + r), rank)
        parts = [q] + ([dkv] if self.own_latent else []) + ([g] if self.gated else [])
        pad = torch.zeros((self.inp.out_features - sum(p.shape[0] for p in parts), q.shape[1]), dtype=q.dtype, device=q.device)
        return {"inp.weight": torch.cat(parts + [pad]), "up.weight": torch.cat([uk_pad, uv]),
                "uk_heads": uk.view(h, d, rank).contiguous(), "uv_heads_t": uv.view(h, dv, rank).transpose(1, 2).contiguous()}

    def forward(self, h: torch.Tensor, batch, cache) -> torch.Tensor:
        t, hd, d, r, dv, rank = h.shape[0], self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank
        y = F.linear(h, self.inp.weight)
        pos = batch.tok[:, 1]
        segments = [HeadSegment(0, hd, self.dk, d, r, self.freq, self.rot_mult)] if r else []
        if self.own_latent:
            segments.append(HeadSegment(self.nq, 1, rank, norm=NORM_WEIGHT, weight=self.latent_norm))
            if r:
                segments.append(HeadSegment(self.nq + rank, 1, r, 0, r, self.freq, self.rot_mult))
        if segments:
            rotate_norm_heads_(y, pos, segments, self.eps)
        q = y[:, :self.nq].view(t, hd, self.dk)
        gate = y[:, self.nq + self.n_own:self.nq + self.n_own + hd] if self.gated else None
        if self.own_latent:
            latent = y[:, self.nq:self.nq + self.nl]                               # c | rotated key part: the cached row
            cache.reserve(max(p + n for p, n in zip(batch.pos0, batch.n_new)), y.dtype, y.device)
            table = cache
        else:
            latent, table = cache.source.step_rows, cache.source                   # the other mixer's rows of this step and its table
            if latent is None or latent.shape[0] != t:
                raise RuntimeError("the mixer that owns the latent rows has not run in this step")
        if not any(batch.pos0) and not batch.decode_only:           # (one-token steps always take the form below: a captured step
                                                                    # is replayed at later positions)
            kv = F.linear(latent[:, :rank], self.up.weight)
            keys = kv[:, :self.nq].view(t, hd, self.dk)
            if r:
                keys[:, :, d:] = latent[:, None, rank:]
            ctx = sink_attend(q, keys, kv[:, self.nq:].view(t, hd, dv), None, batch, self.scale, None, 0, self.sink, gate)
        else:
            qa = head_project(q, self.uk_heads, r)                                 # W_uk^T q | rotated part, per head
            mixed = sink_attend(qa, latent.view(t, 1, self.nl), latent[:, :rank].view(t, 1, rank), table, batch, self.scale, None, 0,
                                self.sink, gate)
            ctx = head_project(mixed.view(t, hd, rank), self.uv_heads_t).view(t, hd * dv)
        if self.own_latent:
            cache_append(cache, latent, None, batch)
            cache.step_rows = latent                                # for mixers that attend over these rows later in the step
        return F.linear(ctx, self.o.weight)
