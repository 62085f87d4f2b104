"""A recurrent block around a real-gated linear recurrent unit, over ragged step batches.

Two branches of ``lru_width`` channels read the block's input h:  y = gelu_tanh(W_y h + b_y)  and  x = W_x h + b_x.  x passes a short
causal convolution over time per channel (``taps`` taps, the last one the current token's, zeros before the sequence, plus a bias,
no activation): u.  The channels form ``blocks`` equal parts; in part b two gates come from square matrices of the part's size,

    r = sigmoid(A_b u_b + a_b),   i = sigmoid(I_b u_b + i_b),

and the unit itself is a diagonal recurrence per channel c, from S = 0 at a sequence's first token (which is no special case):

    log a = -rate * r * softplus(lam_c),   a = exp(log a),   S <- a S + sqrt(1 - a^2) * (i * u).

The block's output is W_o (S * y).  ``rate`` is 8 in the published unit and a parameter here.  State of a sequence: S (fp32, one
value per channel) and the last ``taps - 1`` inputs of the convolution; both live in a ``SlotStateCache`` (the vector state is the
``dk = 1`` case of its per-head matrices).  Gates, decay, softplus, exponential, square root and the state are fp32; the two gate
products accumulate in fp32 from the fp32 convolution output.

GPU tensors: the convolution, the gate products (block-diagonal, one launch for both gates) and the scan (decay arithmetic in
parallel over a chunk of tokens, then the recurrence, then the gelu branch and the product) are HIP launches of ``mixer_ops``; CPU
tensors take the plain torch graph below.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn

from .cache import SlotStateCache
from .recurrent_mixers import conv_tail_update


def causal_conv_rows(x: torch.Tensor, conv: torch.Tensor, bias: Optional[torch.Tensor], cache: SlotStateCache, batch) -> torch.Tensor:
    """x [T, C] rows of a step (activation dtype, unit inner stride), conv [C, taps] (last tap = current token), bias [C] or None
    -> fp32 [T, C].  Inputs before the step come from ``cache.tail`` (oldest first), zeros before the sequence."""
    if x.is_cuda:
        from .. import mixer_ops as M
        return M.causal_conv_rows(x, conv, bias, cache, batch)
    taps, c = conv.shape[1], x.shape[1]
    out = torch.empty((x.shape[0], c), dtype=torch.float32)
    r0 = 0
    for slot, pos0, n in zip(batch.slot, batch.pos0, batch.n_new):
        before = cache.tail[slot].float() if (pos0 and taps > 1) else torch.zeros((taps - 1, c))
        if 0 < pos0 < taps - 1:
            before = before.clone()
            before[:taps - 1 - pos0] = 0
        ext = torch.cat([before, x[r0:r0 + n].float()])
        acc = torch.zeros((n, c))
        for j in range(taps):
            acc += ext[j:j + n] * conv[:, j].float()
        out[r0:r0 + n] = acc if bias is None else acc + bias.float()
        r0 += n
    return out


def block_gate_logits(u: torch.Tensor, w: torch.Tensor, b: torch.Tensor, w_t_f32: Optional[torch.Tensor] = None) -> torch.Tensor:
    """u fp32 [T, C], w [blocks, 2 * bs, bs] (rows: the recurrence gate's matrix over the input gate's, each [out, in]; activation
    dtype), b fp32 [blocks, 2 * bs] -> fp32 logits [T, blocks, 2 * bs]; products and sums in fp32.  ``w_t_f32`` [blocks, bs, 2 * bs]:
    the fp32 image of w transposed, which prompt-sized GPU steps multiply with (a batched vendor product)."""
    if u.is_cuda:
        from .. import mixer_ops as M
        return M.block_gate_logits(u, w, b, w_t_f32)
    blocks, two_bs, bs = w.shape
    ub = u.view(u.shape[0], blocks, bs)
    return torch.einsum("tbi,boi->tbo", ub, w.float()) + b.float()[None]


def gated_lru_scan(u: torch.Tensor, logits: torch.Tensor, lam_sp: torch.Tensor, y: torch.Tensor, rate: float, cache: SlotStateCache, batch) -> torch.Tensor:
    """u fp32 [T, C]; logits fp32 [T, blocks, 2 * bs] (recurrence gate | input gate per block); lam_sp fp32 [C] = softplus(lam);
    y [T, C] rows (activation dtype, unit inner stride): the other branch BEFORE its gelu.  Runs every sequence from the state its
    slot holds (zeros at position 0), leaves the new state there, returns S * gelu_tanh(y) in y's dtype."""
    if u.is_cuda:
        from .. import mixer_ops as M
        return M.gated_lru_scan(u, logits, lam_sp, y, rate, cache, batch)
    t, c = u.shape
    blocks, bs = logits.shape[1], logits.shape[2] // 2
    r = torch.sigmoid(logits[:, :, :bs]).reshape(t, c)
    i = torch.sigmoid(logits[:, :, bs:]).reshape(t, c)
    a = torch.exp(-rate * r * lam_sp.float()[None])
    inp = torch.sqrt(1.0 - a * a) * (i * u)
    s_all = torch.empty_like(u)
    state = cache.state.view(cache.state.shape[0], c)
    r0 = 0
    for slot, pos0, n in zip(batch.slot, batch.pos0, batch.n_new):
        s = state[slot].clone() if pos0 else torch.zeros(c)
        for j in range(r0, r0 + n):
            s = a[j] * s + inp[j]
            s_all[j] = s
        state[slot] = s
        r0 += n
    yf = y.float()
    g = 0.5 * yf * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (yf + 0.044715 * yf.pow(3))))
    return (s_all * g).to(y.dtype)


class GatedLRUBlock(nn.Module):
    def __init__(self, width: int, lru_width: int, blocks: int, taps: int, rate: float = 8.0):
        super().__init__()
        if lru_width % blocks or taps < 1:
            raise ValueError("GatedLRUBlock: equal blocks, at least one tap")
        self.width, self.lru_width, self.blocks, self.taps, self.rate = width, lru_width, blocks, int(taps), float(rate)
        bs = lru_width // blocks
        self.inp = nn.Linear(width, 2 * lru_width, bias=True)                               # x | y
        self.o = nn.Linear(lru_width, width, bias=False)
        self.register_buffer("conv", torch.zeros((lru_width, self.taps)))                  # activation dtype
        self.register_buffer("conv_bias", torch.zeros(lru_width, dtype=torch.float32))
        self.register_buffer("gates", torch.zeros((blocks, 2 * bs, bs)))                   # activation dtype
        self.register_buffer("gates_bias", torch.zeros((blocks, 2 * bs), dtype=torch.float32))
        self.register_buffer("lam_sp", torch.zeros(lru_width, dtype=torch.float32))        # softplus(lam), formed once in fp32
        self._gates_t = None                                                               # fp32 transposed image, formed at the first long GPU step
        for p in self.parameters():
            p.requires_grad_(False)

    def _gates_f32_t(self) -> torch.Tensor:
        g = self.gates
        if self._gates_t is None or self._gates_t.device != g.device or self._gates_src != (g.data_ptr(), g._version):
            self._gates_t, self._gates_src = g.float().transpose(1, 2).contiguous(), (g.data_ptr(), g._version)
        return self._gates_t

    def make_cache(self, slots) -> SlotStateCache:
        return SlotStateCache(1, 1, self.lru_width, self.lru_width, self.taps, slots)

    def forward(self, h: torch.Tensor, batch, cache: SlotStateCache) -> torch.Tensor:
        c = self.lru_width
        xy = F.linear(h, self.inp.weight, self.inp.bias)
        cache.reserve(xy.dtype, xy.device)
        u = causal_conv_rows(xy[:, :c], self.conv, self.conv_bias, cache, batch)
        if self.taps > 1:
            conv_tail_update(xy, c, cache, batch)
        logits = block_gate_logits(u, self.gates, self.gates_bias, self._gates_f32_t() if (u.is_cuda and u.shape[0] > 16) else None)
        return F.linear(gated_lru_scan(u, logits, self.lam_sp, xy[:, c:], self.rate, cache, batch), self.o.weight)
