"""Updates of the fp32 residual stream and the norms that read it.

Branch-norm form:  x <- x + mult * rms_norm(branch) * weight.  Parallel form: ``stream_add_`` / ``stream_add_norm_``.  Several
streams (``hyper_step_``): a sublayer reads a weighted sum of ``s`` streams and its output is written to all of them while a small
matrix mixes the streams among themselves.  ``StreamRMSNorm`` / ``StreamLayerNorm`` turn stream rows into sublayer inputs.
Sandwich form (a norm in front of AND behind every sublayer): ``branch_norm_add_norm_`` is the update by a normed branch together
with the next sublayer's norm, ``norm_token_shift`` the norm in front of a mixer that also reads the previous token's norm,
``normed_pair_mean`` the mean of two separately normed branches.

The stream ``x`` is fp32 whatever the activation dtype is (it is a long sum of small terms); the branch arrives in the activation
dtype, either as rows [T, W] or as ``top`` candidate rows per token [T, top, W] with fp32 mixing weights [T, top] (the routed
experts' outputs: the weighted sum is folded in here, in fp32, so it is never rounded or stored).  Returns the activation-dtype
image of the new stream, which is what the next sublayer reads.  GPU tensors: one launch (mixer_ops.residual_norm_add)."""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn


class BranchNormResidual(nn.Module):
    def __init__(self, width: int, eps: float, mult: float = 1.0):
        super().__init__()
        self.register_buffer("weight", torch.ones(width, dtype=torch.float32))
        self.eps, self.mult = float(eps), float(mult)

    def forward(self, x: torch.Tensor, branch: torch.Tensor, mix: Optional[torch.Tensor], act_dtype: torch.dtype) -> torch.Tensor:
        """Updates ``x`` (fp32 [T, W]) in place and returns its image in ``act_dtype`` (x itself when that is fp32)."""
        if x.is_cuda:
            from .. import mixer_ops as M
            return M.residual_norm_add(x, branch, mix, self.weight, self.eps, self.mult, act_dtype)
        z = branch.float()
        if mix is not None:
            z = (z * mix.float().unsqueeze(-1)).sum(1)
        x.add_(self.mult * z * torch.rsqrt(z.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight.float())
        return x if act_dtype == torch.float32 else x.to(act_dtype)


class StreamRMSNorm(nn.Module):
    """RMS norm of the fp32 stream into the activation dtype (the model's last norm)."""

    def __init__(self, width: int, eps: float):
        super().__init__()
        self.register_buffer("weight", torch.ones(width, dtype=torch.float32))
        self.eps = float(eps)

    def forward(self, x: torch.Tensor, act_dtype: torch.dtype) -> torch.Tensor:
        if x.is_cuda:
            from .. import mixer_ops as M
            return M.stream_rmsnorm(x, self.weight, self.eps, act_dtype)
        return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight.float()).to(act_dtype)


def stream_add_(x: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x += a (+ b) in fp32 on the fp32 stream: the update of a layer whose sublayers all read one norm of the stream and whose
    outputs (activation dtype) are added together.  GPU tensors: one launch."""
    if x.is_cuda:
        from .. import mixer_ops as M
        return M.stream_add_(x, a, b)
    y = a.float() if b is None else a.float() + b.float()
    return x.add_(y)


def stream_add_norm_(x: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor], norm: "StreamRMSNorm") -> torch.Tensor:
    """``stream_add_`` followed by ``norm`` of the updated stream (the next layer's input), as one launch on the GPU."""
    if x.is_cuda:
        from .. import mixer_ops as M
        return M.stream_add_norm_(x, a, b, norm.weight, norm.eps)
    return norm(stream_add_(x, a, b), a.dtype)


class StreamLayerNorm(nn.Module):
    """Layer norm with weight and bias of fp32 stream rows into the activation dtype:  (x - mean) / sqrt(var + eps) * w + b, the
    variance being the mean of the squared deviations."""

    def __init__(self, width: int, eps: float):
        super().__init__()
        self.register_buffer("weight", torch.ones(width, dtype=torch.float32))
        self.register_buffer("bias", torch.zeros(width, dtype=torch.float32))
        self.eps = float(eps)

    def forward(self, x: torch.Tensor, act_dtype: torch.dtype) -> torch.Tensor:
        return hyper_step_(x.unsqueeze(1), None, None, None, None, None, self, act_dtype)


def hyper_step_(streams: torch.Tensor, y: Optional[torch.Tensor], y_mix: Optional[torch.Tensor], mix: Optional[torch.Tensor],
                write: Optional[torch.Tensor], read: Optional[torch.Tensor], norm: Optional[StreamLayerNorm],
                act_dtype: torch.dtype) -> torch.Tensor:
    """One sublayer boundary of a model with ``s`` residual streams, ``streams`` fp32 [T, s, W] (updated in place), as one launch:

    1. if ``y`` is given (the sublayer's output, activation dtype, [T, W] -- or [T, top, W] with fp32 ``y_mix`` [T, top], whose
       weighted sum is folded in here in fp32):  X_j <- sum_i mix[i, j] X_i + write[j] * y  for all j at once from the old streams;
    2. u = sum_i read[i] X_i   (``read`` None: the plain sum of the streams);
    3. returns ``norm(u)`` in ``act_dtype``, or u itself (fp32) when ``norm`` is None."""
    if streams.is_cuda:
        from .. import mixer_ops as M
        return M.hyper_step_(streams, y, y_mix, mix, write, read, norm, act_dtype)
    if y is not None:
        z = y.float()
        if y_mix is not None:
            z = (z * y_mix.float().unsqueeze(-1)).sum(1)
        streams.copy_(torch.einsum("ij,tiw->tjw", mix.float(), streams) + write.float()[None, :, None] * z[:, None, :])
    u = streams.sum(1) if read is None else (streams * read.float()[None, :, None]).sum(1)
    if norm is None:
        return u
    mean = u.mean(-1, keepdim=True)
    var = (u - mean).pow(2).mean(-1, keepdim=True)
    return ((u - mean) * torch.rsqrt(var + norm.eps) * norm.weight.float() + norm.bias.float()).to(act_dtype)


def norm_token_shift(x: torch.Tensor, weight: torch.Tensor, eps: float, shift: torch.Tensor, cache, batch, act_dtype: torch.dtype) -> torch.Tensor:
    """RMS norm of fp32 stream rows followed by a token shift, as one launch on the GPU:

        n_t = x_t / sqrt(mean(x_t^2) + eps) * weight,      h_t = n_t + (n_(t-1) - n_t) * shift     (n_(-1) = 0)

    ``n_(t-1)`` of a step's first row comes from ``cache`` (a ``SlotRowCache`` of fp32 rows: the norm of the sequence's last token,
    which this call leaves there for the next step).  Everything in fp32; returns h in ``act_dtype``."""
    cache.reserve(act_dtype, x.device)
    if x.is_cuda:
        from .. import mixer_ops as M
        return M.norm_token_shift(x, weight, eps, shift, cache.rows, batch, act_dtype)
    n = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    prev = torch.empty_like(n)
    r0 = 0
    for slot, pos0, cnt in zip(batch.slot, batch.pos0, batch.n_new):
        prev[r0] = cache.rows[slot] if pos0 else 0.0
        prev[r0 + 1:r0 + cnt] = n[r0:r0 + cnt - 1]
        cache.rows[slot] = n[r0 + cnt - 1]
        r0 += cnt
    return (n + (prev - n) * shift.float()).to(act_dtype)


def branch_norm_add_norm_(x: torch.Tensor, branch: torch.Tensor, mix: Optional[torch.Tensor], extra: Optional[torch.Tensor], weight: torch.Tensor,
                          eps: float, next_weight: Optional[torch.Tensor], act_dtype: torch.dtype) -> Optional[torch.Tensor]:
    """x += rms_norm(z) * weight in place on the fp32 stream, z = branch [T, W] -- or sum_k mix[t, k] branch[t, k] for candidate rows
    [T, top, W] with fp32 weights [T, top] -- plus ``extra`` [T, W] if given (a branch every token takes, e.g. a shared expert); then,
    with ``next_weight``, returns rms_norm(x) * next_weight in ``act_dtype`` (the next sublayer's input): one launch on the GPU."""
    if x.is_cuda:
        from .. import mixer_ops as M
        return M.branch_norm_add_norm_(x, branch, mix, extra, weight, eps, next_weight, act_dtype)
    z = branch.float()
    if mix is not None:
        z = (z * mix.float().unsqueeze(-1)).sum(1)
    if extra is not None:
        z = z + extra.float()
    x.add_(z * torch.rsqrt(z.pow(2).mean(-1, keepdim=True) + eps) * weight.float())
    if next_weight is None:
        return None
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * next_weight.float()).to(act_dtype)


def normed_pair_mean(a: torch.Tensor, b: torch.Tensor, wa: torch.Tensor, wb: torch.Tensor, eps: float) -> torch.Tensor:
    """(rms_norm(a) * wa + rms_norm(b) * wb) / 2 over rows [T, W] in fp32, result in the rows' dtype: the output of two mixers that
    run side by side."""
    if a.is_cuda:
        from .. import mixer_ops as M
        return M.normed_pair_mean(a, b, wa, wb, eps)
    fa, fb = a.float(), b.float()
    na = fa * torch.rsqrt(fa.pow(2).mean(-1, keepdim=True) + eps) * wa.float()
    nb = fb * torch.rsqrt(fb.pow(2).mean(-1, keepdim=True) + eps) * wb.float()
    return (0.5 * (na + nb)).to(a.dtype)
