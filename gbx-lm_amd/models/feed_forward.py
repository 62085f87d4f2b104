"""Dense feed-forwards of ragged-step models: ``down(act(up h))`` and the gated ``down(act(gate h) * (up h))``, activations as
parameters.

``relu2``: the square of relu; ``gelu_tanh``: 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).  The two products are plain
matrix products (vendor library); the activation is one in-place HIP launch on GPU tensors (fp32 arithmetic, result in the
activation dtype)."""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F
from torch import nn

ACTIVATIONS = ("relu2", "gelu_tanh")


def activate_(z: torch.Tensor, kind: str) -> torch.Tensor:
    if kind not in ACTIVATIONS:
        raise ValueError(f"unknown activation {kind!r}")
    if z.is_cuda:
        from .. import mixer_ops as M
        return M.activate_(z, kind)
    f = z.float()
    if kind == "relu2":
        f = torch.relu(f).pow(2)
    else:
        f = 0.5 * f * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (f + 0.044715 * f.pow(3))))
    return z.copy_(f.to(z.dtype))


class DenseFeedForward(nn.Module):
    def __init__(self, width: int, ff: int, activation: str = "relu2"):
        super().__init__()
        if activation not in ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}")
        self.activation = activation
        self.up = nn.Linear(width, ff, bias=False)
        self.down = nn.Linear(ff, width, bias=False)
        for p in self.parameters():
            p.requires_grad_(False)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(activate_(F.linear(h, self.up.weight), self.activation), self.down.weight)


GLU_KINDS = ("silu", "clamped_swish", "gelu_tanh", "sigmoid")


def _gate_act(g: torch.Tensor, kind: str) -> torch.Tensor:
    if kind == "silu":
        return F.silu(g)
    if kind == "sigmoid":
        return torch.sigmoid(g)
    return 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g.pow(3))))


def gate_mul(gate: torch.Tensor, up: torch.Tensor, kind: str) -> torch.Tensor:
    """act(gate) * up over rows [T, F] that need not be neighbours in memory (unit inner stride), fp32 arithmetic, a new tensor in
    the rows' dtype.  ``kind``: silu, sigmoid or gelu_tanh."""
    if kind not in ("silu", "sigmoid", "gelu_tanh"):
        raise ValueError(f"unknown gate activation {kind!r}")
    if gate.is_cuda:
        from .. import mixer_ops as M
        return M.gate_mul(gate, up, kind)
    return (_gate_act(gate.float(), kind) * up.float()).to(up.dtype)


def glu_(gu: torch.Tensor, kind: str = "silu", limit: float = 0.0, alpha: float = 1.702) -> torch.Tensor:
    """Rows ``gu`` [T, 2F] = gate | up  ->  [T, F] in the same dtype, fp32 arithmetic.  ``silu``: g sigmoid(g) u.  ``clamped_swish``:
    g' = min(g, limit), u' = clamp(u, -limit, limit), g' sigmoid(alpha g') (u' + 1).  ``gelu_tanh``: gelu(g) u in the tanh form.
    ``sigmoid``: sigmoid(g) u."""
    if kind not in GLU_KINDS:
        raise ValueError(f"unknown gated activation {kind!r}")
    if gu.is_cuda:
        from .. import mixer_ops as M
        return M.glu(gu, kind, limit, alpha)
    f = gu.shape[-1] // 2
    g, u = gu[..., :f].float(), gu[..., f:].float()
    if kind != "clamped_swish":
        return (_gate_act(g, kind) * u).to(gu.dtype)
    g, u = g.clamp(max=limit), u.clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


class GatedDenseFeedForward(nn.Module):
    """``down(act(gate h + b_g) * (up h + b_u)) + b_d``; gate and up are one product (rows gate | up); ``kind`` names the gate's
    activation (silu, gelu_tanh); ``bias=False``: no biases."""

    def __init__(self, width: int, ff: int, bias: bool = True, kind: str = "silu"):
        super().__init__()
        self.ff, self.kind = ff, kind
        self.gate_up = nn.Linear(width, 2 * ff, bias=bias)
        self.down = nn.Linear(ff, width, bias=bias)
        for p in self.parameters():
            p.requires_grad_(False)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(glu_(F.linear(h, self.gate_up.weight, self.gate_up.bias), self.kind), self.down.weight, self.down.bias)
