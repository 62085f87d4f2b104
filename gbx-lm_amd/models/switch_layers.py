"""Expert-indexed (mixture-of-experts) linears around the GBA packed format.

PyTorch-ROCm counterpart of gbx_lm/models/switch_layers.py: ``QuantizedSwitchLinear`` (:26-92) keeps the reference's
constructor ``(input_dims, output_dims, num_experts, bias=True, group_size=64, bits=4)``, its parameters
``qweight [E, N, K*bits/32]`` / ``scales, zeros [E, N, K/g]`` / ``bias [E, N]`` and its call ``(x, indices,
sorted_indices=False)``; the arithmetic the reference delegates to ``mx.gather_qmm`` runs in the HIP library
(``ops.gather_quantized_matmul`` -> ``gbx_gather_qlinear_forward`` / per-expert ``gbx_qlinear_forward``).
``SwitchGLU`` (:157-203) routes every token through its top-k experts; sorting tokens by expert (:186-200) only
changes the order of evaluation in the reference and is subsumed by the grouped path here.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops


class QuantizedSwitchLinear(nn.Module):
    def __init__(self, input_dims: int, output_dims: int, num_experts: int, bias: bool = True,
                 group_size: int = 64, bits: int = 4):
        super().__init__()
        self.scale = math.sqrt(1 / input_dims)
        self.input_dims, self.output_dims = input_dims, output_dims
        self.group_size, self.bits, self.num_experts = group_size, bits, num_experts
        for nm in ("qweight", "scales", "zeros", "bias"):
            self.register_buffer(nm, None)
        self.init_params()
        if bias:
            self.bias = torch.zeros((num_experts, output_dims), dtype=torch.float16)

    def init_params(self, *_ignored) -> None:
        """Allocate the packed tensors for the current (bits, group_size) (the reference quantises a random matrix
        with mx.quantize, switch_layers.py:50-60; the values are overwritten by the checkpoint either way)."""
        e, n, k = self.num_experts, self.output_dims, self.input_dims
        self.qweight = torch.zeros((e, n, k // 32 * self.bits), dtype=torch.int32).view(torch.uint32)
        self.scales = torch.zeros((e, n, k // self.group_size), dtype=torch.float16)
        self.zeros = torch.zeros((e, n, k // self.group_size), dtype=torch.float16)

    def set_bias_and_weight(self) -> None:
        """GBA-native zero point -> MLX sign (switch_layers.py:62-71)."""
        self.zeros = -self.zeros

    def create_scales_zeros(self) -> None:       # double quantisation does not apply to the stacked experts
        return

    def extra_repr(self) -> str:
        return (f"input_dims={self.input_dims}, output_dims={self.output_dims}, num_experts={self.num_experts}, "
                f"bias={self.bias is not None}, group_size={self.group_size}, bits={self.bits}")

    def forward(self, x: torch.Tensor, indices: torch.Tensor, sorted_indices: bool = False) -> torch.Tensor:
        return ops.gather_quantized_matmul(x, self.qweight, scales=self.scales, biases=self.zeros, rhs_indices=indices,
                                           transpose=True, group_size=self.group_size, bits=self.bits,
                                           sorted_indices=sorted_indices, bias=self.bias)


class SwitchLinear(nn.Module):
    """Unquantised expert-indexed linear (switch_layers.py:95-141): weight [E, N, K]."""

    def __init__(self, input_dims: int, output_dims: int, num_experts: int, bias: bool = True):
        super().__init__()
        scale = math.sqrt(1 / input_dims)
        self.weight = nn.Parameter(torch.empty((num_experts, output_dims, input_dims)).uniform_(-scale, scale),
                                   requires_grad=False)
        self.bias = nn.Parameter(torch.zeros((num_experts, output_dims)), requires_grad=False) if bias else None

    @property
    def input_dims(self): return self.weight.shape[2]
    @property
    def output_dims(self): return self.weight.shape[1]
    @property
    def num_experts(self): return self.weight.shape[0]

    def forward(self, x: torch.Tensor, indices: torch.Tensor, sorted_indices: bool = False) -> torch.Tensor:
        w = self.weight[indices]                                   # [..., k, N, K]
        y = torch.matmul(x, w.transpose(-1, -2))                   # [..., k, 1, N]
        if self.bias is not None:
            y = y + self.bias[indices].unsqueeze(-2)
        return y


class SwiGLU(nn.Module):
    def forward(self, x: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
        if (gate.is_cuda and gate.dtype in (torch.bfloat16, torch.float16) and gate.shape == x.shape and gate.numel() % 8 == 0
                and gate.is_contiguous() and x.is_contiguous()):
            return ops.swiglu(gate, x)                                # one launch, same two roundings
        return F.silu(gate) * x


class SwitchGLU(nn.Module):
    """Top-k gated MLP over stacked experts: down(act(up(x), gate(x))) per (token, slot)  (switch_layers.py:157-203)."""

    def __init__(self, input_dims: int, hidden_dims: int, num_experts: int, activation: Optional[nn.Module] = None,
                 bias: bool = False, quant: bool = True):
        super().__init__()
        cls = QuantizedSwitchLinear if quant else SwitchLinear
        self.gate_proj = cls(input_dims, hidden_dims, num_experts, bias=bias)
        self.up_proj = cls(input_dims, hidden_dims, num_experts, bias=bias)
        self.down_proj = cls(hidden_dims, input_dims, num_experts, bias=bias)
        self.activation = activation if activation is not None else SwiGLU()

    def forward(self, x: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        x = x.unsqueeze(-2).unsqueeze(-3)                          # [..., 1, 1, D]: one row shared by the k slots
        act = None
        if (isinstance(self.activation, SwiGLU) and isinstance(self.gate_proj, QuantizedSwitchLinear)
                and isinstance(self.up_proj, QuantizedSwitchLinear) and x.is_cuda):
            act = ops.gather_swiglu(x, self.gate_proj, self.up_proj, indices)    # one expert-indexed launch, or None
        if act is None:
            x_up = self.up_proj(x, indices)
            x_gate = self.gate_proj(x, indices)
            act = self.activation(x_up, x_gate)
        y = self.down_proj(act, indices)                            # [..., k, 1, D]
        return y.squeeze(-2)


class DenseRoutedGLU(nn.Module):
    """Top-k routed gated MLPs over unquantised stacked experts, rows of a ragged step in, the chosen experts' outputs out.

    Router, ``scoring = "softmax"``: logits in fp32 (``router`` is kept in fp32), probabilities = softmax over ALL experts, the
    ``top`` largest are chosen (ties: the lower expert index); their mixing weights are those probabilities, divided by their sum
    only if ``renormalize``.  ``scoring = "sigmoid"``: scores s = sigmoid(logits); the choice runs on s + ``correction`` (a vector per
    expert that steers the choice and never the weights); with ``groups = (count, keep)`` the experts form ``count`` equal groups of
    neighbours, a group's score is the sum of its two largest choice scores and only experts of the ``keep`` best groups can be
    chosen; weights = the chosen s, divided by their sum (+ 1e-20) if ``renormalize``, times ``route_scale``.
    Expert e: down_e(act(gate_e h, up_e h)); ``activation = "silu"``: silu(g) u; ``"clamped_swish"``: g' = min(g, limit), u' =
    clamp(u, -limit, limit), g' sigmoid(1.702 g') (u' + 1).  ``gate_up`` stacks gate_e over up_e as [E, 2F, K], ``down`` is [E, K, F].
    ``forward`` returns (y [T, top, K], weights fp32 [T, top]): the weighted sum is left to the caller, which folds it into its
    normalisation / residual launch."""

    def __init__(self, input_dims: int, hidden_dims: int, num_experts: int, top: int, renormalize: bool = False, scoring: str = "softmax",
                 groups=None, route_scale: float = 1.0, activation: str = "silu", limit: float = 0.0):
        super().__init__()
        if not 1 <= top <= num_experts:
            raise ValueError("top must lie in 1..num_experts")
        if scoring not in ("softmax", "sigmoid") or activation not in ("silu", "clamped_swish"):
            raise ValueError("unknown router scoring or expert activation")
        if groups is not None and (num_experts % groups[0] or not 1 <= groups[1] <= groups[0] or top > groups[1] * (num_experts // groups[0])):
            raise ValueError("groups: equal groups, 1 <= keep <= count, and the kept groups hold at least top experts")
        self.input_dims, self.hidden_dims, self.num_experts, self.top, self.renormalize = input_dims, hidden_dims, num_experts, top, renormalize
        self.scoring, self.groups, self.route_scale = scoring, (None if groups is None else (int(groups[0]), int(groups[1]))), float(route_scale)
        self.activation, self.limit = activation, float(limit)
        self.register_buffer("router", torch.zeros((num_experts, input_dims), dtype=torch.float32))
        if scoring == "sigmoid":
            self.register_buffer("correction", torch.zeros(num_experts, dtype=torch.float32))
        self.register_buffer("gate_up", torch.zeros((num_experts, 2 * hidden_dims, input_dims)))
        self.register_buffer("down", torch.zeros((num_experts, input_dims, hidden_dims)))

    def route(self, h: torch.Tensor):
        if h.is_cuda:
            from .. import mixer_ops as M
            if self.scoring == "sigmoid":
                return M.route_sigmoid_groups(h, self.router, self.correction, self.top, self.groups, self.renormalize, self.route_scale)
            return M.route_topk(h, self.router, self.top, self.renormalize)
        logits = F.linear(h.float(), self.router.float())
        if self.scoring == "sigmoid":
            s = torch.sigmoid(logits)
            c = s + self.correction.float()
            if self.groups is not None:
                count, keep = self.groups
                per = c.view(c.shape[0], count, -1)
                score = per.sort(dim=-1, descending=True).values[..., :2].sum(-1)
                best = torch.sort(score, dim=-1, descending=True, stable=True).indices[:, :keep]
                allowed = torch.zeros_like(score, dtype=torch.bool).scatter_(1, best, True)
                c = torch.where(allowed[:, :, None].expand_as(per), per, torch.full_like(per, float("-inf"))).reshape(c.shape)
            idx = torch.sort(c, dim=-1, descending=True, stable=True).indices[..., :self.top]
            w = torch.gather(s, 1, idx)
            if self.renormalize:
                w = w / (w.sum(-1, keepdim=True) + 1e-20)
            return idx.to(torch.int32), w * self.route_scale
        probs = torch.softmax(logits, dim=-1)
        w, idx = torch.sort(probs, dim=-1, descending=True, stable=True)      # of equal experts the lower index first
        w, idx = w[..., :self.top], idx[..., :self.top]
        if self.renormalize:
            w = w / w.sum(-1, keepdim=True)
        return idx.to(torch.int32), w

    def forward(self, h: torch.Tensor):
        idx, w = self.route(h)
        if h.is_cuda:
            from .. import mixer_ops as M
            return M.expert_glu(h, self.gate_up, self.down, idx, self.activation, self.limit), w
        from .feed_forward import glu_
        y = torch.empty((h.shape[0], self.top, self.input_dims), dtype=h.dtype, device=h.device)
        for e in range(self.num_experts):
            t, s = torch.nonzero(idx == e, as_tuple=True)
            if t.numel():
                y[t, s] = F.linear(glu_(F.linear(h[t], self.gate_up[e]), self.activation, self.limit), self.down[e])
        return y, w
