"""Two sequence mixers side by side: both read the same input, each output is RMS-normalised over the model width with a weight of
its own, and the result is half their sum.  The pair's cache is a ``CacheGroup`` with the parts ``left`` and ``right``."""
from __future__ import annotations

import torch
from torch import nn

from .cache import CacheGroup
from .residual import normed_pair_mean


class ParallelMixers(nn.Module):
    def __init__(self, left: nn.Module, right: nn.Module, width: int, eps: float):
        super().__init__()
        self.left, self.right, self.eps = left, right, float(eps)
        self.register_buffer("left_norm", torch.ones(width, dtype=torch.float32))
        self.register_buffer("right_norm", torch.ones(width, dtype=torch.float32))

    def make_cache(self, slots) -> CacheGroup:
        return CacheGroup(slots, left=self.left.make_cache(slots), right=self.right.make_cache(slots))

    def forward(self, h: torch.Tensor, batch, cache: CacheGroup) -> torch.Tensor:
        return normed_pair_mean(self.left(h, batch, cache.left), self.right(h, batch, cache.right), self.left_norm, self.right_norm, self.eps)
