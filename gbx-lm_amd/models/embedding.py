"""Token embeddings of ragged-step models beyond the plain table look-up.

``HashedPairEmbedding``: the stream starts as ``embed[token] + pair[row]`` where ``row`` is a hash of the (previous token, token)
pair, ``(previous * mul_prev + token * mul_cur) mod buckets``; a sequence's first token has no previous one and takes the table's
extra last row (row number ``buckets``).  The previous token is state of the sequence: a ``SlotRowCache`` of one int64 per slot
holds the last token of every step.  The stream is fp32.

GPU tensors: one HIP launch (look-ups, sum, state update); CPU tensors: the plain torch graph below.
"""
from __future__ import annotations

import torch
from torch import nn

from .cache import SlotRowCache


class HashedPairEmbedding(nn.Module):
    def __init__(self, vocab: int, width: int, buckets: int, mul_prev: int, mul_cur: int):
        super().__init__()
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        if self.buckets < 1:
            raise ValueError("HashedPairEmbedding: at least one bucket")
        self.weight = nn.Parameter(torch.zeros((vocab, width)), requires_grad=False)
        self.pair = nn.Parameter(torch.zeros((self.buckets + 1, width)), requires_grad=False)

    def make_cache(self, slots) -> SlotRowCache:
        return SlotRowCache(1, "i64", slots)

    def forward(self, tokens: torch.Tensor, batch, cache: SlotRowCache) -> torch.Tensor:
        """tokens int64 [T] (the step's rows) -> fp32 [T, W]; leaves every sequence's last token in its slot."""
        cache.reserve(self.weight.dtype, tokens.device)
        if tokens.is_cuda:
            from .. import mixer_ops as M
            return M.embed_hashed_pair(self.weight, self.pair, tokens, batch, cache.rows, self.buckets, self.mul_prev, self.mul_cur)
        tokens = tokens.to(torch.long)
        rows = torch.empty_like(tokens)
        r0 = 0
        for slot, pos0, n in zip(batch.slot, batch.pos0, batch.n_new):
            tk = tokens[r0:r0 + n]
            prev = torch.cat([cache.rows[slot] if pos0 else tk[:1], tk[:-1]])
            rows[r0:r0 + n] = (prev * self.mul_prev + tk * self.mul_cur) % self.buckets
            if pos0 == 0:
                rows[r0] = self.buckets
            cache.rows[slot, 0] = tk[-1]
            r0 += n
        return self.weight[tokens].float() + self.pair[rows].float()
