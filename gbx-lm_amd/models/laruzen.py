"""Laruzen: a decoder-only stack in sandwich-norm form whose config.json lists its layers one by one.

The stream starts as the token embedding plus a hashed (previous token, token) pair embedding (models/embedding.py).  A layer is
``x += norm1b(mixer(shift(norm1(x))))`` and, optionally, ``x += norm2b(ff(norm2(x)))``: every norm is an RMS norm whose stored
weight is an offset from one, and ``shift`` mixes each channel of the mixer's input with the previous token's
(models/residual.py:norm_token_shift).  Mixer kinds: ``gla`` (gated linear attention with a decay per key channel) and ``lightning``
(linear attention with a constant decay per head), both models/recurrent_mixers.py, and ``parallel``: a grouped-query sliding-window
softmax attention with a learned sink (models/sink_attention.py:GatedSinkWindowAttention) next to a recurrent block around a
real-gated linear recurrent unit (models/gated_lru.py), joined by models/parallel_mixers.py.  Feed-forward kinds: ``dense`` (gated,
gelu) and ``moe`` (softmax over the chosen experts' logits, silu experts, optionally a shared expert that every token takes).
Every size and constant is read per layer from the config; ranks that only a tensor's shape holds come from the checkpoint.  The
stream, the norms, the router, the attention's scores and everything of the recurrences is fp32; matrix products run in the
activation dtype (bf16 as stored, or fp32 when the model is loaded with ``dtype=torch.float32``).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch
import torch.nn.functional as F
from torch import nn

from ..batching import StepBatch
from .base import BaseModelArgs
from .cache import CacheGroup, SequenceSlots, SlotRowCache
from .embedding import HashedPairEmbedding
from .feed_forward import GatedDenseFeedForward
from .gated_lru import GatedLRUBlock
from .parallel_mixers import ParallelMixers
from .recurrent_mixers import GatedLinearAttention, LightningAttention
from .residual import StreamRMSNorm, branch_norm_add_norm_, norm_token_shift
from .sink_attention import GatedSinkWindowAttention
from .step_model import RaggedStepModel
from .switch_layers import DenseRoutedGLU

LRU_RATE = 8.0          # the recurrent unit's log-decay is -8 * gate * softplus(lam)


@dataclass
class ModelArgs(BaseModelArgs):
    architecture: str
    vocab: int
    width: int
    layers: List[Dict[str, Any]]
    norm: Dict[str, Any]
    embedding: Dict[str, Any] = field(default_factory=dict)
    shapes: Optional[Dict[int, Dict[str, int]]] = None      # sizes that only a tensor's shape gives (the decay's low rank)

    @property
    def model_type(self) -> str:
        return self.architecture.lower()


def _mixer(args: ModelArgs, i: int) -> nn.Module:
    spec = args.layers[i]
    kind, m, eps = spec["type"], spec["mixer"], args.norm["eps"]
    if kind == "gla":
        rank = (args.shapes or {}).get(i, {}).get("decay_rank", m.get("decay_rank", 16))
        return GatedLinearAttention(args.width, m["heads"], m["dim"], m["vdim"], rank, m["tau"], eps)
    if kind == "lightning":
        return LightningAttention(args.width, m["heads"], m["dim"], m["vdim"], m["decay"], eps)
    if kind == "parallel":
        l, r = m["left"], m["right"]
        rot, mask = l.get("rot") or {}, l.get("mask") or {}
        left = GatedSinkWindowAttention(args.width, l["heads"], l.get("kv_heads", l["heads"]), l["dim"], l["vdim"], rot.get("dims", 0),
                                        rot.get("base", 10000.0), rot.get("scaling"), mask.get("size"), l["scale"], eps)
        right = GatedLRUBlock(args.width, r["width"], r["blocks"], r["conv"], LRU_RATE)
        return ParallelMixers(left, right, args.width, eps)
    raise ValueError(f"Laruzen: unknown mixer type {kind!r}")


class SharedExpertMoE(nn.Module):
    """Routed experts plus, optionally, one expert of the same form that every token takes.  Returns the routed candidates, their
    weights and the shared expert's output: the caller's stream update sums them in fp32."""

    def __init__(self, width: int, spec: Dict[str, Any]):
        super().__init__()
        r = spec["router"]
        self.routed = DenseRoutedGLU(width, spec["expert"]["ff"], r["experts"], r["top"], renormalize=True)
        sh = spec.get("shared")
        self.shared = GatedDenseFeedForward(width, sh["ff"], bias=False, kind="silu") if sh else None

    def forward(self, h: torch.Tensor):
        y, mix = self.routed(h)
        return y, mix, (None if self.shared is None else self.shared(h))


def _feed_forward(args: ModelArgs, spec: Optional[Dict[str, Any]]) -> Optional[nn.Module]:
    if spec is None:
        return None
    if spec.get("kind") == "dense":
        return GatedDenseFeedForward(args.width, spec["ff"], bias=False, kind="gelu_tanh")
    if spec.get("kind") == "moe":
        return SharedExpertMoE(args.width, spec)
    raise ValueError(f"Laruzen: unknown feed-forward kind {spec.get('kind')!r}")


class Layer(nn.Module):
    def __init__(self, args: ModelArgs, i: int):
        super().__init__()
        w, self.eps = args.width, float(args.norm["eps"])
        self.mixer = _mixer(args, i)
        self.mlp = _feed_forward(args, args.layers[i].get("mlp"))
        # norm weights as multipliers (1 + stored), fp32
        for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if self.mlp is not None else ()):
            self.register_buffer(nm, torch.ones(w, dtype=torch.float32))
        self.register_buffer("shift", torch.zeros(w, dtype=torch.float32))

    def make_cache(self, slots) -> CacheGroup:
        return CacheGroup(slots, shift=SlotRowCache(self.shift.numel(), "f32", slots), mixer=self.mixer.make_cache(slots))

    def forward(self, x: torch.Tensor, batch: StepBatch, cache: CacheGroup, dt: torch.dtype) -> None:
        """One layer on the fp32 stream ``x`` (in place)."""
        h = norm_token_shift(x, self.norm1, self.eps, self.shift, cache.shift, batch, dt)
        y = self.mixer(h, batch, cache.mixer)
        if self.mlp is None:
            branch_norm_add_norm_(x, y, None, None, self.norm1b, self.eps, None, dt)
            return
        h = branch_norm_add_norm_(x, y, None, None, self.norm1b, self.eps, self.norm2, dt)
        z = self.mlp(h)
        z, mix, extra = z if isinstance(z, tuple) else (z, None, None)
        branch_norm_add_norm_(x, z, mix, extra, self.norm2b, self.eps, None, dt)


class LaruzenModel(nn.Module):
    def __init__(self, args: ModelArgs):
        super().__init__()
        pair = args.embedding.get("bigram")
        if pair:
            self.embed_tokens = HashedPairEmbedding(args.vocab, args.width, pair["buckets"], pair["mul_prev"], pair["mul_cur"])
        else:
            self.embed_tokens = nn.Embedding(args.vocab, args.width)
            self.embed_tokens.weight.requires_grad_(False)
        self.layers = nn.ModuleList(Layer(args, i) for i in range(len(args.layers)))
        self.norm = StreamRMSNorm(args.width, args.norm["eps"])


class Model(RaggedStepModel):
    def __init__(self, args: ModelArgs):
        super().__init__(args)
        self.model = LaruzenModel(args)

    def make_cache(self) -> List[Any]:
        """One ``CacheGroup`` per layer (token shift row + the mixer's state) over one shared slot table; the first layer's also
        carries what the embedding keeps (the previous token)."""
        slots = SequenceSlots(1)
        slots.length[0] = 0
        caches = [layer.make_cache(slots) for layer in self.model.layers]
        emb = self.model.embed_tokens
        if isinstance(emb, HashedPairEmbedding):
            if not caches:
                raise ValueError("Laruzen: a model without layers has nowhere to keep the previous token")
            caches[0] = CacheGroup(slots, embed=emb.make_cache(slots), **caches[0].parts)
        return caches

    def forward_tokens(self, tokens: torch.Tensor, batch: StepBatch, caches) -> torch.Tensor:
        """One ragged step: tokens [T] -> fp32 stream [T, width] after the last layer.  Positions are NOT advanced here."""
        emb = self.model.embed_tokens
        if isinstance(emb, HashedPairEmbedding):
            x = emb(tokens, batch, caches[0].embed)
        elif tokens.is_cuda:
            from .. import mixer_ops as M
            x = M.embed_scaled(emb.weight, tokens, 1.0, image=False)[0]
        else:
            x = emb.weight[tokens].float()
        dt = self.lm_head.weight.dtype
        for layer, cache in zip(self.model.layers, caches):
            layer(x, batch, cache, dt)
            if self.trace_layers is not None:
                self.trace_layers.append(x.clone())
        return x

    @staticmethod
    def shapes_from(weights: Dict[str, torch.Tensor], config: Dict[str, Any]) -> Dict[int, Dict[str, int]]:
        """Sizes the config does not name: the rank of a gla mixer's low-rank decay projection, per layer."""
        return {i: {"decay_rank": weights[f"l{i}.mix.a1"].shape[0]} for i in range(len(config["layers"])) if f"l{i}.mix.a1" in weights}

    def sanitize(self, weights: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
        """Checkpoint names -> module paths.  Projections that read the same input are concatenated, the experts stacked; what only
        enters 32-bit arithmetic (norms as 1 + stored, shift, router, sinks, decay biases, gate biases, softplus(lam)) becomes fp32."""
        out: Dict[str, torch.Tensor] = {}
        f32 = lambda t: t.float()
        one_plus = lambda t: 1.0 + t.float()
        out["model.embed_tokens.weight"] = weights["embed"]
        if "bigram" in weights:
            out["model.embed_tokens.pair"] = weights["bigram"]
        out["model.norm.weight"] = one_plus(weights["final.norm"])
        out["lm_head.weight"] = weights["head"]
        for i, spec in enumerate(self.args.layers):
            p, t = f"l{i}.", f"model.layers.{i}."
            layer = self.model.layers[i]
            mixer, kind = layer.mixer, spec["type"]
            for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if spec.get("mlp") is not None else ()):
                out[t + nm] = one_plus(weights[p + nm])
            out[t + "shift"] = f32(weights[p + "shift"])
            m = p + "mix."
            if kind == "gla":
                parts = [weights[m + "q"], weights[m + "k"], weights[m + "v"], weights[m + "g"], weights[m + "a1"]]
                pad = torch.zeros((mixer.inp.out_features - sum(x.shape[0] for x in parts), self.args.width), dtype=parts[0].dtype, device=parts[0].device)
                out[t + "mixer.inp.weight"] = torch.cat(parts + [pad])
                out[t + "mixer.a2.weight"] = weights[m + "a2"]
                out[t + "mixer.decay_bias"] = f32(weights[m + "a2.b"])
                out[t + "mixer.decay_rate"] = mixer.decay_rate
                out[t + "mixer.out_norm"] = f32(weights[m + "norm"])
                out[t + "mixer.o.weight"] = weights[m + "o"]
            elif kind == "lightning":
                parts = [weights[m + "q"], weights[m + "k"], weights[m + "v"], weights[m + "g"]]
                pad = torch.zeros((mixer.inp.out_features - sum(x.shape[0] for x in parts), self.args.width), dtype=parts[0].dtype, device=parts[0].device)
                out[t + "mixer.inp.weight"] = torch.cat(parts + [pad])
                out[t + "mixer.decay_rate"] = mixer.decay_rate
                out[t + "mixer.out_norm"] = f32(weights[m + "norm"])
                out[t + "mixer.o.weight"] = weights[m + "o"]
            else:
                l, r = m + "left.", m + "right."
                w, b = mixer.left.fuse_weights(weights[l + "q"], weights[l + "k"], weights[l + "v"], weights[l + "g"],
                                               weights[l + "q.b"], weights[l + "k.b"], weights[l + "v.b"])
                out[t + "mixer.left.inp.weight"], out[t + "mixer.left.inp.bias"] = w, b
                out[t + "mixer.left.o.weight"], out[t + "mixer.left.o.bias"] = weights[l + "o"], weights[l + "o.b"]
                out[t + "mixer.left.q_norm"], out[t + "mixer.left.k_norm"] = f32(weights[l + "q.norm"]), f32(weights[l + "k.norm"])
                out[t + "mixer.left.sink"] = f32(weights[l + "sink"])
                out[t + "mixer.left.freq"] = mixer.left.freq
                out[t + "mixer.right.inp.weight"] = torch.cat([weights[r + "x"], weights[r + "y"]])
                out[t + "mixer.right.inp.bias"] = torch.cat([weights[r + "x.b"], weights[r + "y.b"]])
                out[t + "mixer.right.conv"], out[t + "mixer.right.conv_bias"] = weights[r + "conv"], f32(weights[r + "conv.b"])
                out[t + "mixer.right.gates"] = torch.cat([weights[r + "ra"], weights[r + "ri"]], dim=1)
                out[t + "mixer.right.gates_bias"] = torch.cat([f32(weights[r + "ra.b"]), f32(weights[r + "ri.b"])], dim=1)
                out[t + "mixer.right.lam_sp"] = F.softplus(f32(weights[r + "lam"]))
                out[t + "mixer.right.o.weight"] = weights[r + "o"]
                out[t + "mixer.left_norm"], out[t + "mixer.right_norm"] = f32(weights[m + "left.out"]), f32(weights[m + "right.out"])
            ff = spec.get("mlp")
            f = p + "mlp."
            if ff is not None and ff["kind"] == "dense":
                out[t + "mlp.gate_up.weight"] = torch.cat([weights[f + "gate"], weights[f + "up"]])
                out[t + "mlp.down.weight"] = weights[f + "down"]
            elif ff is not None:
                n_e = ff["router"]["experts"]
                out[t + "mlp.routed.router"] = f32(weights[f + "router"])
                out[t + "mlp.routed.gate_up"] = torch.stack([torch.cat([weights[f + f"e{e}.gate"], weights[f + f"e{e}.up"]]) for e in range(n_e)])
                out[t + "mlp.routed.down"] = torch.stack([weights[f + f"e{e}.down"] for e in range(n_e)])
                if ff.get("shared"):
                    out[t + "mlp.shared.gate_up.weight"] = torch.cat([weights[f + "shared.gate"], weights[f + "shared.up"]])
                    out[t + "mlp.shared.down.weight"] = weights[f + "shared.down"]
        return out
