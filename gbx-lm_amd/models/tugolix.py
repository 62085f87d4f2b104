"""Tugolix: a decoder-only stack with several residual streams whose config.json lists its layers one by one.

A layer is a sequence mixer and, optionally, a feed-forward, each in pre-norm form with a layer norm (weight and bias).  With
config ``streams = s`` the residual is ``s`` streams (all equal to the embedding at the start): a sublayer reads a weighted sum of
them, and its output is written to all of them while a small matrix mixes the streams (models/residual.py:hyper_step_); without
``streams`` the same launches run the plain residual ``x += sublayer(norm(x))``.  The logits are
``logit_scale * head . norm(sum of the streams)``.  Mixer kinds: ``gla`` (gated linear attention) and ``channel_delta`` (gated delta
rule with a decay per key channel), both models/recurrent_mixers.py, and ``latent_attention`` without positions, sink or gate
(models/sink_attention.py), where ``kv_from: j`` makes a layer attend over layer j's cached latent rows.  Feed-forward kinds:
``dense`` (gated, with biases: models/feed_forward.py) and ``moe`` (sigmoid router with a choice correction and expert groups,
clamped experts: models/switch_layers.py:DenseRoutedGLU).  Every size and constant is read per layer from the config.  The streams
are fp32; matrix products run in the activation dtype (bf16 as stored, or fp32 when the model is loaded with
``dtype=torch.float32``).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional

import torch
import torch.nn.functional as F
from torch import nn

from ..batching import StepBatch
from .base import BaseModelArgs
from .cache import SequenceSlots
from .feed_forward import GatedDenseFeedForward
from .recurrent_mixers import ChannelDeltaRule, GatedLinearAttention
from .residual import StreamLayerNorm, hyper_step_
from .sink_attention import LatentAttention
from .step_model import RaggedStepModel
from .switch_layers import DenseRoutedGLU


@dataclass
class ModelArgs(BaseModelArgs):
    architecture: str
    vocab: int
    width: int
    layers: List[Dict[str, Any]]
    norm: Dict[str, Any]
    streams: Optional[int] = None
    logit_scale: float = 1.0
    shapes: Optional[Dict[str, Any]] = None      # sizes that only a tensor's shape gives (low ranks), filled in by the loader

    @property
    def model_type(self) -> str:
        return self.architecture.lower()


def _mixer(args: ModelArgs, i: int) -> nn.Module:
    spec = args.layers[i]
    kind, m, eps = spec["type"], spec["mixer"], args.norm["eps"]
    ranks = (args.shapes or {}).get(i, {})
    if kind == "gla":
        return GatedLinearAttention(args.width, m["heads"], m["dim"], m["vdim"], ranks.get("decay_rank", m.get("decay_rank", 16)), m["tau"], eps)
    if kind == "channel_delta":
        return ChannelDeltaRule(args.width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"], m["conv"],
                                ranks.get("decay_rank", m.get("decay_rank", 16)), ranks.get("gate_rank", m.get("gate_rank", 16)), eps)
    if kind == "latent_attention":
        src = m.get("kv_from")
        if src is not None:
            s = args.layers[src] if 0 <= src < i else None
            if s is None or s["type"] != "latent_attention" or "kv_from" in s["mixer"] or s["mixer"]["kv_rank"] != m["kv_rank"]:
                raise ValueError("Tugolix: kv_from names an earlier latent_attention layer with a latent projection of the same rank")
        return LatentAttention(args.width, m["heads"], m["dim"], 0, m["vdim"], m["kv_rank"], 10000.0, None, m["scale"], eps,
                               sink=False, gated=False, own_latent=src is None)
    raise ValueError(f"Tugolix: unknown mixer type {kind!r}")


def _feed_forward(args: ModelArgs, spec: Optional[Dict[str, Any]]) -> Optional[nn.Module]:
    if spec is None:
        return None
    if spec.get("kind") == "dense":
        return GatedDenseFeedForward(args.width, spec["ff"], bias=True)
    if spec.get("kind") == "moe":
        r, g = spec["router"], spec["router"].get("groups")
        return DenseRoutedGLU(args.width, spec["expert"]["ff"], r["experts"], r["top"], renormalize=True, scoring="sigmoid",
                              groups=None if not g else (g["count"], g["keep"]), route_scale=r.get("scale", 1.0),
                              activation="clamped_swish", limit=spec["expert"]["limit"])
    raise ValueError(f"Tugolix: unknown feed-forward kind {spec.get('kind')!r}")


class HyperConnection(nn.Module):
    """The three small tensors of one sublayer boundary: ``read`` [s], ``write`` [s], ``mix`` [s from, s to] (fp32)."""

    def __init__(self, streams: int):
        super().__init__()
        self.register_buffer("read", torch.ones(streams, dtype=torch.float32))
        self.register_buffer("write", torch.ones(streams, dtype=torch.float32))
        self.register_buffer("mix", torch.eye(streams, dtype=torch.float32))


class Layer(nn.Module):
    def __init__(self, args: ModelArgs, i: int):
        super().__init__()
        s = args.streams or 1
        self.norm1 = StreamLayerNorm(args.width, args.norm["eps"])
        self.hc1 = HyperConnection(s)
        self.mixer = _mixer(args, i)
        self.mlp = _feed_forward(args, args.layers[i].get("mlp"))
        if self.mlp is not None:
            self.norm2 = StreamLayerNorm(args.width, args.norm["eps"])
            self.hc2 = HyperConnection(s)

    def forward(self, streams: torch.Tensor, h: torch.Tensor, batch: StepBatch, cache, nxt: Optional["Layer"]) -> torch.Tensor:
        """``h`` = this layer's first norm of what it reads of the fp32 ``streams`` [T, s, W] (updated in place).  Returns the NEXT
        layer's first norm, or after the last layer the fp32 sum of the streams: every sublayer boundary is one launch."""
        dt = h.dtype
        y = self.mixer(h, batch, cache)
        read, norm = (None, None) if nxt is None else (nxt.hc1.read, nxt.norm1)
        if self.mlp is None:
            return hyper_step_(streams, y, None, self.hc1.mix, self.hc1.write, read, norm, dt)
        h = hyper_step_(streams, y, None, self.hc1.mix, self.hc1.write, self.hc2.read, self.norm2, dt)
        y = self.mlp(h)
        y, y_mix = y if isinstance(y, tuple) else (y, None)
        return hyper_step_(streams, y, y_mix, self.hc2.mix, self.hc2.write, read, norm, dt)


class TugolixModel(nn.Module):
    def __init__(self, args: ModelArgs):
        super().__init__()
        self.streams = args.streams or 1
        self.embed_tokens = nn.Embedding(args.vocab, args.width)
        self.embed_tokens.weight.requires_grad_(False)
        self.layers = nn.ModuleList(Layer(args, i) for i in range(len(args.layers)))
        self.norm = StreamLayerNorm(args.width, args.norm["eps"])

    def embed(self, tokens: torch.Tensor) -> torch.Tensor:
        """fp32 [T, s, W]: every stream starts as the embedding."""
        w = self.embed_tokens.weight
        if tokens.is_cuda:
            from .. import mixer_ops as M
            x = M.embed_scaled(w, tokens, 1.0, image=False)[0]
        else:
            x = w[tokens].float()
        return x.unsqueeze(1).repeat(1, self.streams, 1)


class Model(RaggedStepModel):
    def __init__(self, args: ModelArgs):
        super().__init__(args)
        self.model = TugolixModel(args)
        self.logit_scale = float(args.logit_scale)

    def make_cache(self) -> List[Any]:
        """One cache per layer over one shared slot table; a layer with ``kv_from`` gets a reader of the named layer's table."""
        slots = SequenceSlots(1)
        slots.length[0] = 0
        caches: List[Any] = []
        for spec, layer in zip(self.args.layers, self.model.layers):
            src = spec["mixer"].get("kv_from") if spec["type"] == "latent_attention" else None
            caches.append(layer.mixer.make_cache(slots) if src is None else layer.mixer.make_cache(slots, caches[src]))
        return caches

    def forward_tokens(self, tokens: torch.Tensor, batch: StepBatch, caches) -> torch.Tensor:
        """One ragged step: tokens [T] -> fp32 sum of the streams [T, width] after the last layer.  Positions are NOT advanced here."""
        streams = self.model.embed(tokens)
        layers = self.model.layers
        dt = self.lm_head.weight.dtype
        h = hyper_step_(streams, None, None, None, None, layers[0].hc1.read, layers[0].norm1, dt) if len(layers) else streams.sum(1)
        for n, (layer, cache) in enumerate(zip(layers, caches)):
            h = layer(streams, h, batch, cache, layers[n + 1] if n + 1 < len(layers) else None)
            if self.trace_layers is not None:
                self.trace_layers.append(streams.sum(1))
        return h

    def logits(self, x: torch.Tensor) -> torch.Tensor:
        """Last norm, output head and the logit scale (applied in fp32) on rows of the summed stream."""
        w = self.lm_head.weight
        return F.linear(self.model.norm(x, w.dtype), w).float() * self.logit_scale

    @staticmethod
    def shapes_from(weights: Dict[str, torch.Tensor], config: Dict[str, Any]) -> Dict[int, Dict[str, int]]:
        """Sizes the config does not name: the ranks of the low-rank decay and gate projections, per layer."""
        out: Dict[int, Dict[str, int]] = {}
        for i in range(len(config["layers"])):
            d = {}
            if f"l{i}.mix.a1" in weights:
                d["decay_rank"] = weights[f"l{i}.mix.a1"].shape[0]
            if f"l{i}.mix.g1" in weights:
                d["gate_rank"] = weights[f"l{i}.mix.g1"].shape[0]
            out[i] = d
        return out

    def sanitize(self, weights: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
        """Checkpoint names -> module paths.  Projections that read the same input are concatenated, the experts stacked; what only
        enters 32-bit arithmetic (norms, stream mixing, router and its correction, decay biases and rates) becomes fp32."""
        out: Dict[str, torch.Tensor] = {}
        f32 = lambda t: t.float()
        s = self.args.streams
        out["model.embed_tokens.weight"] = weights["embed"]
        out["model.norm.weight"], out["model.norm.bias"] = f32(weights["final.norm"]), f32(weights["final.norm.b"])
        out["lm_head.weight"] = weights["head"]
        for i, spec in enumerate(self.args.layers):
            p, t = f"l{i}.", f"model.layers.{i}."
            layer = self.model.layers[i]
            mixer, kind = layer.mixer, spec["type"]
            for q in (1, 2) if spec.get("mlp") is not None else (1,):
                out[t + f"norm{q}.weight"], out[t + f"norm{q}.bias"] = f32(weights[p + f"norm{q}"]), f32(weights[p + f"norm{q}.b"])
                hc = getattr(layer, f"hc{q}")
                out[t + f"hc{q}.read"] = f32(weights[p + f"hc{q}.in"]) if s else hc.read
                out[t + f"hc{q}.write"] = f32(weights[p + f"hc{q}.out"]) if s else hc.write
                out[t + f"hc{q}.mix"] = f32(weights[p + f"hc{q}.mix"]) if s else hc.mix
            m = p + "mix."
            if kind == "gla":
                parts = [weights[m + "q"], weights[m + "k"], weights[m + "v"], weights[m + "g"], weights[m + "a1"]]
                pad = torch.zeros((mixer.inp.out_features - sum(x.shape[0] for x in parts), self.args.width), dtype=parts[0].dtype, device=parts[0].device)
                out[t + "mixer.inp.weight"] = torch.cat(parts + [pad])
                out[t + "mixer.a2.weight"] = weights[m + "a2"]
                out[t + "mixer.decay_bias"] = f32(weights[m + "a2.b"])
                out[t + "mixer.decay_rate"] = mixer.decay_rate
                out[t + "mixer.out_norm"] = f32(weights[m + "norm"])
            elif kind == "channel_delta":
                out[t + "mixer.inp.weight"] = mixer.fuse_weights(weights[m + "q"], weights[m + "k"], weights[m + "v"], weights[m + "b"],
                                                                 weights[m + "a1"], weights[m + "g1"])
                out[t + "mixer.conv"] = torch.cat([weights[m + "q.conv"], weights[m + "k.conv"], weights[m + "v.conv"]])
                out[t + "mixer.a2.weight"], out[t + "mixer.g2.weight"] = weights[m + "a2"], weights[m + "g2"]
                out[t + "mixer.decay_bias"] = f32(weights[m + "dt_bias"])
                out[t + "mixer.decay_rate"] = torch.exp(f32(weights[m + "A_log"]))
                out[t + "mixer.out_norm"] = f32(weights[m + "norm"])
            else:
                own = mixer.own_latent
                fused = mixer.fuse_weights(weights[m + "q"], weights[m + "dkv"] if own else None, None, weights[m + "uk"], weights[m + "uv"])
                for k, v in fused.items():
                    out[t + "mixer." + k] = v
                if own:
                    out[t + "mixer.latent_norm"] = f32(weights[m + "dkv.norm"])
                out[t + "mixer.freq"] = mixer.freq
            out[t + "mixer.o.weight"] = weights[m + "o"]
            ff = spec.get("mlp")
            if ff is not None and ff["kind"] == "dense":
                f = p + "mlp."
                out[t + "mlp.gate_up.weight"] = torch.cat([weights[f + "gate"], weights[f + "up"]])
                out[t + "mlp.gate_up.bias"] = torch.cat([weights[f + "gate.b"], weights[f + "up.b"]])
                out[t + "mlp.down.weight"], out[t + "mlp.down.bias"] = weights[f + "down"], weights[f + "down.b"]
            elif ff is not None:
                f, n_e = p + "mlp.", ff["router"]["experts"]
                out[t + "mlp.router"], out[t + "mlp.correction"] = f32(weights[f + "router"]), f32(weights[f + "correction"])
                out[t + "mlp.gate_up"] = torch.stack([torch.cat([weights[f + f"e{e}.gate"], weights[f + f"e{e}.up"]]) for e in range(n_e)])
                out[t + "mlp.down"] = torch.stack([weights[f + f"e{e}.down"] for e in range(n_e)])
        return out
