"""Synthetic GBA checkpoints with the real tensor names / shapes / dtypes (no network, no real weights).

Distributions follow SURVEY.md 8d: uniform random packed words, ``scales ~ U(0.5,1.5)*2/(2^b-1)*0.02``,
``zeros = -scales*(2^b-1)/2 + N(0, 0.1*scales)`` (MLX-signed, i.e. added), embeddings ``N(0, 0.02)``.
Used by bench.py, the tests and ``__graft_entry__.smoke()``; the layout written to disk is exactly what
``load()`` reads (gbx_lm/utils.py:752-879 contract).
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, Optional

import torch

from .models import qdeepseek_v3, qllama, qmixtral, qphi3, qqwen2, qqwen3, qqwen3_moe
from .models.switch_layers import QuantizedSwitchLinear
from .models.quantized_linear_gba import QuantizedLinear

PROJ = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")

LLAMA3_8B = dict(model_type="llama", hidden_size=4096, intermediate_size=14336, num_hidden_layers=32,
                 num_attention_heads=32, num_key_value_heads=8, rms_norm_eps=1e-5, vocab_size=128256,
                 rope_theta=500000.0, max_position_embeddings=8192, tie_word_embeddings=False,
                 eos_token_id=128009)
LLAMA32_3B = dict(model_type="llama", hidden_size=3072, intermediate_size=8192, num_hidden_layers=28,
                  num_attention_heads=24, num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-5, vocab_size=128256,
                  rope_theta=500000.0, max_position_embeddings=131072, tie_word_embeddings=True,
                  rope_scaling=dict(factor=32.0, high_freq_factor=4.0, low_freq_factor=1.0,
                                    original_max_position_embeddings=8192, rope_type="llama3"),
                  eos_token_id=128009)
TINY = dict(model_type="llama", hidden_size=256, intermediate_size=512, num_hidden_layers=2,
            num_attention_heads=4, num_key_value_heads=2, rms_norm_eps=1e-5, vocab_size=512,
            rope_theta=10000.0, max_position_embeddings=512, tie_word_embeddings=False, eos_token_id=511)


QWEN3_30B_A3B = dict(model_type="qwen3_moe", hidden_size=2048, intermediate_size=6144, moe_intermediate_size=768,
                     num_hidden_layers=48, num_attention_heads=32, num_key_value_heads=4, head_dim=128, num_experts=128,
                     num_experts_per_tok=8, decoder_sparse_step=1, mlp_only_layers=[], norm_topk_prob=True,
                     rms_norm_eps=1e-6, vocab_size=151936, rope_theta=1000000.0, max_position_embeddings=40960,
                     tie_word_embeddings=False, eos_token_id=151645)          # public Qwen3-30B-A3B shapes
QWEN3_8B = dict(model_type="qwen3", hidden_size=4096, intermediate_size=12288, num_hidden_layers=36, num_attention_heads=32,
                num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-6, vocab_size=151936, rope_theta=1000000.0,
                max_position_embeddings=40960, tie_word_embeddings=False, eos_token_id=151645)     # public Qwen3-8B shapes
TINY_MOE = dict(model_type="qwen3_moe", hidden_size=256, intermediate_size=512, moe_intermediate_size=128,
                num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=64, num_experts=8,
                num_experts_per_tok=2, decoder_sparse_step=1, mlp_only_layers=[], norm_topk_prob=True,
                rms_norm_eps=1e-6, vocab_size=512, rope_theta=10000.0, max_position_embeddings=512,
                tie_word_embeddings=False, eos_token_id=511)


TINY_QWEN2 = dict(model_type="qwen2", hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                  num_key_value_heads=2, rms_norm_eps=1e-6, vocab_size=512, rope_theta=1000000.0,
                  max_position_embeddings=512, tie_word_embeddings=True, eos_token_id=511)
TINY_MIXTRAL = dict(model_type="mixtral", hidden_size=256, intermediate_size=128, num_hidden_layers=2,
                    num_attention_heads=4, num_key_value_heads=2, num_local_experts=4, num_experts_per_tok=2,
                    rms_norm_eps=1e-5, vocab_size=512, rope_theta=1000000.0, max_position_embeddings=512, eos_token_id=511)
TINY_PHI3 = dict(model_type="phi3", hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                 num_key_value_heads=2, rms_norm_eps=1e-5, vocab_size=512, rope_theta=10000.0,
                 max_position_embeddings=4096, original_max_position_embeddings=512, eos_token_id=511,
                 rope_scaling={"type": "su", "short_factor": [1.0] * 32,
                               "long_factor": [1.0 + 0.05 * i for i in range(32)]})
TINY_DEEPSEEK = dict(model_type="deepseek_v3", vocab_size=512, hidden_size=256, intermediate_size=512, moe_intermediate_size=128,
                     num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=4, n_shared_experts=1, n_routed_experts=8,
                     routed_scaling_factor=2.5, kv_lora_rank=128, q_lora_rank=128, qk_rope_head_dim=32, v_head_dim=32,
                     qk_nope_head_dim=32, n_group=4, topk_group=2, num_experts_per_tok=2, first_k_dense_replace=1,
                     max_position_embeddings=512, rms_norm_eps=1e-6, rope_theta=10000.0, eos_token_id=511,
                     rope_scaling={"type": "yarn", "factor": 4.0, "original_max_position_embeddings": 128, "beta_fast": 32,
                                   "beta_slow": 1, "mscale": 1.0, "mscale_all_dim": 1.0})
TINY_QWEN3 = dict(model_type="qwen3", hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                  num_key_value_heads=2, head_dim=64, rms_norm_eps=1e-6, vocab_size=512, rope_theta=1000000.0,
                  max_position_embeddings=512, tie_word_embeddings=False, eos_token_id=511)


def strategy_bits(name: str, layer: int, n_layers: int) -> int:
    """S40: all 4-bit.  S22: first/last layer 4-bit, layers 1,2 and n-2 3-bit, else 2-bit."""
    if name == "S40":
        return 4
    if name == "S22":
        if layer in (0, n_layers - 1):
            return 4
        if layer in (1, 2, n_layers - 2):
            return 3
        return 2
    if name == "S30":
        return 3
    if name == "S20":
        return 2
    raise ValueError(f"unknown synthetic strategy {name}")


def make_strategy(name: str, n_layers: int, group_size: int = 128) -> Dict:
    """quant_strategy.json["measurement"] in the reference's schema (quantized_linear_gba.py:256-272)."""
    strat = {}
    for i in range(n_layers):
        b = strategy_bits(name, i, n_layers)
        strat[f"model.layers.{i}"] = {p: {"bits": [b], "group_size": {str(b): group_size}} for p in PROJ}
        for p in ("kv_a_proj_with_mqa", "kv_b_proj", "q_a_proj", "q_b_proj",            # DeepSeek-V3 latent attention
                  "moe_shared_expert_gate_proj", "moe_shared_expert_up_proj", "moe_shared_expert_down_proj"):
            strat[f"model.layers.{i}"][p] = {"bits": [b], "group_size": {str(b): group_size}}
        for p in ("qkv_proj", "gate_up_proj"):      # Phi-3 fused projections; the reference's substring scan reaches them only
            strat[f"model.layers.{i}"][p] = {"bits": [b], "group_size": {str(b): group_size}}   # when v_proj / up_proj are absent
        # stacked experts (QuantizedSwitchLinear): 'moe_expert_<proj>', one step narrower than the dense projections
        be = max(2, b - 1)
        for p in ("gate_proj", "up_proj", "down_proj"):
            strat[f"model.layers.{i}"]["moe_expert_" + p] = {"bits": [be], "group_size": {str(be): group_size}}
    return strat


def _fill_qlinear(m: QuantizedLinear, gen: torch.Generator, device, act_dtype) -> None:
    n, k, b, g = m.output_dims, m.input_dims, m.bits, m.group_size
    words = k // 32 * b
    qw = torch.randint(0, 2**32, (n, words), dtype=torch.int64, device=device, generator=gen).to(torch.int32)
    qmax = float((1 << b) - 1)
    sc = (torch.rand((n, k // g), device=device, generator=gen) + 0.5) * (2.0 / qmax) * 0.02
    ze = -sc * qmax / 2.0 + torch.randn((n, k // g), device=device, generator=gen) * 0.1 * sc
    m._buffers["qweight"] = qw.view(torch.uint32)
    m._buffers["scales"] = sc.to(act_dtype)
    m._buffers["zeros"] = ze.to(act_dtype)
    m._buffers["channel_scale"] = torch.ones((1, 1, k), dtype=torch.float16, device=device)
    if m.bias is not None:
        m._buffers["bias"] = (torch.randn((n,), device=device, generator=gen) * 0.01).to(act_dtype)


def _fill_switch(m: QuantizedSwitchLinear, gen: torch.Generator, device, act_dtype) -> None:
    e, n, k, b, g = m.num_experts, m.output_dims, m.input_dims, m.bits, m.group_size
    qw = torch.randint(0, 2**32, (e, n, k // 32 * b), dtype=torch.int64, device=device, generator=gen).to(torch.int32)
    qmax = float((1 << b) - 1)
    sc = (torch.rand((e, n, k // g), device=device, generator=gen) + 0.5) * (2.0 / qmax) * 0.02
    ze = -sc * qmax / 2.0 + torch.randn((e, n, k // g), device=device, generator=gen) * 0.1 * sc
    m._buffers["qweight"] = qw.view(torch.uint32)
    m._buffers["scales"] = sc.to(act_dtype)
    m._buffers["zeros"] = ze.to(act_dtype)
    if m.bias is not None:
        m._buffers["bias"] = (torch.randn((e, n), device=device, generator=gen) * 0.01).to(act_dtype)


def build_model(config: Dict, strategy: Optional[Dict] = None, device="cpu", seed: int = 0,
                act_dtype=torch.bfloat16, bits: int = 4, group_size: int = 64) -> qllama.Model:
    """Random-init model with real shapes, generated directly on ``device`` (no files)."""
    device = torch.device(device)
    arch = {"qwen3_moe": qqwen3_moe, "qwen3": qqwen3, "qwen2": qqwen2, "mixtral": qmixtral, "phi3": qphi3, "deepseek_v3": qdeepseek_v3}.get(config.get("model_type"), qllama)
    args = arch.ModelArgs.from_dict(config)
    with torch.device("meta"):
        model = arch.Model(args)
    model = model.to_empty(device=device)
    QuantizedLinear.reinit_module(model, group_size=group_size, bits=bits, strategy=strategy)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    for m in model.modules():
        if isinstance(m, QuantizedLinear):
            for nm in list(m._buffers):
                if m._buffers[nm] is not None and m._buffers[nm].device != device:
                    m._buffers[nm] = torch.empty_like(m._buffers[nm], device=device)
            _fill_qlinear(m, gen, device, act_dtype)
        elif isinstance(m, QuantizedSwitchLinear):
            _fill_switch(m, gen, device, act_dtype)
        elif isinstance(m, qllama.RMSNorm):
            m.weight = torch.nn.Parameter(torch.ones(m.weight.shape, dtype=act_dtype, device=device), requires_grad=False)
        elif isinstance(m, torch.nn.Embedding):
            w = torch.randn(m.weight.shape, device=device, generator=gen) * 0.02
            m.weight = torch.nn.Parameter(w.to(act_dtype), requires_grad=False)
        elif isinstance(m, torch.nn.Linear):
            w = torch.randn(m.weight.shape, device=device, generator=gen) * 0.02
            m.weight = torch.nn.Parameter(w.to(act_dtype), requires_grad=False)
        elif isinstance(m, qdeepseek_v3.MoEGate):
            w = torch.randn(m.weight.shape, device=device, generator=gen) * 0.5
            m.weight = torch.nn.Parameter(w.to(act_dtype), requires_grad=False)
            m.e_score_correction_bias = torch.nn.Parameter(torch.randn(m.e_score_correction_bias.shape, device=device,
                                                                       generator=gen) * 0.1, requires_grad=False)
        elif hasattr(m, "inv_freq") and isinstance(getattr(m, "inv_freq"), torch.Tensor):
            pass
    # rope tables are non-persistent buffers created on meta: rebuild them for real
    from .models.rope_utils import initialize_rope
    for blk in model.model.layers:
        at = blk.self_attn
        if hasattr(at, "build_rope"):               # families with their own embedding (Phi-3 su / longrope)
            at.rope = at.build_rope(args).to(device)
            continue
        at.rope = initialize_rope(at.head_dim, args.rope_theta, getattr(args, "rope_traditional", False),
                                  getattr(args, "rope_scaling", None) if arch in (qllama, qqwen2) else None,
                                  args.max_position_embeddings).to(device)
    model.eval()
    return model


def state_dict_for_disk(model: qllama.Model) -> Dict[str, torch.Tensor]:
    """Checkpoint keys exactly as a ``-mlx`` GBA repo stores them."""
    out = {}
    for name, m in model.named_modules():
        if isinstance(m, QuantizedLinear):
            for nm in ("qweight", "scales", "zeros", "bias", "channel_scale"):
                t = getattr(m, nm, None)
                if t is not None:
                    out[f"{name}.{nm}"] = t.detach().cpu().contiguous()
        elif isinstance(m, QuantizedSwitchLinear):
            # on disk the experts are separate modules ``...mlp.experts.<e>.<proj>`` (Model.sanitize stacks them)
            base, proj = name.rsplit(".switch_mlp.", 1)
            if base.endswith("block_sparse_moe"):                   # Mixtral checkpoints call the projections w1 / w2 / w3
                proj = {"gate_proj": "w1", "down_proj": "w2", "up_proj": "w3"}[proj]
            for e in range(m.num_experts):
                for nm in ("qweight", "scales", "zeros"):
                    out[f"{base}.experts.{e}.{proj}.{nm}"] = getattr(m, nm)[e].detach().cpu().contiguous()
        elif isinstance(m, (qllama.RMSNorm, torch.nn.Embedding, torch.nn.Linear)):
            out[f"{name}.weight"] = m.weight.detach().cpu().contiguous()
        elif isinstance(m, qdeepseek_v3.MoEGate):
            out[f"{name}.weight"] = m.weight.detach().cpu().contiguous()
            out[f"{name}.e_score_correction_bias"] = m.e_score_correction_bias.detach().cpu().contiguous()
    return out


def write_tokenizer(path: str, vocab_size: int, eos_token_id: int) -> None:
    """Tiny offline WordLevel tokenizer so that ``load()`` / ``generate(str)`` run end to end."""
    from tokenizers import Tokenizer, models, pre_tokenizers, decoders
    vocab = {f"w{i}": i for i in range(vocab_size)}
    vocab["<eos>"] = eos_token_id
    vocab = {k: v for k, v in vocab.items() if not (k == f"w{eos_token_id}")}
    vocab["hello"], vocab["world"] = vocab.pop("w1"), vocab.pop("w2")
    tok = Tokenizer(models.WordLevel(vocab=vocab, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.decoder = decoders.Fuse()
    tok.save(os.path.join(path, "tokenizer.json"))
    with open(os.path.join(path, "tokenizer_config.json"), "w") as f:
        json.dump({"tokenizer_class": "PreTrainedTokenizerFast", "eos_token": "<eos>", "unk_token": "w0"}, f)


def write_checkpoint(path: str, config: Dict, strategy: Optional[Dict], seed: int = 0,
                     quantization: Optional[Dict] = None, extra_tensors: Optional[Dict] = None) -> qllama.Model:
    """config.json + quant_strategy.json + model.safetensors (+ tokenizer) for ``load(path)``."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    q = quantization or {"group_size": 64, "bits": 4}
    model = build_model(config, strategy, device="cpu", seed=seed, bits=q["bits"], group_size=q["group_size"])
    cfg = dict(config)
    cfg["quantization"] = q
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    if strategy is not None:
        with open(os.path.join(path, "quant_strategy.json"), "w") as f:
            json.dump({"measurement": strategy}, f)
    sd = state_dict_for_disk(model)
    if extra_tensors:
        sd.update(extra_tensors)
    save_file(sd, os.path.join(path, "model.safetensors"))
    write_tokenizer(path, config["vocab_size"], config.get("eos_token_id", config["vocab_size"] - 1))
    return model


# ------------------------------------------------------------------------------------------------ Revitar (dense, ragged steps)
def revitar_config(width: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int, experts: int, top: int, ff: int,
                   n_layers: int, vocab: int = 32000, softcap: float = 30.0, residual_mult: float = 0.5, embed_scale: float = 1.0) -> Dict:
    """config.json of a Revitar model whose layers are all alike (benchmarks; a checkpoint may mix layers freely)."""
    layer = {"type": "attention",
             "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
                       "scale": dim ** -0.5, "softcap": softcap},
             "mlp": {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}}
    return {"architecture": "Revitar", "vocab": vocab, "width": width, "layers": [dict(layer) for _ in range(n_layers)],
            "norm": {"eps": 1e-6}, "residual_mult": residual_mult, "embedding": {"scale": embed_scale}}


def build_revitar(config: Dict, device="cpu", seed: int = 0, act_dtype=torch.bfloat16):
    """Random-init Revitar with real shapes, generated directly on ``device`` (no files)."""
    from .models import revitar
    device = torch.device(device)
    args = revitar.ModelArgs.from_dict(config)
    with torch.device("meta"):
        model = revitar.Model(args)
    model = model.to_empty(device=device)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)

    def rnd(shape, std, dtype):
        return (torch.randn(tuple(shape), device=device, generator=gen) * std).to(dtype)

    for name, p in list(model.named_parameters()):
        mod, _, attr = name.rpartition(".")
        std = 1.0 if "embed_tokens" in name else p.shape[-1] ** -0.5
        dict(model.named_modules())[mod]._parameters[attr] = torch.nn.Parameter(rnd(p.shape, std, act_dtype), requires_grad=False)
    for name, b in list(model.named_buffers()):
        mod, _, attr = name.rpartition(".")
        m = dict(model.named_modules())[mod]
        if attr in ("gate_up", "down"):
            m._buffers[attr] = rnd(b.shape, b.shape[-1] ** -0.5, act_dtype)
        elif attr == "router":
            m._buffers[attr] = rnd(b.shape, 4.0 * b.shape[-1] ** -0.5, torch.float32)
        elif attr in ("dist_mul", "dist_rate"):
            m._buffers[attr] = torch.rand(tuple(b.shape), device=device, generator=gen) * 0.5 + 0.05
        elif attr == "gate_bias":
            m._buffers[attr] = torch.rand(tuple(b.shape), device=device, generator=gen) * 2.0 - 3.0
        else:                                      # norm weights
            m._buffers[attr] = torch.ones(tuple(b.shape), dtype=torch.float32, device=device)
    model.eval()
    return model


# ------------------------------------------------------------------------------------------------ Radenex (dense, parallel layers)
def radenex_config(width: int, latent: Dict, attention: Dict, ff: int, pattern: str = "la", loop=None, vocab: int = 32000) -> Dict:
    """config.json of a Radenex model: ``pattern`` names the layers in order ('l' latent attention, 'a' windowed attention), every
    layer with a dense feed-forward of ``ff`` channels; ``loop`` = (start, stop, times) or None.
    ``latent``: heads, dim, rot_dim, vdim, kv_rank; ``attention``: heads, kv_heads, dim, vdim, window, keep_first."""
    lat = {"type": "latent_attention",
           "mixer": {"heads": latent["heads"], "dim": latent["dim"], "rot_dim": latent["rot_dim"], "vdim": latent["vdim"],
                     "kv_rank": latent["kv_rank"], "scale": (latent["dim"] + latent["rot_dim"]) ** -0.5,
                     "rot": {"base": 10000.0, "dims": latent["rot_dim"],
                             "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}}},
           "mlp": {"kind": "dense", "ff": ff}}
    att = {"type": "attention",
           "mixer": {"heads": attention["heads"], "kv_heads": attention["kv_heads"], "dim": attention["dim"], "vdim": attention["vdim"],
                     "mask": {"size": attention["window"], "keep_first": attention.get("keep_first", 0)}, "scale": attention["dim"] ** -0.5,
                     "rot": {"base": 10000.0, "dims": attention.get("rot_dims", attention["dim"]), "scaling": {"factor": 2.0}}},
           "mlp": {"kind": "dense", "ff": ff}}
    cfg = {"architecture": "Radenex", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
           "layers": [json.loads(json.dumps(lat if c == "l" else att)) for c in pattern]}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def build_radenex(config: Dict, device="cpu", seed: int = 0, act_dtype=torch.bfloat16):
    """Random-init Radenex with real shapes, generated directly on ``device`` (no files)."""
    from .models import radenex
    from .models.sink_attention import LatentAttention
    device = torch.device(device)
    args = radenex.ModelArgs.from_dict(config)
    tables = {}
    model = radenex.Model(args)                   # on the host first: the frequency tables are computed in the constructors
    for name, b in model.named_buffers():
        if name.endswith("freq"):
            tables[name] = b.clone()
    with torch.device("meta"):
        model = radenex.Model(args)
    model = model.to_empty(device=device)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)

    def rnd(shape, std, dtype):
        return (torch.randn(tuple(shape), device=device, generator=gen) * std).to(dtype)

    mods = dict(model.named_modules())
    for name, p in list(model.named_parameters()):
        mod, _, attr = name.rpartition(".")
        std = 1.0 if "embed_tokens" in name else p.shape[-1] ** -0.5
        mods[mod]._parameters[attr] = torch.nn.Parameter(rnd(p.shape, std, act_dtype), requires_grad=False)
    for name, b in list(model.named_buffers()):
        mod, _, attr = name.rpartition(".")
        m = mods[mod]
        if name in tables:
            m._buffers[attr] = tables[name].to(device)
        elif attr == "sink":
            m._buffers[attr] = (torch.rand(tuple(b.shape), device=device, generator=gen) if isinstance(m, LatentAttention)
                                else torch.zeros(tuple(b.shape), device=device))
        elif attr in ("uk_heads", "uv_heads_t"):
            pass                                   # cut from the key / value product below
        else:                                      # norm weights
            m._buffers[attr] = torch.ones(tuple(b.shape), dtype=torch.float32, device=device)
    for m in model.modules():                      # the per-head images are views of the same numbers as the whole-prompt product
        if isinstance(m, LatentAttention):
            h, d, r, dv, rank = m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank
            up = m.up.weight.data
            keys = up[:h * (d + r)].view(h, d + r, rank)
            keys[:, d:] = 0
            m._buffers["uk_heads"] = keys[:, :d].contiguous()
            m._buffers["uv_heads_t"] = up[h * (d + r):].view(h, dv, rank).transpose(1, 2).contiguous()
    model.eval()
    return model


# ------------------------------------------------------------------------------------------------ Tugolix (several streams, recurrent and latent mixers)
def tugolix_config(width: int, delta: Dict, gla: Dict, latent: Dict, ff: int, moe: Dict, pattern: str = "dgls", streams: int = 4,
                   vocab: int = 32000) -> Dict:
    """config.json of a Tugolix model: ``pattern`` names the layers in order ('d' channel-wise delta rule, 'g' gated linear attention,
    'l' latent attention, 's' latent attention over the rows of the nearest 'l' before it); the first layer has the dense
    feed-forward of ``ff`` channels, the others the routed one.  ``delta``: heads, kv_heads, dim, vdim, conv; ``gla``: heads, dim, vdim,
    tau; ``latent``: heads, dim, vdim, kv_rank; ``moe``: experts, top, ff, groups (count, keep), limit, scale."""
    routed = {"kind": "moe", "expert": {"ff": moe["ff"], "limit": moe.get("limit", 7.0)},
              "router": {"experts": moe["experts"], "top": moe["top"], "scale": moe.get("scale", 1.0),
                         "groups": {"count": moe["groups"][0], "keep": moe["groups"][1]}}}
    layers, owner = [], None
    for i, c in enumerate(pattern):
        if c == "d":
            layer = {"type": "channel_delta", "mixer": {k: delta[k] for k in ("heads", "kv_heads", "dim", "vdim", "conv")}}
        elif c == "g":
            layer = {"type": "gla", "mixer": {k: gla[k] for k in ("heads", "dim", "vdim", "tau")}}
        else:
            layer = {"type": "latent_attention", "mixer": dict({k: latent[k] for k in ("heads", "dim", "vdim", "kv_rank")}, scale=latent["dim"] ** -0.5)}
            if c == "s":
                if owner is None:
                    raise ValueError("tugolix_config: 's' needs an 'l' before it")
                layer["mixer"]["kv_from"] = owner
            else:
                owner = i
        layer["mlp"] = {"kind": "dense", "ff": ff} if i == 0 else json.loads(json.dumps(routed))
        layers.append(layer)
    return {"architecture": "Tugolix", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "streams": streams, "logit_scale": 1.0, "layers": layers}


def tugolix_checkpoint(config: Dict, device="cpu", seed: int = 0, decay_rank: int = 64, gate_rank: int = 64, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors in the design's checkpoint names with real shapes, generated directly on ``device``."""
    device = torch.device(device)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    W, s = config["width"], config.get("streams")

    def mat(o, i, mult=1.0):
        return (torch.randn((o, i), device=device, generator=gen) * (mult * i ** -0.5)).to(dtype)

    def vec(n, lo, hi):
        return (torch.rand((n,), device=device, generator=gen) * (hi - lo) + lo).to(dtype)

    w = {"embed": torch.randn((config["vocab"], W), device=device, generator=gen).to(dtype), "final.norm": vec(W, 0.9, 1.1),
         "final.norm.b": vec(W, -0.1, 0.1), "head": mat(config["vocab"], W)}
    for i, layer in enumerate(config["layers"]):
        p, m, kind = f"l{i}.", layer["mixer"], layer["type"]
        for q in (1, 2) if layer.get("mlp") is not None else (1,):
            w[p + f"norm{q}"], w[p + f"norm{q}.b"] = vec(W, 0.9, 1.1), vec(W, -0.1, 0.1)
            if s:
                w[p + f"hc{q}.in"], w[p + f"hc{q}.out"] = vec(s, 0.1, 0.6), vec(s, 0.8, 1.2)
                w[p + f"hc{q}.mix"] = (torch.eye(s, device=device) * 0.9 + torch.randn((s, s), device=device, generator=gen) * 0.05).to(dtype)
        H, d, dv, x = m["heads"], m["dim"], m["vdim"], p + "mix."
        if kind == "gla":
            w[x + "q"], w[x + "k"], w[x + "v"], w[x + "g"] = mat(H * d, W), mat(H * d, W), mat(H * dv, W), mat(H * dv, W)
            w[x + "a1"], w[x + "a2"], w[x + "a2.b"] = mat(decay_rank, W), mat(H * d, decay_rank), vec(H * d, 0.0, 5.0)
            w[x + "norm"], w[x + "o"] = vec(dv, 0.9, 1.1), mat(W, H * dv)
        elif kind == "channel_delta":
            G, taps = m["kv_heads"], m["conv"]
            w[x + "q"], w[x + "k"], w[x + "v"] = mat(G * d, W), mat(G * d, W), mat(H * dv, W)
            for nm, n in (("q", G * d), ("k", G * d), ("v", H * dv)):
                w[x + nm + ".conv"] = (torch.randn((n, taps), device=device, generator=gen) * 0.5 + 0.25).to(dtype)
            w[x + "b"], w[x + "A_log"], w[x + "dt_bias"] = mat(H, W), vec(H, -4.0, 0.0), vec(H * d, -4.0, -1.0)
            w[x + "a1"], w[x + "a2"], w[x + "g1"], w[x + "g2"] = mat(decay_rank, W), mat(H * d, decay_rank), mat(gate_rank, W), mat(H * dv, gate_rank)
            w[x + "norm"], w[x + "o"] = vec(dv, 0.9, 1.1), mat(W, H * dv)
        else:
            R = m["kv_rank"]
            w[x + "q"], w[x + "uk"], w[x + "uv"], w[x + "o"] = mat(H * d, W), mat(H * d, R), mat(H * dv, R), mat(W, H * dv)
            if "kv_from" not in m:
                w[x + "dkv"], w[x + "dkv.norm"] = mat(R, W), vec(R, 0.9, 1.1)
        ff, f = layer.get("mlp"), p + "mlp."
        if ff is not None and ff["kind"] == "dense":
            n = ff["ff"]
            w[f + "gate"], w[f + "up"], w[f + "down"] = mat(n, W), mat(n, W), mat(W, n)
            w[f + "gate.b"], w[f + "up.b"], w[f + "down.b"] = vec(n, -0.1, 0.1), vec(n, -0.1, 0.1), vec(W, -0.1, 0.1)
        elif ff is not None:
            n, E = ff["expert"]["ff"], ff["router"]["experts"]
            w[f + "router"], w[f + "correction"] = mat(E, W, 2.0), vec(E, -0.5, 0.5)
            for e in range(E):
                w[f + f"e{e}.gate"], w[f + f"e{e}.up"], w[f + f"e{e}.down"] = mat(n, W), mat(n, W), mat(W, n)
    return w


def build_tugolix(config: Dict, device="cpu", seed: int = 0, act_dtype=torch.bfloat16, decay_rank: int = 64, gate_rank: int = 64):
    """Random-init Tugolix with real shapes: a random checkpoint generated on ``device`` goes through the model's own ``sanitize``."""
    from .models import tugolix
    from .utils import load_weights
    device = torch.device(device)
    weights = tugolix_checkpoint(config, device, seed, decay_rank, gate_rank)
    args = tugolix.ModelArgs.from_dict(dict(config, shapes=tugolix.Model.shapes_from(weights, config)))
    model = tugolix.Model(args)                   # (the buffers the constructors compute -- rates, empty frequency tables -- are tiny)
    weights = model.sanitize(weights)
    weights = {k: (v.to(act_dtype) if v.is_floating_point() and v.dtype != torch.float32 else v) for k, v in weights.items()}
    with torch.device("meta"):
        model = tugolix.Model(args)
    model = model.to_empty(device=device)
    skipped = load_weights(model, weights, device=device)
    if skipped:
        raise ValueError(f"tensors without a place in the model: {skipped[:3]}")
    model.eval()
    return model


# ------------------------------------------------------------------------------------------------ Laruzen (sandwich norms, token shift, linear-attention and parallel mixers)
def laruzen_config(width: int, gla: Dict, lightning: Dict, left: Dict, right: Dict, ff: int, moe: Dict, pattern: str = "glpg", vocab: int = 32000,
                   pair: Optional[Dict] = None) -> Dict:
    """config.json of a Laruzen model: ``pattern`` names the layers in order ('g' gated linear attention, 'l' lightning attention, 'p' the
    parallel pair of windowed sink attention and a gated linear recurrent unit); the first layer has the dense feed-forward of ``ff``
    channels, the others the routed one.  ``gla``: heads, dim, vdim, tau; ``lightning``: heads, dim, vdim (decays spread over the
    heads); ``left``: heads, kv_heads, dim, vdim, window, rot_dims; ``right``: width, blocks, conv; ``moe``: experts, top, ff, shared."""
    routed = {"kind": "moe", "expert": {"ff": moe["ff"]}, "router": {"experts": moe["experts"], "top": moe["top"]},
              "shared": {"ff": moe["shared"]} if moe.get("shared") else None}
    layers = []
    for i, c in enumerate(pattern):
        if c == "g":
            layer = {"type": "gla", "mixer": {k: gla[k] for k in ("heads", "dim", "vdim", "tau")}}
        elif c == "l":
            h = lightning["heads"]
            layer = {"type": "lightning", "mixer": dict({k: lightning[k] for k in ("heads", "dim", "vdim")},
                                                        decay=[math.exp(-2.0 ** (-1 - 6.0 * j / max(h - 1, 1))) for j in range(h)])}
        elif c == "p":
            l = {"heads": left["heads"], "kv_heads": left["kv_heads"], "dim": left["dim"], "vdim": left["vdim"], "scale": left["dim"] ** -0.5,
                 "mask": {"size": left["window"]},
                 "rot": {"dims": left.get("rot_dims", left["dim"]), "base": 1e6, "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}
            layer = {"type": "parallel", "mixer": {"left": l, "right": {k: right[k] for k in ("width", "blocks", "conv")}}}
        else:
            raise ValueError(f"laruzen_config: unknown layer letter {c!r}")
        layer["mlp"] = {"kind": "dense", "ff": ff} if i == 0 else json.loads(json.dumps(routed))
        layers.append(layer)
    pair = pair if pair is not None else {"buckets": 65521, "mul_prev": 1000003, "mul_cur": 31}
    return {"architecture": "Laruzen", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "embedding": {"bigram": pair}, "layers": layers}


def laruzen_checkpoint(config: Dict, device="cpu", seed: int = 0, decay_rank: int = 16, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors in the design's checkpoint names with real shapes, generated directly on ``device``."""
    device = torch.device(device)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    W = config["width"]

    def mat(o, i, mult=1.0):
        return (torch.randn((o, i), device=device, generator=gen) * (mult * i ** -0.5)).to(dtype)

    def vec(n, lo, hi):
        return (torch.rand((n,), device=device, generator=gen) * (hi - lo) + lo).to(dtype)

    w = {"embed": torch.randn((config["vocab"], W), device=device, generator=gen).to(dtype), "final.norm": vec(W, -0.1, 0.1), "head": mat(config["vocab"], W)}
    pair = (config.get("embedding") or {}).get("bigram")
    if pair:
        w["bigram"] = torch.randn((pair["buckets"] + 1, W), device=device, generator=gen).to(dtype)
    for i, layer in enumerate(config["layers"]):
        p, m, kind = f"l{i}.", layer["mixer"], layer["type"]
        for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if layer.get("mlp") is not None else ()):
            w[p + nm] = vec(W, -0.1, 0.1)
        w[p + "shift"] = vec(W, 0.0, 1.0)
        x = p + "mix."
        if kind in ("gla", "lightning"):
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            w[x + "q"], w[x + "k"], w[x + "v"], w[x + "g"], w[x + "o"] = mat(H * d, W), mat(H * d, W), mat(H * dv, W), mat(H * dv, W), mat(W, H * dv)
            if kind == "gla":
                w[x + "a1"], w[x + "a2"], w[x + "a2.b"], w[x + "norm"] = mat(decay_rank, W), mat(H * d, decay_rank), vec(H * d, 0.0, 5.0), vec(dv, 0.9, 1.1)
            else:
                w[x + "norm"] = vec(H * dv, 0.9, 1.1)
        else:
            l, r = m["left"], m["right"]
            H, G, d, dv = l["heads"], l.get("kv_heads", l["heads"]), l["dim"], l["vdim"]
            a, b = x + "left.", x + "right."
            w[a + "q"], w[a + "k"], w[a + "v"], w[a + "g"], w[a + "o"] = mat(H * d, W), mat(G * d, W), mat(G * dv, W), mat(H * dv, W), mat(W, H * dv)
            w[a + "q.b"], w[a + "k.b"], w[a + "v.b"], w[a + "o.b"] = vec(H * d, -0.1, 0.1), vec(G * d, -0.1, 0.1), vec(G * dv, -0.1, 0.1), vec(W, -0.1, 0.1)
            w[a + "q.norm"], w[a + "k.norm"], w[a + "sink"] = vec(d, 0.9, 1.1), vec(d, 0.9, 1.1), vec(H, -1.0, 1.0)
            C, nb, taps = r["width"], r["blocks"], r["conv"]
            bs = C // nb
            w[b + "x"], w[b + "y"], w[b + "o"], w[b + "x.b"], w[b + "y.b"] = mat(C, W), mat(C, W), mat(W, C), vec(C, -0.1, 0.1), vec(C, -0.1, 0.1)
            w[b + "conv"], w[b + "conv.b"] = (torch.randn((C, taps), device=device, generator=gen) * 0.5 + 0.25).to(dtype), vec(C, -0.1, 0.1)
            for nm in ("ra", "ri"):
                w[b + nm] = (torch.randn((nb, bs, bs), device=device, generator=gen) * bs ** -0.5).to(dtype)
                w[b + nm + ".b"] = (torch.rand((nb, bs), device=device, generator=gen) - 0.5).to(dtype)
            w[b + "lam"] = vec(C, -5.0, 0.0)
            w[x + "left.out"], w[x + "right.out"] = vec(W, 0.9, 1.1), vec(W, 0.9, 1.1)
        ff, f = layer.get("mlp"), p + "mlp."
        if ff is not None and ff["kind"] == "dense":
            n = ff["ff"]
            w[f + "gate"], w[f + "up"], w[f + "down"] = mat(n, W), mat(n, W), mat(W, n)
        elif ff is not None:
            n, E = ff["expert"]["ff"], ff["router"]["experts"]
            w[f + "router"] = mat(E, W, 2.0)
            for e in range(E):
                w[f + f"e{e}.gate"], w[f + f"e{e}.up"], w[f + f"e{e}.down"] = mat(n, W), mat(n, W), mat(W, n)
            if ff.get("shared"):
                s = ff["shared"]["ff"]
                w[f + "shared.gate"], w[f + "shared.up"], w[f + "shared.down"] = mat(s, W), mat(s, W), mat(W, s)
    return w


def build_laruzen(config: Dict, device="cpu", seed: int = 0, act_dtype=torch.bfloat16, decay_rank: int = 16):
    """Random-init Laruzen with real shapes: a random checkpoint generated on ``device`` goes through the model's own ``sanitize``."""
    from .models import laruzen
    from .utils import load_weights
    device = torch.device(device)
    weights = laruzen_checkpoint(config, device, seed, decay_rank)
    args = laruzen.ModelArgs.from_dict(dict(config, shapes=laruzen.Model.shapes_from(weights, config)))
    model = laruzen.Model(args)                   # (the buffers the constructors compute -- rates, frequency tables -- are tiny)
    weights = model.sanitize(weights)
    weights = {k: (v.to(act_dtype) if v.is_floating_point() and v.dtype != torch.float32 else v) for k, v in weights.items()}
    with torch.device("meta"):
        model = laruzen.Model(args)
    model = model.to_empty(device=device)
    skipped = load_weights(model, weights, device=device)
    if skipped:
        raise ValueError(f"tensors without a place in the model: {skipped[:3]}")
    model.eval()
    return model
