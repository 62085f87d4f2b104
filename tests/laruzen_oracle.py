"""Plain, slow statement of the Laruzen design in float64, one function per mechanism, sharing no code with gbx_lm_amd.  A whole
sequence at a time, token after token where the design recurs: no cache, no batching, no chunking, no fused products.

Notation.  Stream x [T, W].  ``unit(v) = v / sqrt(mean(v^2) + eps)``.  A layer norm of the design is ``unit(v) * (1 + g)`` with the
stored vector g.  Layer:  n = norm1(x);  h_t = n_t + (n_(t-1) - n_t) * shift  (n_(-1) = 0);  x += norm1b(mixer(h));
x += norm2b(ff(norm2(x))).  x_0 = embed[token] + pair[hash(previous token, token)], the pair table's last row for a first token.
logits = head . final_norm(x).
Also here: config builders and a random checkpoint writer (config.json + model.safetensors in the design's tensor names), so that
tests go through the framework's own loader.
"""
import json
import math
import os

import torch

F64 = torch.float64


def unit(v, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def offset_norm(v, g, eps):
    return unit(v, eps) * (1.0 + g)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ------------------------------------------------------------------------------------------------ embedding, token shift
def pair_rows(tokens, buckets, mul_prev, mul_cur):
    rows = []
    for t, tok in enumerate(tokens):
        rows.append(buckets if t == 0 else (tokens[t - 1] * mul_prev + tok * mul_cur) % buckets)
    return rows


def embed(tokens, w, cfg):
    x = w["embed"][tokens]
    pair = (cfg.get("embedding") or {}).get("bigram")
    if pair:
        x = x + w["bigram"][pair_rows(tokens, pair["buckets"], pair["mul_prev"], pair["mul_cur"])]
    return x


def token_shift(n, shift):
    before = torch.cat([torch.zeros_like(n[:1]), n[:-1]])
    return n + (before - n) * shift


# ------------------------------------------------------------------------------------------------ linear-attention mixers
def outer_product_scan(q, k, v, decay):
    """One head.  q, k, decay [T, dk], v [T, dv]:  S_t = diag(decay_t) S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t,  S_(-1) = 0."""
    S = torch.zeros((k.shape[1], v.shape[1]), dtype=F64)
    out = []
    for t in range(k.shape[0]):
        S = decay[t][:, None] * S + torch.outer(k[t], v[t])
        out.append(S.T @ q[t])
    return torch.stack(out)


def gla_mixer(h, w, p, m, eps):
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ w[p + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, d)
    v = (h @ w[p + "v"].T).view(T, H, dv)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = (sigmoid(z) ** (1.0 / m["tau"])).view(T, H, d)
    o = torch.stack([outer_product_scan(q[:, i], k[:, i], v[:, i], alpha[:, i]) for i in range(H)], dim=1)
    o = (unit(o, eps) * w[p + "norm"]).reshape(T, H * dv)
    return (o * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def lightning_mixer(h, w, p, m, eps):
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(h @ w[p + "q"].T).view(T, H, d)
    k = silu(h @ w[p + "k"].T).view(T, H, d)
    v = silu(h @ w[p + "v"].T).view(T, H, dv)
    o = torch.stack([outer_product_scan(q[:, i], k[:, i], v[:, i], torch.full((T, d), float(m["decay"][i]), dtype=F64)) for i in range(H)], dim=1)
    o = unit(o.reshape(T, H * dv), eps) * w[p + "norm"]
    return (o * sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


# ------------------------------------------------------------------------------------------------ windowed attention with a sink
def rotation_table(rot):
    """(frequencies [dims / 2], multiplier of cos and sin)."""
    dims, base = rot["dims"], rot["base"]
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    mult = 1.0
    sc = rot.get("scaling")
    if sc:
        def where(turns):
            return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo, hi = max(math.floor(where(sc["fast"])), 0), min(math.ceil(where(sc["slow"])), dims - 1)
        for i in range(dims // 2):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / sc["factor"] * ramp + f[i] * (1.0 - ramp)
        mult = 0.1 * math.log(sc["factor"]) + 1.0
    return torch.tensor(f, dtype=F64), mult


def rotate_half(v, rot, first_pos=0):
    """v [T, heads, dim]: the first rot.dims channels of every head turn by position * frequency, channel i paired with i + dims / 2."""
    if not rot or not rot.get("dims"):
        return v
    dims = rot["dims"]
    f, mult = rotation_table(rot)
    pos = torch.arange(first_pos, first_pos + v.shape[0], dtype=F64)
    ang = pos[:, None] * f[None, :]
    c, s = (torch.cos(ang) * mult)[:, None, :], (torch.sin(ang) * mult)[:, None, :]
    a, b = v[..., :dims // 2], v[..., dims // 2:dims]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., dims:]], dim=-1)


def sink_softmax_attention(q, k, v, scale, window, sink):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query by query over the keys it sees."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros((T, H, v.shape[2]), dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            first = 0 if window is None else max(0, i - window + 1)
            s = (k[first:i + 1, g] @ q[i, hd]) * scale                      # the visible keys of this query, one score each
            top = max(float(s.max()), float(sink[hd]))
            e = torch.exp(s - top)
            den = e.sum() + math.exp(float(sink[hd]) - top)
            out[i, hd] = (e[:, None] * v[first:i + 1, g]).sum(0) / den
    return out


def window_attention_mixer(h, w, p, m, eps):
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, d)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, d)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, dv)
    q = rotate_half(unit(q, eps) * w[p + "q.norm"], m.get("rot"))
    k = rotate_half(unit(k, eps) * w[p + "k.norm"], m.get("rot"))
    v = unit(v, eps)
    o = sink_softmax_attention(q, k, v, m["scale"], (m.get("mask") or {}).get("size"), w[p + "sink"])
    return (o.reshape(T, H * dv) * sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T + w[p + "o.b"]


# ------------------------------------------------------------------------------------------------ gated linear recurrent unit
def causal_convolution(x, taps_w, bias):
    """x [T, C], taps_w [C, taps]: y[t, c] = bias[c] + sum_j taps_w[c, j] x[t - (taps - 1) + j, c], zeros before the sequence."""
    taps = taps_w.shape[1]
    y = torch.zeros_like(x) + bias
    for t in range(x.shape[0]):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                y[t] += taps_w[:, j] * x[src]
    return y


def block_diagonal(u, mats, bias):
    """u [T, C], mats [blocks, bs, bs] ([out, in] each), bias [blocks, bs] -> [T, C]."""
    blocks, bs, _ = mats.shape
    return torch.cat([u[:, b * bs:(b + 1) * bs] @ mats[b].T + bias[b] for b in range(blocks)], dim=1)


def gated_lru(u, r, i, lam, rate=8.0):
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t,  a_t = exp(-rate r_t softplus(lam)),  S_(-1) = 0."""
    S = torch.zeros(u.shape[1], dtype=F64)
    out = []
    for t in range(u.shape[0]):
        a = torch.exp(-rate * r[t] * softplus(lam))
        S = a * S + torch.sqrt(1.0 - a * a) * (i[t] * u[t])
        out.append(S)
    return torch.stack(out)


def recurrent_block_mixer(h, w, p, m):
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = causal_convolution(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"], w[p + "conv.b"])
    r = sigmoid(block_diagonal(u, w[p + "ra"], w[p + "ra.b"]))
    i = sigmoid(block_diagonal(u, w[p + "ri"], w[p + "ri.b"]))
    return (gated_lru(u, r, i, w[p + "lam"]) * y) @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps):
    left = window_attention_mixer(h, w, p + "left.", m["left"], eps)
    right = recurrent_block_mixer(h, w, p + "right.", m["right"])
    return 0.5 * (unit(left, eps) * w[p + "left.out"] + unit(right, eps) * w[p + "right.out"])


# ------------------------------------------------------------------------------------------------ feed-forwards
def gated_ff(h, w, p, act):
    return (act(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def moe_ff(h, w, p, spec):
    top = spec["router"]["top"]
    logits = h @ w[p + "router"].T
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(logits.shape[1]), key=lambda e: (-float(logits[t, e]), e))[:top]
        z = torch.stack([logits[t, e] for e in order])
        wt = torch.exp(z - z.max())
        wt = wt / wt.sum()
        for j, e in enumerate(order):
            out[t] += wt[j] * gated_ff(h[t:t + 1], w, p + f"e{e}.", silu)[0]
    if spec.get("shared"):
        out = out + gated_ff(h, w, p + "shared.", silu)
    return out


def chosen_experts(h, w, p, top):
    logits = h.to(F64) @ w[p + "router"].to(F64).T
    return [sorted(range(logits.shape[1]), key=lambda e: (-float(logits[t, e]), e))[:top] for t in range(h.shape[0])]


# ------------------------------------------------------------------------------------------------ the model
def forward(cfg, weights, tokens):
    """-> (logits [T, vocab], stream after every layer [layers, T, W]), float64."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = embed(list(tokens), w, cfg)
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = token_shift(offset_norm(x, w[p + "norm1"], eps), w[p + "shift"])
        kind, m = layer["type"], layer["mixer"]
        if kind == "gla":
            y = gla_mixer(h, w, p + "mix.", m, eps)
        elif kind == "lightning":
            y = lightning_mixer(h, w, p + "mix.", m, eps)
        else:
            y = parallel_mixer(h, w, p + "mix.", m, eps)
        x = x + offset_norm(y, w[p + "norm1b"], eps)
        ff = layer.get("mlp")
        if ff is not None:
            h2 = offset_norm(x, w[p + "norm2"], eps)
            z = gated_ff(h2, w, p + "mlp.", gelu_tanh) if ff["kind"] == "dense" else moe_ff(h2, w, p + "mlp.", ff)
            x = x + offset_norm(z, w[p + "norm2b"], eps)
        after.append(x.clone())
    return offset_norm(x, w["final.norm"], eps) @ w["head"].T, torch.stack(after)


# ------------------------------------------------------------------------------------------------ configurations and checkpoints
def gla_layer(heads, dim, vdim, tau, mlp=None):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "mlp": mlp}


def lightning_layer(heads, dim, vdim, decay, mlp=None):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}, "mlp": mlp}


def parallel_layer(heads, kv_heads, dim, vdim, window, rot_dims, lru_width, blocks, conv, scale=None, base=10000.0, scaling=None, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
            "mask": {"size": window}, "rot": {"dims": rot_dims, "base": base, "scaling": scaling}}
    return {"type": "parallel", "mixer": {"left": left, "right": {"width": lru_width, "blocks": blocks, "conv": conv}}, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}, "shared": None if shared is None else {"ff": shared}}


def make_config(layers, vocab=61, width=64, eps=1e-5, pair=(53, 31, 5)):
    cfg = {"architecture": "Laruzen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if pair is not None:
        cfg["embedding"] = {"bigram": {"buckets": pair[0], "mul_prev": pair[1], "mul_cur": pair[2]}}
    return cfg


def make_weights(cfg, seed=0, decay_rank=6, wide_router=False):
    """``wide_router``: router rows are large and far apart, so that the rounding of a token's input rarely changes its experts (whole
    models in bfloat16, where a changed choice in one layer changes the recurrent state of every later token)."""
    gen = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    bf = torch.bfloat16

    def mat(o, i, scale=1.0):
        return (torch.randn((o, i), generator=gen) * scale / math.sqrt(i)).to(bf)

    def vec(n, lo, hi):
        return (torch.rand((n,), generator=gen) * (hi - lo) + lo).to(bf)

    w = {"embed": torch.randn((cfg["vocab"], W), generator=gen).to(bf), "final.norm": vec(W, -0.4, 0.4), "head": mat(cfg["vocab"], W)}
    pair = (cfg.get("embedding") or {}).get("bigram")
    if pair:
        w["bigram"] = torch.randn((pair["buckets"] + 1, W), generator=gen).to(bf)
    for i, layer in enumerate(cfg["layers"]):
        p, m, kind = f"l{i}.", layer["mixer"], layer["type"]
        for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if layer.get("mlp") is not None else ()):
            w[p + nm] = vec(W, -0.4, 0.4)
        w[p + "shift"] = vec(W, -0.2, 1.1)
        x = p + "mix."
        if kind in ("gla", "lightning"):
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            w[x + "q"], w[x + "k"], w[x + "v"], w[x + "g"], w[x + "o"] = mat(H * d, W), mat(H * d, W), mat(H * dv, W), mat(H * dv, W), mat(W, H * dv)
            if kind == "gla":
                w[x + "a1"], w[x + "a2"], w[x + "a2.b"] = mat(decay_rank, W), mat(H * d, decay_rank, 2.0), vec(H * d, -1.0, 5.0)
                w[x + "norm"] = vec(dv, 0.5, 1.5)
            else:
                w[x + "norm"] = vec(H * dv, 0.5, 1.5)
        else:
            l, r = m["left"], m["right"]
            H, G, d, dv = l["heads"], l.get("kv_heads", l["heads"]), l["dim"], l["vdim"]
            a = x + "left."
            w[a + "q"], w[a + "k"], w[a + "v"], w[a + "g"], w[a + "o"] = mat(H * d, W), mat(G * d, W), mat(G * dv, W), mat(H * dv, W), mat(W, H * dv)
            w[a + "q.b"], w[a + "k.b"], w[a + "v.b"], w[a + "o.b"] = vec(H * d, -0.3, 0.3), vec(G * d, -0.3, 0.3), vec(G * dv, -0.3, 0.3), vec(W, -0.3, 0.3)
            w[a + "q.norm"], w[a + "k.norm"], w[a + "sink"] = vec(d, 0.5, 1.5), vec(d, 0.5, 1.5), vec(H, -1.0, 2.0)
            b = x + "right."
            C, nb, taps = r["width"], r["blocks"], r["conv"]
            bs = C // nb
            w[b + "x"], w[b + "y"], w[b + "o"] = mat(C, W), mat(C, W), mat(W, C)
            w[b + "x.b"], w[b + "y.b"] = vec(C, -0.3, 0.3), vec(C, -0.3, 0.3)
            w[b + "conv"], w[b + "conv.b"] = (torch.randn((C, taps), generator=gen) * 0.6 + 0.25).to(bf), vec(C, -0.2, 0.2)
            w[b + "ra"] = (torch.randn((nb, bs, bs), generator=gen) / math.sqrt(bs)).to(bf)
            w[b + "ri"] = (torch.randn((nb, bs, bs), generator=gen) / math.sqrt(bs)).to(bf)
            w[b + "ra.b"], w[b + "ri.b"] = (torch.rand((nb, bs), generator=gen) * 2 - 1).to(bf), (torch.rand((nb, bs), generator=gen) * 2 - 1).to(bf)
            w[b + "lam"] = vec(C, -6.0, 1.0)
            w[x + "left.out"], w[x + "right.out"] = vec(W, 0.5, 1.5), vec(W, 0.5, 1.5)
        ff = layer.get("mlp")
        f = p + "mlp."
        if ff is not None and ff["kind"] == "dense":
            n = ff["ff"]
            w[f + "gate"], w[f + "up"], w[f + "down"] = mat(n, W), mat(n, W), mat(W, n)
        elif ff is not None:
            n, E = ff["expert"]["ff"], ff["router"]["experts"]
            w[f + "router"] = mat(E, W, 6.0 if wide_router else 1.5)
            for e in range(E):
                w[f + f"e{e}.gate"], w[f + f"e{e}.up"], w[f + f"e{e}.down"] = mat(n, W, 1.5), mat(n, W, 1.5), mat(W, n)
            if ff.get("shared"):
                s = ff["shared"]["ff"]
                w[f + "shared.gate"], w[f + "shared.up"], w[f + "shared.down"] = mat(s, W), mat(s, W), mat(W, s)
    return w


def save_checkpoint(folder, cfg, weights):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def row_errors(got, want):
    """Root mean square of the difference over that of the reference, per row."""
    got, want = got.to(F64).cpu(), want.to(F64).cpu()
    return (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-12)


def rel_err(got, want):
    """The worst row's error."""
    return float(row_errors(got, want).max())


def rel_err_most(got, want, share=0.9):
    """The error that ``share`` of the rows stay under (whole models in bfloat16: a router whose candidates lie closer than the
    rounding of its input may choose another expert, and that row then differs by a whole expert)."""
    e = row_errors(got, want).flatten().sort().values
    return float(e[min(int(math.ceil(share * e.numel())) - 1, e.numel() - 1)])
