"""Plain, slow statement of the Tugolix design in float64, one function per mechanism, sharing no code with gbx_lm_amd.  A whole
sequence at a time, token after token where the design recurs: no cache, no batching, no chunking, no fused products.

Notation: ``s`` residual streams X [T, s, W] (all equal to the embedding at the start).  Sublayer q of a layer (1 mixer, 2
feed-forward) with vectors a_q (read), b_q (write) and matrix M_q [from, to]:
    u = sum_i a_q[i] X_i,   y = sublayer(LN(u)),   X_j <- sum_i M_q[i, j] X_i + b_q[j] y      (all j at once)
LN is a layer norm with weight and bias.  logits = logit_scale * head . LN_final(sum_i X_i).  Without 'streams' in the config
the layer is the plain pre-norm residual x <- x + sublayer(LN(x)).
Also here: a random checkpoint writer (config.json + model.safetensors in the design's tensor names), so that tests go through
the framework's own loader.
"""
import json
import math
import os

import torch

F64 = torch.float64


def rms(y, eps, w=None):
    y = y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def layer_norm(x, w, b, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * w + b


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ------------------------------------------------------------------------------------------------ recurrent mixers
def short_convolution(x, taps_w):
    """x [T, C], taps_w [C, taps]: y[t, c] = sum_j taps_w[c, j] x[t - (taps - 1) + j, c], zeros before the sequence."""
    T, C = x.shape
    taps = taps_w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                y[t] += taps_w[:, j] * x[src]
    return y


def decayed_outer_scan(q, k, v, decay):
    """One head of gated linear attention.  q, k, decay [T, dk], v [T, dv]:  S_t = diag(decay_t) S_{t-1} + k_t v_t^T,  o_t = S_t^T q_t."""
    T, dk = k.shape
    S = torch.zeros((dk, v.shape[1]), dtype=F64)
    out = []
    for t in range(T):
        S = decay[t][:, None] * S + torch.outer(k[t], v[t])
        out.append(S.T @ q[t])
    return torch.stack(out)


def decayed_delta_scan(q, k, v, decay, beta):
    """One head of the gated delta rule.  Per token: S <- diag(decay) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T, dk = k.shape
    S = torch.zeros((dk, v.shape[1]), dtype=F64)
    out = []
    for t in range(T):
        S = decay[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out)


def gla_mixer(h, w, p, m, eps):
    H, d, dv, tau = m["heads"], m["dim"], m["vdim"], m["tau"]
    T = h.shape[0]
    q = (h @ w[p + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, d)
    v = (h @ w[p + "v"].T).view(T, H, dv)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = (sigmoid(z) ** (1.0 / tau)).view(T, H, d)
    o = torch.stack([decayed_outer_scan(q[:, i], k[:, i], v[:, i], alpha[:, i]) for i in range(H)], dim=1)     # [T, H, dv]
    o = rms(o, eps, w[p + "norm"]).reshape(T, H * dv)
    return (o * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def channel_delta_mixer(h, w, p, m, eps):
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(short_convolution(h @ w[p + "q"].T, w[p + "q.conv"])).view(T, G, d)
    k = silu(short_convolution(h @ w[p + "k"].T, w[p + "k.conv"])).view(T, G, d)
    v = silu(short_convolution(h @ w[p + "v"].T, w[p + "v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = sigmoid(h @ w[p + "b"].T)                                                   # [T, H]
    a = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]
    decay = torch.exp(-torch.exp(w[p + "A_log"])[None, :, None] * softplus(a).view(T, H, d))
    rep = H // G
    o = torch.stack([decayed_delta_scan(q[:, i // rep], k[:, i // rep], v[:, i], decay[:, i], beta[:, i]) for i in range(H)], dim=1)
    gate = sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).view(T, H, dv)
    o = rms(o, eps, w[p + "norm"]) * gate
    return o.reshape(T, H * dv) @ w[p + "o"].T


# ------------------------------------------------------------------------------------------------ latent attention
def latent_rows(h, w, p, eps):
    return rms(h @ w[p + "dkv"].T, eps, w[p + "dkv.norm"])


def latent_attention_mixer(h, w, p, m, latent):
    """``latent`` [T, kv_rank]: this layer's own rows, or those of the layer named by 'kv_from'."""
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ w[p + "q"].T).view(T, H, d)
    k = (latent @ w[p + "uk"].T).view(T, H, d)
    v = (latent @ w[p + "uv"].T).view(T, H, dv)
    out = torch.zeros((T, H, dv), dtype=F64)
    for i in range(T):
        for a in range(H):
            s = (k[:i + 1, a] @ q[i, a]) * m["scale"]
            e = torch.exp(s - s.max())
            out[i, a] = (e / e.sum()) @ v[:i + 1, a]
    return out.reshape(T, H * dv) @ w[p + "o"].T


# ------------------------------------------------------------------------------------------------ feed-forwards
def dense_ff(h, w, p):
    g = h @ w[p + "gate"].T + w[p + "gate.b"]
    u = h @ w[p + "up"].T + w[p + "up.b"]
    return (silu(g) * u) @ w[p + "down"].T + w[p + "down.b"]


def clamped_expert(h, w, p, limit):
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def grouped_choice(s, correction, top, groups):
    """One token.  s [E] scores; returns the chosen experts (ties: the lower index).  The choice runs on s + correction; experts
    outside the best groups (group score: sum of its two largest choice scores) cannot be chosen."""
    c = s + correction
    E = c.shape[0]
    allowed = torch.ones(E, dtype=torch.bool)
    if groups:
        n, keep = groups["count"], groups["keep"]
        size = E // n
        gs = torch.stack([torch.sort(c[g * size:(g + 1) * size], descending=True).values[:2].sum() for g in range(n)])
        order = sorted(range(n), key=lambda g: (-float(gs[g]), g))[:keep]
        allowed[:] = False
        for g in order:
            allowed[g * size:(g + 1) * size] = True
    ranked = sorted((e for e in range(E) if allowed[e]), key=lambda e: (-float(c[e]), e))
    return ranked[:top]


def moe_ff(h, w, p, spec):
    r, limit = spec["router"], spec["expert"]["limit"]
    s = sigmoid(h @ w[p + "router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = grouped_choice(s[t], w[p + "correction"], r["top"], r.get("groups"))
        weights = s[t][chosen] / (s[t][chosen].sum() + 1e-20) * r["scale"]
        for e, g in zip(chosen, weights):
            out[t] += g * clamped_expert(h[t:t + 1], w, f"{p}e{e}.", limit)[0]
    return out


# ------------------------------------------------------------------------------------------------ the model
def forward(cfg, weights, tokens):
    """tokens: list of ids.  Returns (logits [T, vocab], sum of the streams after every layer [L, T, W]), float64."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps, s = cfg["norm"]["eps"], cfg.get("streams")
    x = w["embed"][torch.tensor(tokens)]
    T, W = x.shape
    X = x[:, None, :].repeat(1, s or 1, 1)
    latents, after = {}, []

    def sublayer(X, i, q, fn):
        p = f"l{i}."
        if s:
            a, b, M = w[p + f"hc{q}.in"], w[p + f"hc{q}.out"], w[p + f"hc{q}.mix"]
        else:
            a, b, M = torch.ones(1, dtype=F64), torch.ones(1, dtype=F64), torch.ones((1, 1), dtype=F64)
        u = (a[None, :, None] * X).sum(1)
        y = fn(layer_norm(u, w[p + f"norm{q}"], w[p + f"norm{q}.b"], eps))
        return torch.einsum("ij,tiw->tjw", M, X) + b[None, :, None] * y[:, None, :]

    for i, layer in enumerate(cfg["layers"]):
        p, m, kind = f"l{i}.mix.", layer["mixer"], layer["type"]
        if kind == "gla":
            mix = lambda h: gla_mixer(h, w, p, m, eps)
        elif kind == "channel_delta":
            mix = lambda h: channel_delta_mixer(h, w, p, m, eps)
        elif kind == "latent_attention":
            def mix(h):
                if "kv_from" in m:
                    c = latents[m["kv_from"]]
                else:
                    c = latents[i] = latent_rows(h, w, p, eps)
                return latent_attention_mixer(h, w, p, m, c)
        else:
            raise ValueError(kind)
        X = sublayer(X, i, 1, mix)
        spec = layer.get("mlp")
        if spec is not None:
            ff = (lambda h: dense_ff(h, w, f"l{i}.mlp.")) if spec["kind"] == "dense" else (lambda h: moe_ff(h, w, f"l{i}.mlp.", spec))
            X = sublayer(X, i, 2, ff)
        after.append(X.sum(1))
    logits = layer_norm(X.sum(1), w["final.norm"], w["final.norm.b"], eps) @ w["head"].T * cfg.get("logit_scale", 1.0)
    return logits, torch.stack(after)


# ------------------------------------------------------------------------------------------------ configurations and checkpoints
def gla_layer(heads, dim, vdim, tau, mlp=None):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "mlp": mlp}


def delta_layer(heads, kv_heads, dim, vdim, conv, mlp=None):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def latent_layer(heads, dim, vdim, kv_rank, scale=None, kv_from=None, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale if scale is not None else dim ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit=1.0, groups=None, scale=1.0):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": r}


def make_config(layers, vocab=61, width=64, eps=1e-5, streams=3, logit_scale=1.0):
    cfg = {"architecture": "Tugolix", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps}, "logit_scale": logit_scale}
    if streams:
        cfg["streams"] = streams
    return cfg


def make_weights(cfg, seed=0, decay_rank=6, gate_rank=5, steady_router=False):
    """``steady_router``: the corrections are distinct powers of two (times -1/8: all sums of two differ by 1/8 or more) and the
    router matrix is small, so that no rounding of a token's input can change its groups or experts (for whole models in bfloat16,
    where a changed choice in one layer would change the recurrent state of every later token)."""
    gen = torch.Generator().manual_seed(seed)
    W, s = cfg["width"], cfg.get("streams")
    bf = torch.bfloat16

    def mat(o, i, scale=1.0):
        return (torch.randn((o, i), generator=gen) * scale / math.sqrt(i)).to(bf)

    def vec(n, lo, hi):
        return (torch.rand((n,), generator=gen) * (hi - lo) + lo).to(bf)

    w = {"embed": torch.randn((cfg["vocab"], W), generator=gen).to(bf), "final.norm": vec(W, 0.5, 1.5), "final.norm.b": vec(W, -0.3, 0.3),
         "head": mat(cfg["vocab"], W)}
    for i, layer in enumerate(cfg["layers"]):
        p, m, kind = f"l{i}.", layer["mixer"], layer["type"]
        for q in (1, 2) if layer.get("mlp") is not None else (1,):
            w[p + f"norm{q}"], w[p + f"norm{q}.b"] = vec(W, 0.5, 1.5), vec(W, -0.3, 0.3)
            if s:
                w[p + f"hc{q}.in"], w[p + f"hc{q}.out"] = vec(s, 0.1, 0.7), vec(s, 0.7, 1.3)
                w[p + f"hc{q}.mix"] = (torch.eye(s) * 0.8 + torch.randn((s, s), generator=gen) * 0.2).to(bf)
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        x = p + "mix."
        if kind == "gla":
            w[x + "q"], w[x + "k"], w[x + "v"], w[x + "g"] = mat(H * d, W), mat(H * d, W), mat(H * dv, W), mat(H * dv, W)
            w[x + "a1"], w[x + "a2"], w[x + "a2.b"] = mat(decay_rank, W), mat(H * d, decay_rank, 2.0), vec(H * d, -1.0, 5.0)
            w[x + "norm"], w[x + "o"] = vec(dv, 0.5, 1.5), mat(W, H * dv)
        elif kind == "channel_delta":
            G, taps = m["kv_heads"], m["conv"]
            w[x + "q"], w[x + "k"], w[x + "v"] = mat(G * d, W), mat(G * d, W), mat(H * dv, W)
            for nm, n in (("q", G * d), ("k", G * d), ("v", H * dv)):
                w[x + nm + ".conv"] = (torch.randn((n, taps), generator=gen) * 0.7 + 0.25).to(bf)
            w[x + "b"], w[x + "A_log"], w[x + "dt_bias"] = mat(H, W, 2.0), vec(H, -4.0, 0.0), vec(H * d, -4.0, -1.0)
            w[x + "a1"], w[x + "a2"] = mat(decay_rank, W), mat(H * d, decay_rank, 2.0)
            w[x + "g1"], w[x + "g2"] = mat(gate_rank, W), mat(H * dv, gate_rank, 2.0)
            w[x + "norm"], w[x + "o"] = vec(dv, 0.5, 1.5), mat(W, H * dv)
        else:
            R = m["kv_rank"]
            w[x + "q"], w[x + "uk"], w[x + "uv"], w[x + "o"] = mat(H * d, W), mat(H * d, R), mat(H * dv, R), mat(W, H * dv)
            if "kv_from" not in m:
                w[x + "dkv"], w[x + "dkv.norm"] = mat(R, W, 2.0), vec(R, 0.5, 1.5)
        ff = layer.get("mlp")
        f = p + "mlp."
        if ff is not None and ff["kind"] == "dense":
            n = ff["ff"]
            w[f + "gate"], w[f + "up"], w[f + "down"] = mat(n, W), mat(n, W), mat(W, n)
            w[f + "gate.b"], w[f + "up.b"], w[f + "down.b"] = vec(n, -0.3, 0.3), vec(n, -0.3, 0.3), vec(W, -0.3, 0.3)
        elif ff is not None:
            n, E = ff["expert"]["ff"], ff["router"]["experts"]
            w[f + "router"], w[f + "correction"] = mat(E, W, 1.5), vec(E, -1.5, -0.5)
            if steady_router:
                w[f + "router"] = mat(E, W, 0.1)
                w[f + "correction"] = (-0.125 * 2.0 ** torch.randperm(E, generator=gen).float()).to(bf)
            for e in range(E):
                w[f + f"e{e}.gate"], w[f + f"e{e}.up"], w[f + f"e{e}.down"] = mat(n, W, 1.5), mat(n, W, 1.5), mat(W, n)
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
    """The error that ``share`` of the rows stay under.  For whole models in bfloat16: a router whose two candidates lie closer than
    the rounding of its input may choose the other one, and that row then differs by a whole expert."""
    e = row_errors(got, want).flatten().sort().values
    return float(e[min(int(math.ceil(share * e.numel())) - 1, e.numel() - 1)])
