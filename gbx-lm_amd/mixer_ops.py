"""Operator wrappers of libgbx_mixers.so: torch tensors in, raw device pointers across the C-ABI (include/gbx_mixers.h).

These are the GPU halves of models/window_attention.py, models/sink_attention.py, models/switch_layers.py:DenseRoutedGLU,
models/feed_forward.py and models/residual.py; each takes
rows of a ragged step (batching.StepBatch).  CPU tensors are refused: the modules run their plain torch graph for those.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib

_DT = {torch.bfloat16: _lib.GBXM_BF16, torch.float32: _lib.GBXM_F32}


def _stream(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _act(t: torch.Tensor, name: str) -> int:
    if not t.is_cuda:
        raise RuntimeError(f"gbx_lm_amd.mixer_ops: `{name}` lives on {t.device}; these operators are HIP kernels only")
    if t.dtype not in _DT:
        raise TypeError(f"gbx_lm_amd.mixer_ops: `{name}` is {t.dtype}; activations are bfloat16 or float32")
    return _DT[t.dtype]


def _f32(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype != torch.float32 or not t.is_contiguous():
        raise TypeError(f"gbx_lm_amd.mixer_ops: `{name}` must be contiguous float32 (it enters 32-bit arithmetic only)")
    return t


def embed_scaled(table: torch.Tensor, tokens: torch.Tensor, scale: float, image: bool = True):
    """(x fp32 [T, W], h in the table's dtype): x = table[tokens] * scale; h is x itself for an fp32 table or when no image is asked
    for (a model whose first layer norms the stream itself)."""
    act = _act(table, "table")
    t, w = tokens.numel(), table.shape[1]
    tokens = tokens.reshape(-1).to(torch.long).contiguous()
    x = torch.empty((t, w), dtype=torch.float32, device=table.device)
    h = x if (table.dtype == torch.float32 or not image) else torch.empty((t, w), dtype=table.dtype, device=table.device)
    _lib.check_mixers(_lib.mixers().gbxm_embed_scaled(table.data_ptr(), tokens.data_ptr(), x.data_ptr(), None if h is x else h.data_ptr(),
                                                     t, w, float(scale), act, _stream(table.device)))
    return x, h


def segment_rmsnorm_(rows: torch.Tensor, n0: int, n1: int, w0: torch.Tensor, w1: torch.Tensor, eps: float) -> None:
    act = _act(rows, "rows")
    if rows.dim() != 2 or rows.stride(1) != 1:
        raise ValueError("segment_rmsnorm_: rows must be [T, N] with unit inner stride")
    if w0.numel() != n0 or w1.numel() != n1:
        raise ValueError("segment_rmsnorm_: one weight per channel of each segment")
    _lib.check_mixers(_lib.mixers().gbxm_segment_rmsnorm(rows.data_ptr(), rows.shape[0], rows.stride(0), n0, n1, _f32(w0, "w0").data_ptr(),
                                                        _f32(w1, "w1").data_ptr(), float(eps), act, _stream(rows.device)))


def residual_norm_add(x: torch.Tensor, branch: torch.Tensor, mix: Optional[torch.Tensor], w: torch.Tensor, eps: float, mult: float,
                      act_dtype: torch.dtype) -> torch.Tensor:
    act = _act(branch, "branch")
    if branch.dtype != act_dtype:
        raise TypeError("residual_norm_add: the branch must be in the activation dtype")
    _f32(x, "x")
    t, width = x.shape
    top = 1 if mix is None else mix.shape[-1]
    branch = branch.contiguous()
    if branch.numel() != t * top * width or w.numel() != width:
        raise ValueError("residual_norm_add: shapes do not fit")
    h = x if act_dtype == torch.float32 else torch.empty((t, width), dtype=act_dtype, device=x.device)
    _lib.check_mixers(_lib.mixers().gbxm_residual_norm_add(x.data_ptr(), branch.data_ptr(), None if mix is None else _f32(mix, "mix").data_ptr(),
                                                          _f32(w, "w").data_ptr(), None if h is x else h.data_ptr(), t, width, top,
                                                          float(eps), float(mult), act, _stream(x.device)))
    return h


def stream_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, act_dtype: torch.dtype) -> torch.Tensor:
    if not x.is_cuda:
        raise RuntimeError("gbx_lm_amd.mixer_ops: stream_rmsnorm is a HIP kernel only")
    x = _f32(x.contiguous(), "x")
    out = torch.empty(x.shape, dtype=act_dtype, device=x.device)
    _lib.check_mixers(_lib.mixers().gbxm_stream_rmsnorm(x.data_ptr(), _f32(w, "w").data_ptr(), out.data_ptr(), x.shape[0], x.shape[1], float(eps),
                                                       _DT[act_dtype], _stream(x.device)))
    return out


def route_topk(h: torch.Tensor, router: torch.Tensor, top: int, renormalize: bool = False):
    """(idx int32 [T, top], weights fp32 [T, top]).  The logits are an fp32 product of the rows (their bf16 image widened, when
    activations are bf16) with the fp32 router -- the vendor library's GEMM / GEMV; softmax and the choice are one launch."""
    _act(h, "h")
    logits = torch.matmul(h if h.dtype == torch.float32 else h.float(), _f32(router, "router").t())
    t, e = logits.shape
    idx = torch.empty((t, top), dtype=torch.int32, device=h.device)
    w = torch.empty((t, top), dtype=torch.float32, device=h.device)
    _lib.check_mixers(_lib.mixers().gbxm_route_topk(logits.data_ptr(), idx.data_ptr(), w.data_ptr(), t, e, top, int(bool(renormalize)),
                                                   _stream(h.device)))
    return idx, w


_GLU = {"silu": 1, "clamped_swish": 2, "gelu_tanh": 3, "sigmoid": 4}


def expert_glu(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, idx: torch.Tensor, activation: str = "silu",
               limit: float = 0.0) -> torch.Tensor:
    act = _act(h, "h")
    h = h.contiguous()
    t, k = h.shape
    e, f2, k2 = gate_up.shape
    f, top = f2 // 2, idx.shape[1]
    if k2 != k or tuple(down.shape) != (e, k, f) or gate_up.dtype != h.dtype or down.dtype != h.dtype or idx.dtype != torch.int32:
        raise ValueError("expert_glu: weights do not fit the rows")
    if not (gate_up.is_contiguous() and down.is_contiguous() and idx.is_contiguous()):
        raise ValueError("expert_glu: contiguous operands")
    y = torch.empty((t, top, k), dtype=h.dtype, device=h.device)
    L = _lib.mixers()
    nbytes = L.gbxm_expert_glu_workspace(t, k, f, e, top, act)
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=h.device) if nbytes else None
    _lib.check_mixers(L.gbxm_expert_glu_act(h.data_ptr(), gate_up.data_ptr(), down.data_ptr(), idx.data_ptr(), y.data_ptr(), t, k, f, e, top, act,
                                            _GLU[activation], float(limit), None if ws is None else ws.data_ptr(), nbytes, _stream(h.device)))
    return y


def window_attention(qkv: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, batch, m) -> torch.Tensor:
    """Context rows [T, heads * vdim] of module ``m`` (models/window_attention.py:GatedWindowAttention) for the step ``batch``; the
    rings hold the positions before the step."""
    act = _act(qkv, "qkv")
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[0] != batch.total:
        raise ValueError("window_attention: qkv must be the step's rows [T, q|k|v]")
    if kcache.dtype != qkv.dtype or vcache.dtype != qkv.dtype or not (kcache.is_contiguous() and vcache.is_contiguous()):
        raise ValueError("window_attention: caches must be contiguous and of the activation dtype")
    if tuple(kcache.shape[1:]) != (m.window, m.nk) or tuple(vcache.shape[1:]) != (m.window, m.nv) or kcache.shape[0] <= max(batch.slot):
        raise ValueError("window_attention: caches do not fit the module or the step's slots")
    out = torch.empty((batch.total, m.heads * m.vdim), dtype=qkv.dtype, device=qkv.device)
    partial, splits = None, 0
    if batch.total * m.kv_heads < 256 and m.window > 128:     # few rows, long windows: room for key-split partial sums
        keys = max(min(m.window, p + n) for p, n in zip(batch.pos0, batch.n_new))      # the longest key range a row of this step has
        splits = min(64, (keys + 63) // 64)
        if splits > 1:
            partial = torch.empty((splits, batch.total, m.heads * m.vdim), dtype=torch.float32, device=qkv.device)
    a = _lib.WindowAttnArgs(qkv.data_ptr(), qkv.stride(0), kcache.data_ptr(), vcache.data_ptr(), batch.seq.data_ptr(), batch.tok.data_ptr(),
                            batch.tiles.data_ptr() if batch.tiles is not None and batch.tiles.numel() else None, out.data_ptr(),
                            _f32(m.dist_mul, "dist_mul").data_ptr(), _f32(m.dist_rate, "dist_rate").data_ptr(),
                            _f32(m.gate_bias, "gate_bias").data_ptr(), batch.total, len(batch.slot),
                            0 if batch.tiles is None else batch.tiles.shape[0], batch.q_tile, m.heads, m.kv_heads, m.dim, m.vdim, m.window,
                            m.scale, m.softcap, int(batch.decode_only), act, None if partial is None else partial.data_ptr(), splits)
    _lib.check_mixers(_lib.mixers().gbxm_window_attention(ctypes.byref(a), _stream(qkv.device)))
    return out


def window_append(qkv: torch.Tensor, nq: int, nk: int, kcache: torch.Tensor, vcache: torch.Tensor, batch, window: int) -> None:
    act = _act(qkv, "qkv")
    nv = qkv.shape[1] - nq - nk
    _lib.check_mixers(_lib.mixers().gbxm_window_append(qkv.data_ptr(), qkv.stride(0), nq, nk, nv, kcache.data_ptr(), vcache.data_ptr(),
                                                      batch.seq.data_ptr(), batch.tok.data_ptr(), batch.total, window, act, _stream(qkv.device)))


# ------------------------------------------------------------------------------- softmax attention with a sink and its row kernels
def stream_add_(x: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    act = _act(a, "a")
    _f32(x, "x")
    if a.shape != x.shape or not a.is_contiguous() or (b is not None and (b.shape != x.shape or b.dtype != a.dtype or not b.is_contiguous())):
        raise ValueError("stream_add_: contiguous branches of the stream's shape and one dtype")
    _lib.check_mixers(_lib.mixers().gbxm_stream_add(x.data_ptr(), a.data_ptr(), None if b is None else b.data_ptr(), x.numel(), act,
                                                   _stream(x.device)))
    return x


def stream_add_norm_(x: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor], w: torch.Tensor, eps: float) -> torch.Tensor:
    """x += a (+ b) in place, returns rms_norm(x) * w in the branches' dtype: one launch for a layer's update and the next layer's norm."""
    act = _act(a, "a")
    _f32(x, "x")
    if x.dim() != 2 or a.shape != x.shape or not a.is_contiguous() or (b is not None and (b.shape != x.shape or b.dtype != a.dtype or not b.is_contiguous())):
        raise ValueError("stream_add_norm_: contiguous branches of the stream's shape and one dtype")
    if w.numel() != x.shape[1]:
        raise ValueError("stream_add_norm_: one norm weight per channel")
    h = torch.empty(x.shape, dtype=a.dtype, device=x.device)
    _lib.check_mixers(_lib.mixers().gbxm_stream_add_norm(x.data_ptr(), a.data_ptr(), None if b is None else b.data_ptr(), _f32(w, "w").data_ptr(),
                                                        h.data_ptr(), x.shape[0], x.shape[1], float(eps), act, _stream(x.device)))
    return h


def head_project(x: torch.Tensor, w: torch.Tensor, n_tail: int = 0) -> torch.Tensor:
    """x [T, H, n_in + n_tail] (unit channel stride), w [H, n_in, n_out] -> [T, H, n_out + n_tail]: every head's own matrix on its
    first n_in channels, the tail copied through.  For the few rows of decode steps (one workgroup per row and head)."""
    act = _act(x, "x")
    t, heads, width = x.shape
    n_in, n_out = w.shape[1], w.shape[2]
    if w.shape[0] != heads or width != n_in + n_tail or x.stride(2) != 1 or w.dtype != x.dtype or not w.is_contiguous():
        raise ValueError("head_project: operands do not fit")
    out = torch.empty((t, heads, n_out + n_tail), dtype=x.dtype, device=x.device)
    _lib.check_mixers(_lib.mixers().gbxm_head_project(x.data_ptr(), x.stride(0), x.stride(1), w.data_ptr(), out.data_ptr(), out.stride(0), out.stride(1),
                                                     t, heads, n_in, n_out, n_tail, act, _stream(x.device)))
    return out


_ACTIVATION = {"relu2": 1, "gelu_tanh": 2}


def activate_(z: torch.Tensor, kind: str) -> torch.Tensor:
    act = _act(z, "z")
    if not z.is_contiguous():
        raise ValueError("activate_: contiguous rows")
    _lib.check_mixers(_lib.mixers().gbxm_activate(z.data_ptr(), z.numel(), _ACTIVATION[kind], act, _stream(z.device)))
    return z


def rotate_norm_heads_(rows: torch.Tensor, positions: torch.Tensor, segments, eps: float) -> None:
    """In place on rows [T, N] (unit inner stride): each ``HeadSegment`` (models/sink_attention.py) rotated and / or normalised."""
    act = _act(rows, "rows")
    if rows.dim() != 2 or rows.stride(1) != 1 or positions.dtype != torch.int32 or positions.dim() != 1 or positions.shape[0] != rows.shape[0]:
        raise ValueError("rotate_norm_heads_: rows [T, N] with unit inner stride and int32 positions [T]")
    segs = (_lib.HeadSegment * len(segments))()
    for c, s in zip(segs, segments):
        if s.offset + s.heads * s.head_dim > rows.shape[1]:
            raise ValueError("rotate_norm_heads_: a segment ends outside the rows")
        if s.rot_dims and s.freq.numel() != s.rot_dims // 2:
            raise ValueError("rotate_norm_heads_: one frequency per rotated pair")
        if s.weight is not None and s.weight.numel() != s.head_dim:
            raise ValueError("rotate_norm_heads_: one weight per channel of the head")
        c.offset, c.heads, c.head_dim, c.rot_offset, c.rot_dims = s.offset, s.heads, s.head_dim, s.rot_offset, s.rot_dims
        c.interleaved, c.norm, c.mult, c.sign = int(s.interleaved), s.norm + (2 if (s.norm and getattr(s, "norm_first", False)) else 0), s.mult, s.sign
        c.freq = _f32(s.freq, "freq").data_ptr() if s.rot_dims else None
        c.weight = _f32(s.weight, "weight").data_ptr() if s.weight is not None else None
    _lib.check_mixers(_lib.mixers().gbxm_rotate_norm_heads(rows.data_ptr(), rows.shape[0], rows.stride(0), positions.data_ptr(), positions.stride(0),
                                                          segs, len(segments), float(eps), act, _stream(rows.device)))


def slot_append(cache, k_rows: torch.Tensor, v_rows: Optional[torch.Tensor], batch) -> None:
    act = _act(k_rows, "k_rows")
    if k_rows.stride(1) != 1 or k_rows.shape[1] != cache.k_width or cache.keys.dtype != k_rows.dtype or cache.keys.shape[0] <= max(batch.slot):
        raise ValueError("slot_append: key rows do not fit the table")
    two = v_rows is not None
    if two != bool(cache.v_width) or (two and (v_rows.stride(1) != 1 or v_rows.shape[1] != cache.v_width)):
        raise ValueError("slot_append: value rows do not fit the table")
    _lib.check_mixers(_lib.mixers().gbxm_slot_append(k_rows.data_ptr(), k_rows.stride(0), cache.k_width, v_rows.data_ptr() if two else None,
                                                    v_rows.stride(0) if two else 0, cache.v_width, cache.keys.data_ptr(),
                                                    cache.values.data_ptr() if two else None, batch.seq.data_ptr(), batch.tok.data_ptr(), batch.total,
                                                    cache.keep, cache.ring, act, _stream(k_rows.device)))


def sink_attention(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor, cache, batch, scale: float, window: Optional[int], keep: int,
                   sink: Optional[torch.Tensor], gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Context rows [T, H * dv]; q [T, H, dk], k_new [T, G, dk], v_new [T, G, dv] views with unit channel stride, gate [T, H] or None;
    ``cache`` (models/cache.py:SlotKVCache, or None for a step without history) holds the positions before the step."""
    act = _act(q, "q")
    t, heads, dk = q.shape
    groups, dv = v_new.shape[1], v_new.shape[2]
    if t != batch.total or k_new.shape != (t, groups, dk) or v_new.shape[0] != t or any(x.stride(2) != 1 or x.dtype != q.dtype for x in (q, k_new, v_new)):
        raise ValueError("sink_attention: q / k / v do not fit the step")
    if sink is not None and sink.numel() != heads:
        raise ValueError("sink_attention: one sink per head")
    if gate is not None and (gate.shape != (t, heads) or gate.stride(1) != 1 or gate.dtype != q.dtype):
        raise ValueError("sink_attention: gate [T, H] in the activation dtype")
    a = _lib.SinkAttnArgs()
    a.q, a.q_row, a.q_head = q.data_ptr(), q.stride(0), q.stride(1)
    a.k_new, a.k_row, a.k_head = k_new.data_ptr(), k_new.stride(0), k_new.stride(1)
    a.v_new, a.v_row, a.v_head = v_new.data_ptr(), v_new.stride(0), v_new.stride(1)
    longest = max(p + n for p, n in zip(batch.pos0, batch.n_new))
    if cache is not None and cache.keys is not None:
        kc, vc = cache.keys, cache.values
        if kc.dtype != q.dtype or kc.shape[0] <= max(batch.slot) or kc.shape[2] < groups * dk or vc.shape[2] < groups * dv:
            raise ValueError("sink_attention: the table does not fit the step")
        if cache.window is None and cache.ring < longest:
            raise ValueError("sink_attention: the table is shorter than the step's longest sequence")
        a.kcache, a.kc_slot, a.kc_row, a.kc_head = kc.data_ptr(), kc.stride(0), kc.stride(1), dk
        a.vcache, a.vc_slot, a.vc_row, a.vc_head = vc.data_ptr(), vc.stride(0), vc.stride(1), dv
        a.keep, a.ring = cache.keep, cache.ring
    else:
        if any(batch.pos0):
            raise ValueError("sink_attention: a step with history needs its table")
        a.keep, a.ring = (keep, window) if window is not None else (0, 1)
    if window is not None and (a.keep != keep or a.ring < window):
        raise ValueError("sink_attention: the table's kept rows / ring do not fit the mask")
    out = torch.empty((t, heads * dv), dtype=q.dtype, device=q.device)
    a.seq, a.tok = batch.seq.data_ptr(), batch.tok.data_ptr()
    a.tiles = batch.tiles.data_ptr() if batch.tiles is not None and batch.tiles.numel() else None
    a.out = out.data_ptr()
    a.sink = _f32(sink, "sink").data_ptr() if sink is not None else None
    if gate is not None:
        a.gate, a.gate_row = gate.data_ptr(), gate.stride(0)
    a.T, a.B, a.n_tiles, a.q_tile = t, len(batch.slot), 0 if batch.tiles is None else batch.tiles.shape[0], batch.q_tile
    a.H, a.G, a.dk, a.dv = heads, groups, dk, dv
    a.window, a.scale = (0 if window is None else int(window)), float(scale)
    a.decode_only, a.act = int(batch.decode_only), act
    partial = None
    if t * groups < 256 and t <= 64:                            # few rows: room for key-split partial sums
        # keys of the longest row; launches that are being captured are replayed for longer sequences: size for the table then
        keys = longest if window is None else min(window + keep, longest)
        if torch.cuda.is_current_stream_capturing() and cache is not None:
            keys = cache.rows
        splits = min(64, (keys + 63) // 64)
        if splits > 1:
            partial = torch.empty((splits, t, heads, (dv + 3) // 4 * 4 + 4), dtype=torch.float32, device=q.device)
            a.partial, a.partial_splits = partial.data_ptr(), splits
    _lib.check_mixers(_lib.mixers().gbxm_sink_attention(ctypes.byref(a), _stream(q.device)))
    return out


# ------------------------------------------------------------------------------- several streams, gated activations, grouped sigmoid router
def hyper_step_(streams: torch.Tensor, y: Optional[torch.Tensor], y_mix: Optional[torch.Tensor], mix: Optional[torch.Tensor],
                write: Optional[torch.Tensor], read: Optional[torch.Tensor], norm, act_dtype: torch.dtype) -> torch.Tensor:
    """models/residual.py:hyper_step_ as one launch.  streams fp32 [T, S, W] contiguous, updated in place."""
    if not streams.is_cuda or streams.dim() != 3:
        raise RuntimeError("gbx_lm_amd.mixer_ops: hyper_step_ takes fp32 device streams [T, S, W]")
    _f32(streams, "streams")
    t, s, width = streams.shape
    top = 1
    if y is not None:
        if y.dtype != act_dtype or not y.is_contiguous():
            raise TypeError("hyper_step_: the sublayer's output must be contiguous and in the activation dtype")
        top = 1 if y_mix is None else y_mix.shape[-1]
        if y.numel() != t * top * width or mix.shape != (s, s) or write.numel() != s:
            raise ValueError("hyper_step_: shapes do not fit")
    if read is not None and read.numel() != s:
        raise ValueError("hyper_step_: one read weight per stream")
    ptr = lambda x, nm: None if x is None else _f32(x, nm).data_ptr()
    h = u = None
    if norm is not None:
        if norm.weight.numel() != width or norm.bias.numel() != width:
            raise ValueError("hyper_step_: one norm weight and bias per channel")
        h = torch.empty((t, width), dtype=act_dtype, device=streams.device)
    else:
        u = torch.empty((t, width), dtype=torch.float32, device=streams.device)
    _lib.check_mixers(_lib.mixers().gbxm_hyper_step(
        streams.data_ptr(), None if y is None else y.data_ptr(), ptr(y_mix, "y_mix"), ptr(mix, "mix"), ptr(write, "write"), ptr(read, "read"),
        None if norm is None else _f32(norm.weight, "norm.weight").data_ptr(), None if norm is None else _f32(norm.bias, "norm.bias").data_ptr(),
        None if h is None else h.data_ptr(), None if u is None else u.data_ptr(), t, s, width, top, 0.0 if norm is None else float(norm.eps),
        _DT[act_dtype], _stream(streams.device)))
    return h if norm is not None else u


def glu(gu: torch.Tensor, kind: str, limit: float = 0.0, alpha: float = 1.702) -> torch.Tensor:
    act = _act(gu, "gu")
    if gu.dim() != 2 or gu.stride(1) != 1 or gu.shape[1] % 2:
        raise ValueError("glu: rows [T, 2F] with unit inner stride")
    t, f = gu.shape[0], gu.shape[1] // 2
    out = torch.empty((t, f), dtype=gu.dtype, device=gu.device)
    _lib.check_mixers(_lib.mixers().gbxm_glu(gu.data_ptr(), gu.stride(0), out.data_ptr(), t, f, _GLU[kind], float(limit), float(alpha), act,
                                            _stream(gu.device)))
    return out


def route_sigmoid_groups(h: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, top: int, groups, renormalize: bool, scale: float):
    """(idx int32 [T, top], weights fp32 [T, top]).  The logits are an fp32 product of the rows (their bf16 image widened, when
    activations are bf16) with the fp32 router (vendor library); scores, groups and the choice are one launch."""
    _act(h, "h")
    logits = torch.matmul(h if h.dtype == torch.float32 else h.float(), _f32(router, "router").t())
    t, e = logits.shape
    idx = torch.empty((t, top), dtype=torch.int32, device=h.device)
    w = torch.empty((t, top), dtype=torch.float32, device=h.device)
    count, keep = groups if groups is not None else (0, 0)
    _lib.check_mixers(_lib.mixers().gbxm_route_sigmoid_groups(logits.data_ptr(), _f32(correction, "correction").data_ptr(), idx.data_ptr(), w.data_ptr(),
                                                             t, e, top, count, keep, int(bool(renormalize)), float(scale), _stream(h.device)))
    return idx, w


# ------------------------------------------------------------------------------- recurrent mixers (models/recurrent_mixers.py)
def recurrent_prepare(y: torch.Tensor, a: Optional[torch.Tensor], lay, decay_bias: Optional[torch.Tensor], decay_rate: torch.Tensor, sign: float,
                      conv: Optional[torch.Tensor], cache, batch, unit: bool, q_scale: float, qkv_silu: bool = False) -> torch.Tensor:
    act = _act(y, "y")
    t = y.shape[0]
    if y.dim() != 2 or y.stride(1) != 1 or t != batch.total or (a is not None and (a.dim() != 2 or a.stride(1) != 1 or a.dtype != y.dtype or a.shape != (t, lay.nd))):
        raise ValueError("recurrent_prepare: projection rows do not fit the step")
    if max(lay.off_q + lay.nq, lay.off_k + lay.nq, lay.off_v + lay.nv, lay.off_beta + lay.heads) > y.shape[1]:
        raise ValueError("recurrent_prepare: the layout ends outside the rows")
    if (a is not None and decay_bias.numel() != lay.nd) or decay_rate.numel() != lay.heads:
        raise ValueError("recurrent_prepare: one decay bias per head and key channel, one rate per head")
    out = torch.empty((t, lay.out_width), dtype=torch.float32, device=y.device)
    p = _lib.RecurrentPrepArgs()
    p.y, p.y_stride = y.data_ptr(), y.stride(0)
    p.a, p.a_stride = (a.data_ptr(), a.stride(0)) if a is not None else (None, 0)
    p.qkv_silu = int(bool(qkv_silu))
    p.conv = p.tail = None
    p.taps = 0
    if conv is not None:
        c = 2 * lay.nq + lay.nv
        if conv.dtype != y.dtype or not conv.is_contiguous() or conv.shape[0] != c:
            raise ValueError("recurrent_prepare: convolution taps [q | k | v channels, taps] in the activation dtype")
        p.conv, p.taps = conv.data_ptr(), conv.shape[1]
        if p.taps > 1:
            tail = cache.tail
            if tail is None or tail.dtype != y.dtype or tuple(tail.shape[1:]) != (p.taps - 1, c) or tail.shape[0] <= max(batch.slot) or not tail.is_contiguous():
                raise ValueError("recurrent_prepare: the cache's tails do not fit the convolution or the step's slots")
            p.tail = tail.data_ptr()
    p.decay_bias = _f32(decay_bias, "decay_bias").data_ptr() if a is not None else None
    p.decay_rate = _f32(decay_rate, "decay_rate").data_ptr()
    p.seq, p.tok, p.out, p.out_stride, p.T = batch.seq.data_ptr(), batch.tok.data_ptr(), out.data_ptr(), out.stride(0), t
    p.H, p.G, p.dk, p.dv = lay.heads, lay.groups, lay.dk, lay.dv
    p.off_q, p.off_k, p.off_v, p.off_beta = lay.off_q, lay.off_k, lay.off_v, lay.off_beta
    p.unit, p.sign, p.q_scale, p.act = int(bool(unit)), float(sign), float(q_scale), act
    _lib.check_mixers(_lib.mixers().gbxm_recurrent_prepare(ctypes.byref(p), _stream(y.device)))
    return out


def conv_tail_update(y: torch.Tensor, channels: int, cache, batch) -> None:
    act = _act(y, "y")
    tail = cache.tail
    if y.stride(1) != 1 or y.shape[1] < channels or tail.dtype != y.dtype or tuple(tail.shape[1:]) != (cache.taps - 1, channels) or tail.shape[0] <= max(batch.slot):
        raise ValueError("conv_tail_update: the cache's tails do not fit the rows or the step's slots")
    _lib.check_mixers(_lib.mixers().gbxm_conv_tail_update(y.data_ptr(), y.stride(0), tail.data_ptr(), batch.seq.data_ptr(), len(batch.slot), channels,
                                                         cache.taps, act, _stream(y.device)))


def decayed_state_scan(r: torch.Tensor, lay, cache, batch, delta: bool) -> torch.Tensor:
    _f32(r, "r")
    state = cache.state
    if not r.is_cuda or r.shape != (batch.total, lay.out_width) or (delta and lay.off_beta < 0):
        raise ValueError("decayed_state_scan: prepared rows do not fit the step")
    if state is None or state.dtype != torch.float32 or tuple(state.shape[1:]) != (lay.heads, lay.dv, lay.dk) or state.shape[0] <= max(batch.slot) or not state.is_contiguous():
        raise ValueError("decayed_state_scan: the cache's states do not fit the mixer or the step's slots")
    out = torch.empty((batch.total, lay.nv), dtype=torch.float32, device=r.device)
    _lib.check_mixers(_lib.mixers().gbxm_state_scan(r.data_ptr(), r.stride(0), state.data_ptr(), out.data_ptr(), batch.seq.data_ptr(), len(batch.slot),
                                                   batch.total, lay.heads, lay.groups, lay.dk, lay.dv, int(bool(delta)), _stream(r.device)))
    return out


def head_norm_gate(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, heads: int, eps: float, kind: int) -> torch.Tensor:
    act = _act(gate, "gate")
    _f32(o, "o")
    t, n = o.shape
    if gate.shape != (t, n) or gate.stride(1) != 1 or n % heads or weight.numel() != n // heads:
        raise ValueError("head_norm_gate: read-outs, gate and weight do not fit")
    out = torch.empty((t, n), dtype=gate.dtype, device=o.device)
    _lib.check_mixers(_lib.mixers().gbxm_head_norm_gate(o.data_ptr(), gate.data_ptr(), gate.stride(0), _f32(weight, "weight").data_ptr(), out.data_ptr(),
                                                       t, heads, n // heads, float(eps), int(kind), act, _stream(o.device)))
    return out


# ------------------------------------------------------------------------------- sandwich-norm layers, token shift, hashed pair embedding
def embed_hashed_pair(table: torch.Tensor, pair: torch.Tensor, tokens: torch.Tensor, batch, state: torch.Tensor, buckets: int, mul_prev: int,
                      mul_cur: int) -> torch.Tensor:
    """models/embedding.py:HashedPairEmbedding as one launch: fp32 [T, W]; ``state`` int64 [slots, 1] holds each sequence's last token."""
    act = _act(table, "table")
    t, w = tokens.numel(), table.shape[1]
    if tokens.dtype != torch.int64 or not tokens.is_contiguous() or t != batch.total:
        raise ValueError("embed_hashed_pair: the step's tokens as contiguous int64")
    if pair.dtype != table.dtype or tuple(pair.shape) != (buckets + 1, w) or not (pair.is_contiguous() and table.is_contiguous()):
        raise ValueError("embed_hashed_pair: the pair table is [buckets + 1, width] in the embedding's dtype")
    if state.dtype != torch.int64 or not state.is_contiguous() or state.shape[0] <= max(batch.slot):
        raise ValueError("embed_hashed_pair: one int64 per slot")
    x = torch.empty((t, w), dtype=torch.float32, device=table.device)
    _lib.check_mixers(_lib.mixers().gbxm_embed_hashed_pair(table.data_ptr(), pair.data_ptr(), tokens.data_ptr(), state.data_ptr(), batch.seq.data_ptr(),
                                                          batch.tok.data_ptr(), x.data_ptr(), t, w, int(buckets), int(mul_prev), int(mul_cur), act,
                                                          _stream(table.device)))
    return x


def norm_token_shift(x: torch.Tensor, w: torch.Tensor, eps: float, shift: torch.Tensor, state: torch.Tensor, batch, act_dtype: torch.dtype) -> torch.Tensor:
    _f32(x, "x")
    if not x.is_cuda or x.dim() != 2 or x.shape[0] != batch.total or w.numel() != x.shape[1] or shift.numel() != x.shape[1]:
        raise ValueError("norm_token_shift: fp32 device rows of the step, one weight and one shift per channel")
    if state.dtype != torch.float32 or not state.is_contiguous() or state.shape[1] != x.shape[1] or state.shape[0] <= max(batch.slot):
        raise ValueError("norm_token_shift: one fp32 row per slot")
    h = torch.empty(x.shape, dtype=act_dtype, device=x.device)
    _lib.check_mixers(_lib.mixers().gbxm_norm_token_shift(x.data_ptr(), _f32(w, "w").data_ptr(), _f32(shift, "shift").data_ptr(), state.data_ptr(),
                                                         batch.seq.data_ptr(), batch.tok.data_ptr(), h.data_ptr(), x.shape[0], x.shape[1], float(eps),
                                                         _DT[act_dtype], _stream(x.device)))
    return h


def branch_norm_add_norm_(x: torch.Tensor, branch: torch.Tensor, mix: Optional[torch.Tensor], extra: Optional[torch.Tensor], w: torch.Tensor, eps: float,
                          next_w: Optional[torch.Tensor], act_dtype: torch.dtype) -> Optional[torch.Tensor]:
    act = _act(branch, "branch")
    _f32(x, "x")
    t, width = x.shape
    top = 1 if mix is None else mix.shape[-1]
    branch = branch.contiguous()
    if branch.dtype != act_dtype or branch.numel() != t * top * width or w.numel() != width:
        raise ValueError("branch_norm_add_norm_: the branch is [T, (top,) W] in the activation dtype")
    if extra is not None and (extra.dtype != act_dtype or extra.shape != (t, width) or not extra.is_contiguous()):
        raise ValueError("branch_norm_add_norm_: the extra branch is contiguous [T, W] in the activation dtype")
    h = None if next_w is None else torch.empty((t, width), dtype=act_dtype, device=x.device)
    _lib.check_mixers(_lib.mixers().gbxm_branch_norm_add_norm(
        x.data_ptr(), branch.data_ptr(), None if mix is None else _f32(mix, "mix").data_ptr(), None if extra is None else extra.data_ptr(),
        _f32(w, "w").data_ptr(), None if next_w is None else _f32(next_w, "next_w").data_ptr(), None if h is None else h.data_ptr(), t, width, top,
        float(eps), act, _stream(x.device)))
    return h


def normed_pair_mean(a: torch.Tensor, b: torch.Tensor, wa: torch.Tensor, wb: torch.Tensor, eps: float) -> torch.Tensor:
    act = _act(a, "a")
    if a.dim() != 2 or b.shape != a.shape or b.dtype != a.dtype or not (a.is_contiguous() and b.is_contiguous()) or wa.numel() != a.shape[1] or wb.numel() != a.shape[1]:
        raise ValueError("normed_pair_mean: two contiguous [T, W] branches of one dtype, a weight per channel each")
    out = torch.empty_like(a)
    _lib.check_mixers(_lib.mixers().gbxm_normed_pair_mean(a.data_ptr(), b.data_ptr(), _f32(wa, "wa").data_ptr(), _f32(wb, "wb").data_ptr(), out.data_ptr(),
                                                         a.shape[0], a.shape[1], float(eps), act, _stream(a.device)))
    return out


def gate_mul(gate: torch.Tensor, up: torch.Tensor, kind: str) -> torch.Tensor:
    act = _act(up, "up")
    if gate.dim() != 2 or gate.shape != up.shape or gate.dtype != up.dtype or gate.stride(1) != 1 or up.stride(1) != 1:
        raise ValueError("gate_mul: rows [T, F] of one dtype with unit inner stride")
    out = torch.empty(up.shape, dtype=up.dtype, device=up.device)
    _lib.check_mixers(_lib.mixers().gbxm_gate_mul(gate.data_ptr(), gate.stride(0), up.data_ptr(), up.stride(0), out.data_ptr(), up.shape[0], up.shape[1],
                                                 _GLU[kind], act, _stream(up.device)))
    return out


# ------------------------------------------------------------------------------- gated linear recurrent unit (models/gated_lru.py)
def causal_conv_rows(x: torch.Tensor, conv: torch.Tensor, bias: Optional[torch.Tensor], cache, batch) -> torch.Tensor:
    act = _act(x, "x")
    t, c = x.shape
    taps = conv.shape[1]
    if x.stride(1) != 1 or t != batch.total or conv.shape[0] != c or conv.dtype != x.dtype or not conv.is_contiguous():
        raise ValueError("causal_conv_rows: rows of the step, taps [C, taps] in the rows' dtype")
    tail = cache.tail if taps > 1 else None
    if taps > 1 and (tail is None or tail.dtype != x.dtype or tuple(tail.shape[1:]) != (taps - 1, c) or tail.shape[0] <= max(batch.slot) or not tail.is_contiguous()):
        raise ValueError("causal_conv_rows: the cache's tails do not fit the convolution or the step's slots")
    out = torch.empty((t, c), dtype=torch.float32, device=x.device)
    _lib.check_mixers(_lib.mixers().gbxm_causal_conv_rows(x.data_ptr(), x.stride(0), conv.data_ptr(), None if bias is None else _f32(bias, "bias").data_ptr(),
                                                         None if tail is None else tail.data_ptr(), batch.seq.data_ptr(), batch.tok.data_ptr(), out.data_ptr(),
                                                         t, c, taps, act, _stream(x.device)))
    return out


def block_gate_logits(u: torch.Tensor, w: torch.Tensor, b: torch.Tensor, w_t_f32: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 logits, element (t, block, o) of the returned tensor (which may be a permuted view).  Few rows: one HIP launch; prompt-sized
    steps: a batched fp32 product of the vendor library over ``w_t_f32`` [blocks, bs, n_out], the fp32 image of ``w`` transposed."""
    act = _act(w, "w")
    _f32(u, "u")
    blocks, n_out, bs = w.shape
    t = u.shape[0]
    if u.shape[1] != blocks * bs or not w.is_contiguous() or tuple(b.shape) != (blocks, n_out):
        raise ValueError("block_gate_logits: operands do not fit")
    if t <= 16 or w_t_f32 is None:
        out = torch.empty((t, blocks, n_out), dtype=torch.float32, device=u.device)
        _lib.check_mixers(_lib.mixers().gbxm_block_gate_logits(u.data_ptr(), w.data_ptr(), _f32(b, "b").data_ptr(), out.data_ptr(), t, blocks, bs, n_out, act,
                                                              _stream(u.device)))
        return out
    if w_t_f32.dtype != torch.float32 or tuple(w_t_f32.shape) != (blocks, bs, n_out):
        raise ValueError("block_gate_logits: the fp32 image is [blocks, bs, n_out]")
    return torch.baddbmm(b.unsqueeze(1), u.view(t, blocks, bs).transpose(0, 1), w_t_f32).transpose(0, 1)


def gated_lru_scan(u: torch.Tensor, logits: torch.Tensor, lam_sp: torch.Tensor, y: torch.Tensor, rate: float, cache, batch) -> torch.Tensor:
    act = _act(y, "y")
    _f32(u, "u")
    t, c = u.shape
    blocks, bs = logits.shape[1], logits.shape[2] // 2
    state = cache.state
    if t != batch.total or logits.dtype != torch.float32 or logits.shape != (t, blocks, 2 * bs) or blocks * bs != c or logits.stride(2) != 1:
        raise ValueError("gated_lru_scan: logits [T, blocks, 2 * block size] in fp32")
    if y.shape != (t, c) or y.stride(1) != 1 or lam_sp.numel() != c:
        raise ValueError("gated_lru_scan: the other branch's rows and one rate per channel")
    if state is None or state.dtype != torch.float32 or state.numel() != state.shape[0] * c or state.shape[0] <= max(batch.slot) or not state.is_contiguous():
        raise ValueError("gated_lru_scan: the cache's states do not fit the unit or the step's slots")
    out = torch.empty((t, c), dtype=y.dtype, device=y.device)
    _lib.check_mixers(_lib.mixers().gbxm_gated_lru_scan(u.data_ptr(), logits.data_ptr(), logits.stride(0), logits.stride(1), _f32(lam_sp, "lam_sp").data_ptr(),
                                                       y.data_ptr(), y.stride(0), state.data_ptr(), out.data_ptr(), batch.seq.data_ptr(), len(batch.slot), t, c, bs,
                                                       float(rate), act, _stream(y.device)))
    return out
