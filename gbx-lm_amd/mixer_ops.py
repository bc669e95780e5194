"""Operator wrappers of libgbx_mixers.so: torch tensors in, raw device pointers across the C-ABI (include/gbx_mixers.h).

These are the GPU halves of models/window_attention.py, models/switch_layers.py:DenseRoutedGLU and models/residual.py; each takes
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


def embed_scaled(table: torch.Tensor, tokens: torch.Tensor, scale: float):
    """(x fp32 [T, W], h in the table's dtype): x = table[tokens] * scale; h is x itself for an fp32 table."""
    act = _act(table, "table")
    t, w = tokens.numel(), table.shape[1]
    tokens = tokens.reshape(-1).to(torch.long).contiguous()
    x = torch.empty((t, w), dtype=torch.float32, device=table.device)
    h = x if table.dtype == torch.float32 else torch.empty((t, w), dtype=table.dtype, device=table.device)
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


def expert_glu(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
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
    _lib.check_mixers(L.gbxm_expert_glu(h.data_ptr(), gate_up.data_ptr(), down.data_ptr(), idx.data_ptr(), y.data_ptr(), t, k, f, e, top, act,
                                        None if ws is None else ws.data_ptr(), nbytes, _stream(h.device)))
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
