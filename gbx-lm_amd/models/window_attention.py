"""Sliding-window attention with independent (unnormalised) key gates, for ragged step batches.

The mechanism, with all of its constants as parameters:

* one fused projection ``q | k | v``; q and k are each RMS-normalised over their WHOLE projection row (all heads at once, one
  weight per channel) before the split into heads;
* no rotation: a position enters only through the window and a logarithmic distance penalty;
* score  s_ij = cap * tanh(scale * <q_i, k_j> / cap) - a_h * log(1 + b_h * (i - j))      (cap <= 0: no soft cap)
* gate   g_ij = sigmoid(s_ij + c_h)   for 0 <= i - j < window, else 0   -- every visible key is gated on its own, the gates of a
  query are not normalised over its keys;
* output o_i = sum_j g_ij v_j per head (query head h reads key / value head h // (heads / kv_heads)), then the output projection.

Scores, gates and the two norms are 32-bit whatever the activation dtype is.  On the GPU the step runs as HIP launches
(``mixer_ops``): norm of both segments, attention over (ring cache | the step's own rows), append; CPU tensors take the plain
torch graph below, which is also what the kernels are tested against.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn

from .cache import WindowKVCache


def segment_rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm over the whole last axis in fp32, result in x's dtype."""
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(x.dtype)


class GatedWindowAttention(nn.Module):
    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int, scale: float,
                 softcap: float = 0.0, eps: float = 1e-6):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.width, self.heads, self.kv_heads, self.dim, self.vdim = width, heads, kv_heads, dim, vdim
        self.window, self.scale, self.softcap, self.eps = int(window), float(scale), float(softcap or 0.0), float(eps)
        self.nq, self.nk, self.nv = heads * dim, kv_heads * dim, kv_heads * vdim
        self.qkv = nn.Linear(width, self.nq + self.nk + self.nv, bias=False)
        self.o = nn.Linear(heads * vdim, width, bias=False)
        self.register_buffer("q_norm", torch.ones(self.nq))
        self.register_buffer("k_norm", torch.ones(self.nk))
        self.register_buffer("dist_mul", torch.zeros(heads))       # a_h
        self.register_buffer("dist_rate", torch.zeros(heads))      # b_h
        self.register_buffer("gate_bias", torch.zeros(heads))      # c_h
        for p in self.parameters():
            p.requires_grad_(False)

    def make_cache(self, slots) -> WindowKVCache:
        return WindowKVCache(self.window, slots)

    # ------------------------------------------------------------------------------------------ plain torch graph
    def _attend_torch(self, q, k_new, v_new, cache: WindowKVCache, slot: int, pos0: int) -> torch.Tensor:
        n, w = q.shape[0], self.window
        old = min(pos0, w - 1)                                     # rows of the ring a query of this step can still see
        if old:
            rows = torch.arange(pos0 - old, pos0, device=q.device) % w
            k = torch.cat([cache.keys[slot, rows], k_new])
            v = torch.cat([cache.values[slot, rows], v_new])
        else:
            k, v = k_new, v_new
        qi = torch.arange(pos0, pos0 + n, device=q.device)[:, None]
        kj = torch.arange(pos0 - old, pos0 + n, device=q.device)[None, :]
        dist = qi - kj
        seen = (dist >= 0) & (dist < w)
        qh = q.float().view(n, self.heads, self.dim).transpose(0, 1)
        rep = self.heads // self.kv_heads
        kh = k.float().view(-1, self.kv_heads, self.dim).transpose(0, 1).repeat_interleave(rep, 0)
        vh = v.float().view(-1, self.kv_heads, self.vdim).transpose(0, 1).repeat_interleave(rep, 0)
        s = torch.matmul(qh, kh.transpose(1, 2)) * self.scale
        if self.softcap > 0:
            s = self.softcap * torch.tanh(s / self.softcap)
        d = dist.clamp(min=0).float()[None]
        s = s - self.dist_mul.float()[:, None, None] * torch.log1p(self.dist_rate.float()[:, None, None] * d)
        g = torch.sigmoid(s + self.gate_bias.float()[:, None, None]) * seen[None]
        return torch.matmul(g, vh).transpose(0, 1).reshape(n, self.heads * self.vdim).to(q.dtype)

    def forward(self, h: torch.Tensor, batch, cache: WindowKVCache) -> torch.Tensor:
        """h [T, width] (the step's rows back to back) -> [T, width]; the step's keys / values are in ``cache`` afterwards."""
        qkv = F.linear(h, self.qkv.weight)
        cache.reserve(qkv[:, self.nq:self.nq + self.nk], qkv[:, self.nq + self.nk:])
        if h.is_cuda:
            from .. import mixer_ops as M
            M.segment_rmsnorm_(qkv, self.nq, self.nk, self.q_norm, self.k_norm, self.eps)
            ctx = M.window_attention(qkv, cache.keys, cache.values, batch, self)
            M.window_append(qkv, self.nq, self.nk, cache.keys, cache.values, batch, self.window)
        else:
            q = segment_rms_norm(qkv[:, :self.nq], self.q_norm, self.eps)
            k = segment_rms_norm(qkv[:, self.nq:self.nq + self.nk], self.k_norm, self.eps)
            v = qkv[:, self.nq + self.nk:]
            ctx = torch.empty((h.shape[0], self.heads * self.vdim), dtype=h.dtype, device=h.device)
            r0 = 0
            for slot, pos0, n in zip(batch.slot, batch.pos0, batch.n_new):
                ctx[r0:r0 + n] = self._attend_torch(q[r0:r0 + n], k[r0:r0 + n], v[r0:r0 + n], cache, slot, pos0)
                r0 += n
            r0 = 0
            for slot, pos0, n in zip(batch.slot, batch.pos0, batch.n_new):       # append only after every query has attended
                cache.append_rows(k[r0:r0 + n], v[r0:r0 + n], slot, pos0)
                r0 += n
        return F.linear(ctx, self.o.weight)
