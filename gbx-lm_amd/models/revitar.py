"""Revitar: a decoder-only stack whose config.json lists its layers one by one.

Each layer is a sequence mixer and, optionally, a feed-forward; both read the residual stream directly and their OUTPUT is
RMS-normalised and scaled before it is added (models/residual.py).  The mixer kind this file knows is ``attention``: sliding-window
attention with independently gated keys (models/window_attention.py); the feed-forward kind is ``moe``: top-k routed gated MLPs
with un-renormalised softmax weights (models/switch_layers.py:DenseRoutedGLU).  Every size and constant is read per layer from
the config, so layers of one model may differ.  The stream is fp32; matrix products run in the activation dtype (bf16 as stored,
or fp32 when the model is loaded with ``dtype=torch.float32``).

The model works on ragged step batches (batching.py): ``forward_tokens`` takes a step's rows back to back with their descriptor
tables; ``forward(inputs [B, L], cache=)`` is the ``generate_step`` calling convention on top of it.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch
import torch.nn.functional as F
from torch import nn

from ..batching import StepBatch
from .base import BaseModelArgs
from .residual import BranchNormResidual, StreamRMSNorm
from .step_model import RaggedStepModel
from .switch_layers import DenseRoutedGLU
from .window_attention import GatedWindowAttention


@dataclass
class ModelArgs(BaseModelArgs):
    architecture: str
    vocab: int
    width: int
    layers: List[Dict[str, Any]]
    norm: Dict[str, Any]
    residual_mult: float = 1.0
    embedding: Dict[str, Any] = field(default_factory=dict)

    @property
    def model_type(self) -> str:
        return self.architecture.lower()


def _mixer(args: ModelArgs, spec: Dict[str, Any]) -> nn.Module:
    kind, m = spec["type"], spec["mixer"]
    if kind == "attention":
        return GatedWindowAttention(args.width, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["mask"]["size"], m["scale"],
                                    m.get("softcap") or 0.0, args.norm["eps"])
    raise ValueError(f"Revitar: unknown mixer type {kind!r}")


def _feed_forward(args: ModelArgs, spec: Optional[Dict[str, Any]]) -> Optional[nn.Module]:
    if spec is None:
        return None
    if spec.get("kind") == "moe":
        return DenseRoutedGLU(args.width, spec["expert"]["ff"], spec["router"]["experts"], spec["router"]["top"], renormalize=False)
    raise ValueError(f"Revitar: unknown feed-forward kind {spec.get('kind')!r}")


class Layer(nn.Module):
    def __init__(self, args: ModelArgs, spec: Dict[str, Any]):
        super().__init__()
        eps, mult = args.norm["eps"], args.residual_mult
        self.mixer = _mixer(args, spec)
        self.norm1 = BranchNormResidual(args.width, eps, mult)
        self.mlp = _feed_forward(args, spec.get("mlp"))
        self.norm2 = BranchNormResidual(args.width, eps, mult) if self.mlp is not None else None

    def forward(self, x: torch.Tensor, h: torch.Tensor, batch: StepBatch, cache) -> torch.Tensor:
        """x: fp32 stream (updated in place), h: its activation-dtype image; returns the new image."""
        h = self.norm1(x, self.mixer(h, batch, cache), None, h.dtype)
        if self.mlp is not None:
            y, mix = self.mlp(h)
            h = self.norm2(x, y, mix, h.dtype)
        return h


class RevitarModel(nn.Module):
    def __init__(self, args: ModelArgs):
        super().__init__()
        self.args = args
        self.embed_scale = float(args.embedding.get("scale", 1.0))
        self.embed_tokens = nn.Embedding(args.vocab, args.width)
        self.embed_tokens.weight.requires_grad_(False)
        self.layers = nn.ModuleList(Layer(args, spec) for spec in args.layers)
        self.norm = StreamRMSNorm(args.width, args.norm["eps"])

    def embed(self, tokens: torch.Tensor):
        w = self.embed_tokens.weight
        if tokens.is_cuda:
            from .. import mixer_ops as M
            return M.embed_scaled(w, tokens, self.embed_scale)
        x = w[tokens].float() * self.embed_scale
        return x, (x if w.dtype == torch.float32 else x.to(w.dtype))


class Model(RaggedStepModel):
    def __init__(self, args: ModelArgs):
        super().__init__(args)
        self.model = RevitarModel(args)

    def forward_tokens(self, tokens: torch.Tensor, batch: StepBatch, caches) -> torch.Tensor:
        """One ragged step: tokens [T] -> fp32 stream [T, width] after the last layer.  Positions are NOT advanced here."""
        x, h = self.model.embed(tokens)
        for layer, cache in zip(self.model.layers, caches):
            h = layer(x, h, batch, cache)
            if self.trace_layers is not None:
                self.trace_layers.append(x.clone())
        return x

    def sanitize(self, weights: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
        """Checkpoint names -> module paths.  q | k | v are concatenated into one projection, the experts stacked; norm weights,
        router and the per-head constants become fp32 (they only enter fp32 arithmetic), the rest keeps its dtype."""
        out: Dict[str, torch.Tensor] = {}
        f32 = lambda t: t.float()
        out["model.embed_tokens.weight"] = weights["embed"]
        out["model.norm.weight"] = f32(weights["final.norm"])
        out["lm_head.weight"] = weights["head"]
        for i, spec in enumerate(self.args.layers):
            p, t = f"l{i}.", f"model.layers.{i}."
            out[t + "norm1.weight"] = f32(weights[p + "norm1"])
            if spec["type"] == "attention":
                out[t + "mixer.qkv.weight"] = torch.cat([weights[p + "mix.q"], weights[p + "mix.k"], weights[p + "mix.v"]])
                out[t + "mixer.o.weight"] = weights[p + "mix.o"]
                out[t + "mixer.q_norm"] = f32(weights[p + "mix.q.norm"])
                out[t + "mixer.k_norm"] = f32(weights[p + "mix.k.norm"])
                out[t + "mixer.dist_mul"] = f32(weights[p + "mix.r1"])
                out[t + "mixer.dist_rate"] = f32(weights[p + "mix.r2"])
                out[t + "mixer.gate_bias"] = f32(weights[p + "mix.pb"])
            if spec.get("mlp") is not None:
                out[t + "norm2.weight"] = f32(weights[p + "norm2"])
                n_e = spec["mlp"]["router"]["experts"]
                out[t + "mlp.router"] = f32(weights[p + "mlp.router"])
                out[t + "mlp.gate_up"] = torch.stack([torch.cat([weights[p + f"mlp.e{e}.gate"], weights[p + f"mlp.e{e}.up"]]) for e in range(n_e)])
                out[t + "mlp.down"] = torch.stack([weights[p + f"mlp.e{e}.down"] for e in range(n_e)])
        return out
