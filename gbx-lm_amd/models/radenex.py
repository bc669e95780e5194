"""Radenex: a decoder-only stack of PARALLEL layers whose config.json lists its layers one by one.

A layer run reads one RMS norm of the residual stream, ``h = norm1(x)``, feeds it to its mixer and (optionally) its feed-forward,
and adds both outputs to the stream together: ``x += mixer(h) + ff(h)``.  Mixer kinds: ``latent_attention`` (keys and values of
all heads from one cached latent row per token, learned softmax sink, output gate) and ``attention`` (grouped-query sliding window
that keeps a sequence's first tokens, unit-norm rotated q / k, rotated values, one added to the softmax denominator); both live in
models/sink_attention.py.  Feed-forward kind ``dense``: ``down(relu(up h)^2)`` (models/feed_forward.py).  Config ``loop`` runs the
layers ``start .. stop-1`` ``times`` times in a row with the same weights; every run has a cache of its own.  Every size and
constant is read per layer from the config.  The stream is fp32; matrix products run in the activation dtype (bf16 as stored, or
fp32 when the model is loaded with ``dtype=torch.float32``).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional

import torch
from torch import nn

from ..batching import StepBatch
from .base import BaseModelArgs
from .feed_forward import DenseFeedForward
from .residual import StreamRMSNorm, stream_add_, stream_add_norm_
from .sink_attention import LatentAttention, RotatedValueWindowAttention
from .step_model import RaggedStepModel


@dataclass
class ModelArgs(BaseModelArgs):
    architecture: str
    vocab: int
    width: int
    layers: List[Dict[str, Any]]
    norm: Dict[str, Any]
    loop: Optional[Dict[str, int]] = None

    @property
    def model_type(self) -> str:
        return self.architecture.lower()

    def layer_runs(self) -> List[int]:
        n = len(self.layers)
        if not self.loop:
            return list(range(n))
        start, stop, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        if not 0 <= start <= stop <= n or times < 0:
            raise ValueError("Radenex: loop span outside the layers")
        return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))


def _mixer(args: ModelArgs, spec: Dict[str, Any]) -> nn.Module:
    kind, m, eps = spec["type"], spec["mixer"], args.norm["eps"]
    rot = m.get("rot") or {}
    if kind == "latent_attention":
        if rot.get("dims", m["rot_dim"]) != m["rot_dim"]:
            raise ValueError("Radenex: a latent mixer rotates exactly its rot_dim part")
        return LatentAttention(args.width, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], rot.get("base", 10000.0),
                               rot.get("scaling"), m["scale"], eps)
    if kind == "attention":
        mask = m.get("mask") or {}
        return RotatedValueWindowAttention(args.width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"], rot.get("dims", 0),
                                           rot.get("base", 10000.0), rot.get("scaling"), mask.get("size"), mask.get("keep_first", 0),
                                           m["scale"], eps)
    raise ValueError(f"Radenex: unknown mixer type {kind!r}")


def _feed_forward(args: ModelArgs, spec: Optional[Dict[str, Any]]) -> Optional[nn.Module]:
    if spec is None:
        return None
    if spec.get("kind") == "dense":
        return DenseFeedForward(args.width, spec["ff"], "relu2")
    raise ValueError(f"Radenex: unknown feed-forward kind {spec.get('kind')!r}")


class Layer(nn.Module):
    def __init__(self, args: ModelArgs, spec: Dict[str, Any]):
        super().__init__()
        self.norm1 = StreamRMSNorm(args.width, args.norm["eps"])
        self.mixer = _mixer(args, spec)
        self.mlp = _feed_forward(args, spec.get("mlp"))

    def forward(self, x: torch.Tensor, h: torch.Tensor, batch: StepBatch, cache, next_norm: Optional[StreamRMSNorm]) -> Optional[torch.Tensor]:
        """``h`` = this layer's norm of the fp32 stream ``x``.  Updates ``x`` in place and returns the NEXT run's norm of it (the update
        and that norm are one launch), or None after the last run."""
        y, z = self.mixer(h, batch, cache), (None if self.mlp is None else self.mlp(h))
        if next_norm is None:
            stream_add_(x, y, z)
            return None
        return stream_add_norm_(x, y, z, next_norm)


class RadenexModel(nn.Module):
    def __init__(self, args: ModelArgs):
        super().__init__()
        self.embed_tokens = nn.Embedding(args.vocab, args.width)
        self.embed_tokens.weight.requires_grad_(False)
        self.layers = nn.ModuleList(Layer(args, spec) for spec in args.layers)
        self.norm = StreamRMSNorm(args.width, args.norm["eps"])

    def embed(self, tokens: torch.Tensor) -> torch.Tensor:
        w = self.embed_tokens.weight
        if tokens.is_cuda:
            from .. import mixer_ops as M
            return M.embed_scaled(w, tokens, 1.0, image=False)[0]
        return w[tokens].float()


class Model(RaggedStepModel):
    def __init__(self, args: ModelArgs):
        super().__init__(args)
        self.model = RadenexModel(args)
        self._runs = args.layer_runs()

    @property
    def layer_runs(self) -> List[int]:
        return self._runs

    def forward_tokens(self, tokens: torch.Tensor, batch: StepBatch, caches) -> torch.Tensor:
        """One ragged step: tokens [T] -> fp32 stream [T, width] after the last layer run.  Positions are NOT advanced here."""
        x = self.model.embed(tokens)
        layers, runs = self.model.layers, self._runs
        h = layers[runs[0]].norm1(x, self.lm_head.weight.dtype) if runs else None
        for n, (i, cache) in enumerate(zip(runs, caches)):
            h = layers[i](x, h, batch, cache, layers[runs[n + 1]].norm1 if n + 1 < len(runs) else None)
            if self.trace_layers is not None:
                self.trace_layers.append(x.clone())
        return x

    def sanitize(self, weights: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
        """Checkpoint names -> module paths.  Projections that read the same input are concatenated; norm weights and sinks become
        fp32 (they only enter fp32 arithmetic); tables the modules computed from the config are kept as they are."""
        out: Dict[str, torch.Tensor] = {}
        f32 = lambda t: t.float()
        out["model.embed_tokens.weight"] = weights["embed"]
        out["model.norm.weight"] = f32(weights["final.norm"])
        out["lm_head.weight"] = weights["head"]
        for i, spec in enumerate(self.args.layers):
            p, t = f"l{i}.", f"model.layers.{i}."
            mixer = self.model.layers[i].mixer
            out[t + "norm1.weight"] = f32(weights[p + "norm1"])
            if spec["type"] == "latent_attention":
                fused = mixer.fuse_weights(weights[p + "mix.q"], weights[p + "mix.dkv"], weights[p + "mix.g"], weights[p + "mix.uk"],
                                           weights[p + "mix.uv"])
                for k, v in fused.items():
                    out[t + "mixer." + k] = v
                out[t + "mixer.latent_norm"] = f32(weights[p + "mix.dkv.norm"])
                out[t + "mixer.sink"] = f32(weights[p + "mix.sink"])
                out[t + "mixer.freq"] = mixer.freq
            else:
                out[t + "mixer.qkv.weight"] = torch.cat([weights[p + "mix.q"], weights[p + "mix.k"], weights[p + "mix.v"]])
                out[t + "mixer.freq"], out[t + "mixer.vfreq"], out[t + "mixer.sink"] = mixer.freq, mixer.vfreq, mixer.sink
            out[t + "mixer.o.weight"] = weights[p + "mix.o"]
            if spec.get("mlp") is not None:
                out[t + "mlp.up.weight"] = weights[p + "mlp.up"]
                out[t + "mlp.down.weight"] = weights[p + "mlp.down"]
        return out
