"""Dense feed-forward of ragged-step models: ``down(act(up h))`` with the activation as a parameter.

``relu2``: the square of relu; ``gelu_tanh``: 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).  The two products are plain
matrix products (vendor library); the activation is one in-place HIP launch on GPU tensors (fp32 arithmetic, result in the
activation dtype)."""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F
from torch import nn

ACTIVATIONS = ("relu2", "gelu_tanh")


def activate_(z: torch.Tensor, kind: str) -> torch.Tensor:
    if kind not in ACTIVATIONS:
        raise ValueError(f"unknown activation {kind!r}")
    if z.is_cuda:
        from .. import mixer_ops as M
        return M.activate_(z, kind)
    f = z.float()
    if kind == "relu2":
        f = torch.relu(f).pow(2)
    else:
        f = 0.5 * f * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (f + 0.044715 * f.pow(3))))
    return z.copy_(f.to(z.dtype))


class DenseFeedForward(nn.Module):
    def __init__(self, width: int, ff: int, activation: str = "relu2"):
        super().__init__()
        if activation not in ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}")
        self.activation = activation
        self.up = nn.Linear(width, ff, bias=False)
        self.down = nn.Linear(ff, width, bias=False)
        for p in self.parameters():
            p.requires_grad_(False)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(activate_(F.linear(h, self.up.weight), self.activation), self.down.weight)
