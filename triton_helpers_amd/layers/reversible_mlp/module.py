"""``nn.Module`` wrapper of the reversible MLP (style of the reference's FullyFusedMLP module)."""
from __future__ import annotations

import torch
import torch.nn as nn
from torch import Tensor

from .kernel import reversible_mlp


class ReversibleMLP(nn.Module):
    """``blocks`` additive couplings over rows of width ``d_model`` (even, at most 128).

    Every F / G is ``Linear(H, H) -> activation -> Linear(H, H)`` with ``H = d_model // 2``, initialised like
    ``nn.Linear`` (Kaiming-uniform).  Parameters: ``w1, w2 (blocks*2*H, H)``, ``b1, b2 (blocks*2, H)``.
    """

    def __init__(self, d_model: int, blocks: int, activation: str = "gelu", bias: bool = True):
        super().__init__()
        assert d_model % 2 == 0 and d_model // 2 <= 64
        H = d_model // 2
        first = [nn.Linear(H, H, bias=bias) for _ in range(2 * blocks)]
        second = [nn.Linear(H, H, bias=bias) for _ in range(2 * blocks)]
        self.w1 = nn.Parameter(torch.cat([l.weight for l in first], 0))
        self.w2 = nn.Parameter(torch.cat([l.weight for l in second], 0))
        if bias:
            self.b1 = nn.Parameter(torch.stack([l.bias for l in first], 0))
            self.b2 = nn.Parameter(torch.stack([l.bias for l in second], 0))
        else:
            self.b1 = self.b2 = None
        self.activation = activation
        self.blocks = blocks

    def forward(self, x: Tensor) -> Tensor:
        return reversible_mlp(x, self.w1, self.b1, self.w2, self.b2, self.activation)
