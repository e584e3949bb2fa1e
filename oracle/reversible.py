"""CPU oracle for the reversible (additive-coupling) fused MLP -- test infrastructure only.

PARITY UNPINNED BY THE REFERENCE: ``triton_helpers/layers/`` holds no
reversible MLP, so there is no reference function, test or vector for it.
What pins this file is mathematics: the RevNet additive coupling

    y1 = x1 + F(x2)          x2 = y2 - G(y1)
    y2 = x2 + G(y1)          x1 = y1 - F(x2)

``inverse(forward(x)) == x`` and gradients equal to ``torch.autograd`` through
the plain composition.  F and G are two-layer MLPs ``act(u W1^T + b1) W2^T + b2``
built from the same layer math as the fused MLP
(``triton_helpers/layers/fully_fused_mlp/kernel.py:17-47``).

Weight layout: ``w1, w2 : [blocks*2*H, H]`` -- for block ``k`` rows
``[(2k)*H, (2k+1)*H)`` are F's and ``[(2k+1)*H, (2k+2)*H)`` are G's;
``b1, b2 : [blocks*2, H]`` or ``None``.  ``x : [rows, 2*H]`` with
``x1 = x[:, :H]`` and ``x2 = x[:, H:]``.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch
import torch.nn.functional as F
from torch import Tensor

from .mlp import activation, ste_round


def _sub(u: Tensor, w1: Tensor, b1, w2: Tensor, b2, i: int, h: int, act: str, rnd) -> Tensor:
    bb1 = None if b1 is None else b1[i]
    bb2 = None if b2 is None else b2[i]
    t = rnd(activation(F.linear(rnd(u), w1[i * h : (i + 1) * h], bb1), act))
    return F.linear(t, w2[i * h : (i + 1) * h], bb2)


def rev_forward(
    x: Tensor,
    w1: Tensor,
    b1: Optional[Tensor],
    w2: Tensor,
    b2: Optional[Tensor],
    act: str = "gelu",
    round_to: Optional[torch.dtype] = None,
    stream_round_every: int = 1,
) -> Tensor:
    """Float32 forward over all coupling blocks.  With ``round_to`` every matmul operand
    (sub-MLP input and hidden activation) is rounded to that dtype, and the residual stream
    itself after every ``stream_round_every``-th block (0: never) -- the points at which a
    storage-dtype kernel that runs that many blocks per launch rounds."""
    rnd = lambda t: ste_round(t, round_to)  # noqa: E731
    f32 = lambda t: None if t is None else t.to(torch.float32)  # noqa: E731
    x, w1, b1, w2, b2 = f32(x), f32(w1), f32(b1), f32(w2), f32(b2)
    h = x.shape[-1] // 2
    blocks = w1.shape[0] // (2 * h)
    x1, x2 = x[..., :h], x[..., h:]
    for k in range(blocks):
        y1 = x1 + _sub(x2, w1, b1, w2, b2, 2 * k, h, act, rnd)
        y2 = x2 + _sub(y1, w1, b1, w2, b2, 2 * k + 1, h, act, rnd)
        if stream_round_every and (k + 1) % stream_round_every == 0:
            y1, y2 = rnd(y1), rnd(y2)
        x1, x2 = y1, y2
    return torch.cat([x1, x2], -1)


def rev_inverse(
    y: Tensor, w1: Tensor, b1: Optional[Tensor], w2: Tensor, b2: Optional[Tensor], act: str = "gelu"
) -> Tensor:
    """Float32 inverse: walks the blocks in reverse and undoes each coupling."""
    f32 = lambda t: None if t is None else t.to(torch.float32)  # noqa: E731
    y, w1, b1, w2, b2 = f32(y), f32(w1), f32(b1), f32(w2), f32(b2)
    h = y.shape[-1] // 2
    blocks = w1.shape[0] // (2 * h)
    ident = lambda t: t  # noqa: E731
    y1, y2 = y[..., :h], y[..., h:]
    for k in reversed(range(blocks)):
        x2 = y2 - _sub(y1, w1, b1, w2, b2, 2 * k + 1, h, act, ident)
        x1 = y1 - _sub(x2, w1, b1, w2, b2, 2 * k, h, act, ident)
        y1, y2 = x1, x2
    return torch.cat([y1, y2], -1)


def rev_backward(
    x: Tensor, dy: Tensor, w1: Tensor, b1: Optional[Tensor], w2: Tensor, b2: Optional[Tensor], act: str = "gelu",
    round_to: Optional[torch.dtype] = None,
) -> Dict[str, Optional[Tensor]]:
    """Float32 gradients via autograd through ``rev_forward`` (stored activations)."""
    leaves = {}

    def leaf(name, t):
        if t is None:
            leaves[name] = None
            return None
        v = t.detach().to(torch.float32).clone().requires_grad_(True)
        leaves[name] = v
        return v

    args = [leaf(n, t) for n, t in (("x", x), ("w1", w1), ("b1", b1), ("w2", w2), ("b2", b2))]
    y = rev_forward(*args, act=act, round_to=round_to)
    y.backward(dy.to(torch.float32))
    return {("d" + k): (None if v is None else v.grad) for k, v in leaves.items()}
