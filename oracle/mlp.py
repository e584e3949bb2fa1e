"""CPU oracle for the fully fused MLP (test infrastructure only).

The reference checks its fused kernel against a chain of ``nn.Linear`` layers
with an activation between them and none after the last
(``tests/test_layers/test_fully_fused_mlp.py:21-35``); the kernel's own layer
math is ``triton_helpers/layers/fully_fused_mlp/kernel.py:17-74`` with the
activations of ``triton_helpers/ops.py:37-66``.  This file restates both: a
float32 chain (the parity target) and a variant that rounds every layer's
result to the storage dtype, as the kernel does (kernel.py:47).

Weight layout (kernel.py:77-136): ``w_in [H, D_in]``, ``w_hid [(depth-1)*H, H]``
hidden layers stacked along rows, ``b_hid [depth-1, H]``, ``w_out [D_out, H]``.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch
import torch.nn.functional as F
from torch import Tensor


def activation(z: Tensor, name: str) -> Tensor:
    """relu / silu / relu2 / none / gelu (ops.py:37-66; gelu = exact erf form)."""
    if name == "relu":
        return torch.where(z < 0, torch.zeros_like(z), z)
    if name == "silu":
        return z * torch.sigmoid(z)
    if name == "relu2":
        return torch.clamp_min(z, 0) * z
    if name == "gelu":
        return F.gelu(z)
    if name == "none":
        return z
    raise ValueError(name)


def ste_round(t: Tensor, dtype: Optional[torch.dtype]) -> Tensor:
    """Round to ``dtype`` (back in float32) with a straight-through gradient, so that autograd
    sees the rounded values -- and therefore the same activation gates as a kernel that stores
    ``dtype`` between layers -- while the derivative of the rounding itself is taken as one."""
    if dtype is None:
        return t
    return t + (t.detach().to(dtype).to(torch.float32) - t.detach())


def split_hidden(w_hid: Optional[Tensor], b_hid: Optional[Tensor], hidden: int):
    """Un-stack ``w_hid``/``b_hid`` into per-layer lists (kernel.py:534-542)."""
    if w_hid is None or w_hid.numel() == 0:
        return [], []
    n = w_hid.shape[0] // hidden
    ws = [w_hid[i * hidden : (i + 1) * hidden] for i in range(n)]
    bs = [None if b_hid is None else b_hid[i] for i in range(n)]
    return ws, bs


def mlp_forward(
    x: Tensor,
    w_in: Tensor,
    b_in: Optional[Tensor],
    w_out: Tensor,
    b_out: Optional[Tensor],
    w_hid: Optional[Tensor] = None,
    b_hid: Optional[Tensor] = None,
    act: str = "relu",
    round_to: Optional[torch.dtype] = None,
) -> Tensor:
    """``act(x W_in^T + b) -> [act(h W_k^T + b_k)]* -> h W_out^T + b`` in float32.

    With ``round_to`` set, each layer's result is rounded to that dtype (and
    brought back to float32) before the next layer, mirroring kernel.py:47.
    """

    def rnd(t: Tensor) -> Tensor:
        return ste_round(t, round_to)

    f32 = lambda t: None if t is None else t.to(torch.float32)  # noqa: E731
    h = rnd(activation(F.linear(f32(x), f32(w_in), f32(b_in)), act))
    ws, bs = split_hidden(w_hid, b_hid, w_in.shape[0])
    for w, b in zip(ws, bs):
        h = rnd(activation(F.linear(h, f32(w), f32(b)), act))
    return rnd(F.linear(h, f32(w_out), f32(b_out)))


def mlp_backward(
    x: Tensor,
    dy: Tensor,
    w_in: Tensor,
    b_in: Optional[Tensor],
    w_out: Tensor,
    b_out: Optional[Tensor],
    w_hid: Optional[Tensor] = None,
    b_hid: Optional[Tensor] = None,
    act: str = "relu",
    round_to: Optional[torch.dtype] = None,
) -> Dict[str, Optional[Tensor]]:
    """Float32 gradients of ``mlp_forward`` via autograd (the reference tests'
    baseline, test_fully_fused_mlp.py:253-260).  ``round_to`` evaluates the forward
    with storage-dtype rounding between layers (what a 16-bit ``nn.Linear`` chain does)."""
    leaves = {}

    def leaf(name, t):
        if t is None:
            leaves[name] = None
            return None
        v = t.detach().to(torch.float32).clone().requires_grad_(True)
        leaves[name] = v
        return v

    xx = leaf("x", x)
    args = [leaf(n, t) for n, t in (("w_in", w_in), ("b_in", b_in), ("w_out", w_out), ("b_out", b_out), ("w_hid", w_hid), ("b_hid", b_hid))]
    y = mlp_forward(xx, *args, act=act, round_to=round_to)
    y.backward(dy.to(torch.float32))
    return {("d" + k): (None if v is None else v.grad) for k, v in leaves.items()}
