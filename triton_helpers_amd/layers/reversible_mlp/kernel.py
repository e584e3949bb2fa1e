"""Reversible (additive-coupling) fused MLP on MI355X.

The reference has no such layer; the surface follows its siblings' style.  Rows of
width ``2*H`` are split into halves ``x1, x2`` and pass through ``blocks`` couplings

    y1 = x1 + F_k(x2),   y2 = x2 + G_k(y1),   F/G(u) = act(u W1^T + b1) W2^T + b2.

``w1, w2 : (blocks*2*H, H)`` hold, per block, F's matrix then G's; ``b1, b2 : (blocks*2, H)``
or ``None``.  The autograd Function saves only the OUTPUT: the backward kernel rebuilds each
block's input from its output while it back-propagates, so no activation is stored.

Choice of activation.  The rebuilt inputs come from 16-bit outputs, so a pre-activation that the forward saw within
rounding of zero can land on the other side of zero in the backward.  Smooth activations (``"gelu"``, ``"silu"``) do not
notice: at 65 536 rows, width 128, four couplings, no element of ``dx`` or of the weight gradients is outside rtol 2e-2 /
atol 1e-2 of a float32 evaluation.  ``"relu"`` and ``"relu2"`` take their gates from the rebuilt inputs: a gate that flips
moves a gradient by a whole weight, and 12 % of the elements of ``dx`` are outside that tolerance in the same measurement
(largest error 7 % of the largest entry).  Use a smooth activation when the gradients matter to that level.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor
from torch.autograd import Function

from ... import _lib

_ACTIVATIONS = ("gelu", "relu", "relu2", "silu", "none")


def _rows2d(t: Tensor, width: int) -> Tensor:
    t2 = t.reshape(-1, width)
    # rows that overlap (an expanded / broadcast tensor has row stride 0) or a strided inner dimension: copy
    if t2.stride(1) != 1 or (t2.shape[0] > 1 and t2.stride(0) < width):
        t2 = t2.contiguous()
    return t2


def _validate(x: Tensor, w1: Tensor, b1: Optional[Tensor], w2: Tensor, b2: Optional[Tensor], activation: str):
    assert x.shape[-1] % 2 == 0, "Feature dimension must be even"
    H = x.shape[-1] // 2
    assert H <= 64, f"Half width {H} too large for full fusion"
    assert w1.ndim == 2 and w1.shape[1] == H and w1.shape[0] % (2 * H) == 0, "w1 must be (blocks*2*H, H)"
    assert w2.shape == w1.shape, "w2 must have the shape of w1"
    blocks = w1.shape[0] // (2 * H)
    for b in (b1, b2):
        assert b is None or b.shape == (2 * blocks, H), "biases must be (blocks*2, H)"
    assert activation in _ACTIVATIONS, f"Invalid activation function: {activation}"
    if x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise NotImplementedError(f"reversible_mlp runs on float16 / bfloat16 / float32 storage, got {x.dtype}")
    for t in (w1, b1, w2, b2):
        assert t is None or (t.dtype == x.dtype and t.device == x.device), "All tensors must share dtype and device"
    assert x.device.type == "cuda", "All tensors must be on a GPU device"
    return H, blocks


def _c(t: Optional[Tensor]) -> Optional[Tensor]:
    return None if t is None else (t if t.is_contiguous() else t.contiguous())


class _reversible_mlp(Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.float16)
    @torch.no_grad()
    def forward(ctx, x: Tensor, w1: Tensor, b1: Optional[Tensor], w2: Tensor, b2: Optional[Tensor], activation: str = "gelu") -> Tensor:
        H, blocks = _validate(x, w1, b1, w2, b2, activation)
        # float32 tensors run with float16 operands (float32 accumulation) and come back as float32, like the fused MLP
        wide = x.dtype == torch.float32
        if wide:
            x, w1, b1, w2, b2 = (None if t is None else t.to(torch.float16) for t in (x, w1, b1, w2, b2))
        w1, b1, w2, b2 = (_c(t) for t in (w1, b1, w2, b2))
        x2 = _rows2d(x, 2 * H)
        y = x.new_empty(x.shape)
        y2 = y.view(-1, 2 * H)
        lib = _lib.load()
        rc = lib.nf_revmlp_fwd(
            x2.data_ptr(), x2.stride(0), y2.data_ptr(), y2.stride(0), w1.data_ptr(), _lib.ptr(b1), w2.data_ptr(), _lib.ptr(b2),
            x2.shape[0], H, blocks, _lib.NF_ACT[activation], _lib.dtype_code(x.dtype), _lib.current_stream(x.device),
        )
        _lib.check(rc, "nf_revmlp_fwd")
        ctx.save_for_backward(y, w1, b1, w2, b2)  # the output, not the input
        ctx.activation = activation
        ctx.half = H
        ctx.blocks = blocks
        ctx.wide = wide
        return y.float() if wide else y

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    @torch.no_grad()
    def backward(ctx, dy: Tensor):
        y, w1, b1, w2, b2 = ctx.saved_tensors
        H = ctx.half
        if dy.dtype != y.dtype:
            dy = dy.to(y.dtype)
        y2 = _rows2d(y, 2 * H)
        dy2 = _rows2d(dy, 2 * H)
        dx = y.new_empty(y.shape)
        x_rec = y.new_empty(y.shape)

        grads = _lib.GradBuffers(w1, b1, w2, b2)
        p_dw1, p_db1, p_dw2, p_db2 = grads.pointers()
        lib = _lib.load()
        rc = lib.nf_revmlp_bwd(
            y2.data_ptr(), y2.stride(0), dy2.data_ptr(), dy2.stride(0), dx.data_ptr(), 2 * H, x_rec.data_ptr(), 2 * H,
            w1.data_ptr(), _lib.ptr(b1), w2.data_ptr(), _lib.ptr(b2),
            p_dw1, p_db1, p_dw2, p_db2,
            y2.shape[0], H, ctx.blocks, _lib.NF_ACT[ctx.activation], _lib.dtype_code(y.dtype), _lib.current_stream(y.device),
        )
        _lib.check(rc, "nf_revmlp_bwd")
        dw1, db1, dw2, db2 = grads.rounded(torch.float32 if ctx.wide else w1.dtype)
        return (dx.float() if ctx.wide else dx), dw1, db1, dw2, db2, None


def reversible_mlp(x: Tensor, w1: Tensor, b1: Optional[Tensor], w2: Tensor, b2: Optional[Tensor], activation: str = "gelu") -> Tensor:
    r"""Reversible MLP forward; differentiable without stored activations.

    Shapes:
        - x: :math:`(..., 2H)`, :math:`H \le 64`
        - w1, w2: :math:`(\text{blocks} \cdot 2H, H)`; b1, b2: :math:`(\text{blocks} \cdot 2, H)` or ``None``
        - Output: same shape and dtype as ``x``
    """
    return _reversible_mlp.apply(x, w1, b1, w2, b2, activation)


@torch.no_grad()
def reversible_mlp_inverse(y: Tensor, w1: Tensor, b1: Optional[Tensor], w2: Tensor, b2: Optional[Tensor], activation: str = "gelu") -> Tensor:
    """Input reconstructed from the output by the backward kernel's in-kernel inverse."""
    H, blocks = _validate(y, w1, b1, w2, b2, activation)
    wide = y.dtype == torch.float32
    if wide:
        y, w1, b1, w2, b2 = (None if t is None else t.to(torch.float16) for t in (y, w1, b1, w2, b2))
    w1, b1, w2, b2 = (_c(t) for t in (w1, b1, w2, b2))
    y2 = _rows2d(y, 2 * H)
    zeros = torch.zeros_like(y2)
    dx = torch.empty_like(y2)
    x_rec = y.new_empty(y.shape)
    dw1 = torch.zeros(w1.shape, dtype=torch.float32, device=y.device)
    dw2 = torch.zeros_like(dw1)
    lib = _lib.load()
    rc = lib.nf_revmlp_bwd(
        y2.data_ptr(), y2.stride(0), zeros.data_ptr(), zeros.stride(0), dx.data_ptr(), 2 * H, x_rec.data_ptr(), 2 * H,
        w1.data_ptr(), _lib.ptr(b1), w2.data_ptr(), _lib.ptr(b2), dw1.data_ptr(), None, dw2.data_ptr(), None,
        y2.shape[0], H, blocks, _lib.NF_ACT[activation], _lib.dtype_code(y.dtype), _lib.current_stream(y.device),
    )
    _lib.check(rc, "nf_revmlp_bwd")
    return x_rec.float() if wide else x_rec
