"""Fully fused small MLP on MI355X.

Drop-in for ``triton_helpers/layers/fully_fused_mlp/kernel.py`` of the reference:
same ``fully_fused_mlp(...)`` functional and ``_fully_fused_mlp`` autograd Function
(argument order, 9-tuple returned by ``backward``), same assertions and the same
weight layout (``w_hid`` = hidden layers stacked along rows, ``b_hid [depth-1, H]``).
The Triton launches are replaced by ``nf_mlp_fwd`` / ``nf_mlp_bwd`` of ``libnf_cdna4.so``.

Supersets / differences:
  * any bias may be ``None`` (the reference always has biases);
  * weight gradients are accumulated in float32 inside the kernel and rounded once
    (the reference sums per-program partials in the storage dtype, kernel.py:599-633);
  * ``fp16_acc`` is accepted and ignored: accumulation is always float32 (MFMA);
  * float16 and bfloat16 storage (what autocast produces) runs on the 16-bit matrix instructions: the fast path.
    float32 tensors (the reference feeds them to ``tl.dot``, which multiplies in TF32: float32 range, 10-bit
    mantissa) run on the float32 matrix instruction: float32 range and mantissa, about a sixth of the 16-bit rate, and
    a backward scratch of ``depth * rows * d_hidden * 4`` bytes.  ``set_float32_operands("float16")`` trades the
    range for speed: float32 tensors are then multiplied with float16 operands (the same 10-bit mantissa as TF32,
    float32 accumulation and results; operands beyond +-65504 overflow).
"""
from __future__ import annotations

from typing import Final, Optional

import torch
import torch.nn.functional as F
from torch import Tensor
from torch.autograd import Function

from ... import _lib

# Above this size the weights do not stay on chip (reference kernel.py:13-14)
FULLY_FUSED_MAX_DIM: Final = 64

_ACTIVATIONS = ("relu", "relu2", "silu", "none")

_FLOAT32_OPERANDS = "float32"


def set_float32_operands(kind: str) -> str:
    """How float32 tensors are multiplied: ``"float32"`` (default: float32 range and mantissa) or ``"float16"``
    (float16 operands, float32 accumulation: several times faster, operands limited to +-65504).  Returns the
    previous setting.  (The counterpart of ``allow_tf32`` for ``tl.dot`` in the reference, kernel.py:17-47.)"""
    global _FLOAT32_OPERANDS
    assert kind in ("float32", "float16"), f"float32 operands are 'float32' or 'float16', got {kind!r}"
    previous, _FLOAT32_OPERANDS = _FLOAT32_OPERANDS, kind
    return previous


def get_float32_operands() -> str:
    return _FLOAT32_OPERANDS


# ---------------------------------------------------------------------------
# Per-layer math with the reference's names (kernel.py:17-74).  In the reference these
# are Triton device functions; here they are plain torch functions for users' tests.
# No operator of this package calls them.
# ---------------------------------------------------------------------------
def _activate(z: Tensor, activation: str) -> Tensor:
    if activation == "relu":
        return torch.where(z < 0, torch.zeros_like(z), z)
    if activation == "silu":
        return z * torch.sigmoid(z)
    if activation == "relu2":
        return torch.clamp_min(z, 0) * z
    if activation == "none":
        return z
    raise ValueError(f"Invalid activation function: {activation}")


def feedforward(x: Tensor, w: Tensor, b: Optional[Tensor], HAS_BIAS: bool = True, ACTIVATION: str = "relu",
                DTYPE: torch.dtype = torch.float32) -> Tensor:
    z = x.to(DTYPE) @ w.to(DTYPE).t()
    if HAS_BIAS and b is not None:
        z = z + b.to(DTYPE)
    return _activate(z, ACTIVATION).to(x.dtype)


def feedforward_bwd_dz(z: Tensor, do: Tensor, ACTIVATION: str) -> Tensor:
    zf, g = z.float(), do.float()
    if ACTIVATION == "relu":
        dz = torch.where(zf > 0, g, torch.zeros_like(g))
    elif ACTIVATION == "silu":
        s = torch.sigmoid(zf)
        dz = g * s * (zf * (1 - s) + 1)
    elif ACTIVATION == "relu2":
        dz = torch.where(zf > 0, g * (2 * zf), torch.zeros_like(g))
    elif ACTIVATION == "none":
        dz = g
    else:
        raise ValueError(f"Invalid activation function: {ACTIVATION}")
    return dz.to(do.dtype)


def feedforward_bwd_dw(x: Tensor, dz: Tensor, DTYPE: torch.dtype = torch.float32) -> Tensor:
    return (dz.to(DTYPE).t() @ x.to(DTYPE)).to(dz.dtype)


def feedforward_bwd_dx(w: Tensor, dz: Tensor, DTYPE: torch.dtype = torch.float32) -> Tensor:
    return (dz.to(DTYPE) @ w.to(DTYPE)).to(dz.dtype)


# ---------------------------------------------------------------------------
def _check_storage(x: Tensor, w_in: Tensor, *others: Optional[Tensor]) -> None:
    """Parameters share one dtype.  With 16-bit parameters ``x`` may be in the other 16-bit dtype (an fp16 encoder
    output in front of bf16 weights): the kernels convert it while loading, exactly as a cast in front would.
    float32 runs as a whole (``x`` and parameters)."""
    if w_in.dtype == torch.float32:
        assert x.dtype == torch.float32, f"float32 parameters take a float32 input, got {x.dtype}"
    else:
        for t in (x, w_in):
            if t.dtype not in (torch.float16, torch.bfloat16):
                raise NotImplementedError(
                    f"fully_fused_mlp runs on float16 / bfloat16 / float32 storage, got {t.dtype}; cast the tensors or use autocast"
                )
    for t in others:
        assert t is None or t.dtype == w_in.dtype, f"All parameters must share one dtype, got {w_in.dtype} and {t.dtype}"
    for t in (w_in, *others):
        assert t is None or t.device == x.device, "All tensors must be on the same device"
    assert x.device.type == "cuda", "All tensors must be on a GPU device"


def _rows2d(t: Tensor, width: int) -> Tensor:
    t2 = t.reshape(-1, width)
    # rows that overlap (an expanded / broadcast tensor has row stride 0) or a strided inner dimension: copy
    if t2.stride(1) != 1 or (t2.shape[0] > 1 and t2.stride(0) < width):
        t2 = t2.contiguous()
    return t2


def _half(t: Optional[Tensor]) -> Optional[Tensor]:
    return None if t is None else t.to(torch.float16)


def _c(t: Optional[Tensor]) -> Optional[Tensor]:
    return None if t is None else (t if t.is_contiguous() else t.contiguous())


_workspace_sizes: dict = {}


def _workspace(lib, rows2d: Tensor, d_hidden: int, depth: int, activation: str, backward: bool, dtype: torch.dtype):
    """Scratch for networks that run as several launches (none for the usual depths) and for the float32 backward."""
    key = (rows2d.shape[0], d_hidden, depth, activation, backward, dtype)
    n = _workspace_sizes.get(key)
    if n is None:
        n = lib.nf_mlp_workspace_bytes(rows2d.shape[0], d_hidden, depth, _lib.NF_ACT[activation], int(backward),
                                       _lib.dtype_code(dtype))
        if len(_workspace_sizes) < 4096:
            _workspace_sizes[key] = n
    if n == 0:
        return None, 0
    return torch.empty(n, dtype=torch.uint8, device=rows2d.device), n


class _fully_fused_mlp(Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.float16)
    def forward(
        ctx,
        x: Tensor,
        w_in: Tensor, b_in: Optional[Tensor],
        w_out: Tensor, b_out: Optional[Tensor],
        w_hid: Optional[Tensor], b_hid: Optional[Tensor],
        activation: str = "relu",
        fp16_acc: bool = False,
    ) -> Tensor:
        B, L, D = x.shape
        D_hidden, D_in = w_in.shape
        D_out, _ = w_out.shape
        assert D_in == D, "Input dimension mismatch"
        assert D_hidden == w_out.shape[-1], "Hidden dimension mismatch"

        assert D_in <= FULLY_FUSED_MAX_DIM, f"Input dimension {D_in} too large for full fusion"
        assert D_hidden <= FULLY_FUSED_MAX_DIM, f"Hidden dimension {D_hidden} too large for full fusion"
        assert D_out <= FULLY_FUSED_MAX_DIM, f"Output dimension {D_out} too large for full fusion"

        assert D_hidden & (D_hidden - 1) == 0, "Hidden dimension must be a power of 2"
        assert D_hidden >= 16, "Hidden dimension must be at least 16"

        if w_hid is not None and w_hid.numel() > 0:
            n_hid = w_hid.shape[0] // D_hidden
            assert w_hid.shape == (n_hid * D_hidden, D_hidden), "Hidden weight shape mismatch"
            assert b_hid is None or b_hid.shape == (n_hid, D_hidden), "Hidden bias shape mismatch"
            depth = n_hid + 1
        else:
            depth = 1
            w_hid = b_hid = None
        assert b_in is None or b_in.shape == (D_hidden,), "Input bias shape mismatch"
        assert b_out is None or b_out.shape == (D_out,), "Output bias shape mismatch"

        assert activation in _ACTIVATIONS, f"Invalid activation function: {activation}"
        _check_storage(x, w_in, b_in, w_out, b_out, w_hid, b_hid)

        ctx.save_for_backward(x, w_in, b_in, w_out, b_out, w_hid, b_hid)
        ctx.activation = activation
        ctx.fp16_acc = fp16_acc
        ctx.depth = depth
        ctx.wide = wide = w_in.dtype == torch.float32 and _FLOAT32_OPERANDS == "float16"
        if wide:  # float16 operands, float32 accumulation and results
            x, w_in, b_in, w_out, b_out, w_hid, b_hid = (_half(t) for t in (x, w_in, b_in, w_out, b_out, w_hid, b_hid))
        w_in, b_in, w_out, b_out, w_hid, b_hid = (_c(t) for t in (w_in, b_in, w_out, b_out, w_hid, b_hid))
        x2 = _rows2d(x, D_in)
        o = x.new_empty((B, L, D_out), dtype=w_in.dtype)
        o2 = o.view(-1, D_out)
        lib = _lib.load()
        ws, ws_bytes = _workspace(lib, x2, D_hidden, depth, activation, False, w_in.dtype)
        rc = lib.nf_mlp_fwd(
            x2.data_ptr(), x2.stride(0), o2.data_ptr(), o2.stride(0),
            w_in.data_ptr(), _lib.ptr(b_in), _lib.ptr(w_hid), _lib.ptr(b_hid), w_out.data_ptr(), _lib.ptr(b_out),
            x2.shape[0], D_in, D_hidden, D_out, depth, _lib.NF_ACT[activation], _lib.dtype_code(w_in.dtype),
            _lib.dtype_code(x.dtype), _lib.ptr(ws), ws_bytes, _lib.current_stream(x.device),
        )
        _lib.check(rc, "nf_mlp_fwd")
        return o.float() if wide else o

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, do: Tensor):
        x, w_in, b_in, w_out, b_out, w_hid, b_hid = ctx.saved_tensors
        B, L, D_in = x.shape
        D_hidden = w_in.shape[0]
        D_out = w_out.shape[0]
        wide = ctx.wide
        if wide:
            x, w_in, b_in, w_out, b_out, w_hid, b_hid = (_half(t) for t in (x, w_in, b_in, w_out, b_out, w_hid, b_hid))
        if do.dtype != w_in.dtype:
            do = do.to(w_in.dtype)
        converts = (ctx.depth == 2 and D_hidden > 32) or (ctx.depth == 1 and D_hidden == 64)
        if x.dtype != w_in.dtype and not (w_in.dtype != torch.float32 and converts and ctx.activation == "relu"):
            x = x.to(w_in.dtype)  # only the ReLU backward of one or two 64-wide hidden layers converts on the fly
        do2 = _rows2d(do, D_out)
        need_dx = ctx.needs_input_grad[0]
        decoder = D_in <= 32 and D_out <= 16  # the wider shapes need x in the parameters' dtype
        # (one hidden layer runs on the same kernels behind an identity layer that the library supplies)
        if (not wide and w_in.dtype != torch.float32 and ctx.depth in (1, 2) and D_hidden == 64 and D_in <= 64 and D_out <= 64
                and (decoder or x.dtype == w_in.dtype)
                and D_in % 4 == 0 and D_out % 4 == 0 and ctx.activation == "relu" and do2.shape[0] > 0):
            done = _backward_rounded(x, do2, w_in, b_in, w_out, b_out, w_hid, b_hid, need_dx, D_in, D_hidden, D_out, ctx.depth)
            if done is not None:
                return done
        grads = _lib.GradBuffers(w_in, b_in, w_out, b_out, w_hid, b_hid)
        p_dw_in, p_db_in, p_dw_out, p_db_out, p_dw_hid, p_db_hid = grads.pointers()
        lib = _lib.load()
        ws, ws_bytes = _workspace(lib, do2, D_hidden, ctx.depth, ctx.activation, True, w_in.dtype)
        while True:
            x2 = _rows2d(x, D_in)
            dx = x.new_empty(x.shape) if need_dx else None
            rc = lib.nf_mlp_bwd(
                x2.data_ptr(), x2.stride(0), do2.data_ptr(), do2.stride(0),
                _lib.ptr(dx), D_in,
                w_in.data_ptr(), _lib.ptr(b_in), _lib.ptr(w_hid), _lib.ptr(b_hid), w_out.data_ptr(), _lib.ptr(b_out),
                p_dw_in, p_db_in, p_dw_hid, p_db_hid, p_dw_out, p_db_out,
                x2.shape[0], D_in, D_hidden, D_out, ctx.depth, _lib.NF_ACT[ctx.activation], _lib.dtype_code(w_in.dtype),
                _lib.dtype_code(x.dtype), _lib.ptr(ws), ws_bytes, _lib.current_stream(x.device),
            )
            if rc == _lib.NF_EUNSUPPORTED and x.dtype != w_in.dtype:
                x = x.to(w_in.dtype)  # a shape / alignment the converting backward does not cover: cast first
                continue
            break
        _lib.check(rc, "nf_mlp_bwd")
        # float32 accumulators, rounded once to the parameters' dtype (one kernel for all of them)
        dw_in, db_in, dw_out, db_out, dw_hid, db_hid = grads.rounded(torch.float32 if wide else w_in.dtype)
        if wide and dx is not None:
            dx = dx.float()
        return dx, dw_in, db_in, dw_out, db_out, dw_hid, db_hid, None, None


_rounded_plans: dict = {}


def _rounded_plan(lib, like, D_in, D_hidden, D_out):
    """Where each gradient sits in the flat buffer (16-byte aligned pieces), its length and the scratch size, per
    combination of parameter shapes (a handful per process)."""
    key = tuple(None if t is None else (tuple(t.shape), t.stride(), t.dtype) for t in like)
    plan = _rounded_plans.get(key)
    if plan is None:
        offsets, off = [], 0
        for t in like:
            offsets.append(off)
            if t is not None:
                off += (t.numel() + 7) // 8 * 8
        plan = (tuple(offsets), off, lib.nf_mlp_bwd_rounded_workspace_bytes(D_in, D_hidden, D_out))
        if len(_rounded_plans) < 4096:
            _rounded_plans[key] = plan
    return plan


def _backward_rounded(x, do2, w_in, b_in, w_out, b_out, w_hid, b_hid, need_dx, D_in, D_hidden, D_out, depth=2):
    """Backward of the one-hidden-layer ReLU shapes through ``nf_mlp_bwd_rounded``: the weight gradients come back summed
    in a fixed order and rounded to the parameters' dtype, into one uninitialised buffer (no clearing, no cast kernel).
    ``None`` when the library declines (rows not 8-byte aligned): the caller takes the general path.  The buffer is
    allocated per call: its pieces become the ``.grad`` tensors, which a later backward must not overwrite."""
    lib = _lib.load()
    like = (w_in, b_in, w_out, b_out, w_hid, b_hid)
    offsets, total, ws_bytes = _rounded_plan(lib, like, D_in, D_hidden, D_out)
    flat = torch.empty(total, dtype=w_in.dtype, device=w_in.device)
    base, es = flat.data_ptr(), flat.element_size()
    p = [None if t is None else base + es * o for t, o in zip(like, offsets)]
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=w_in.device)
    x2 = _rows2d(x, D_in)
    dx = x.new_empty(x.shape) if need_dx else None
    rc = lib.nf_mlp_bwd_rounded(
        x2.data_ptr(), x2.stride(0), do2.data_ptr(), do2.stride(0), _lib.ptr(dx), D_in,
        w_in.data_ptr(), _lib.ptr(b_in), _lib.ptr(w_hid), _lib.ptr(b_hid), w_out.data_ptr(), _lib.ptr(b_out),
        p[0], p[1], p[4], p[5], p[2], p[3],
        x2.shape[0], D_in, D_hidden, D_out, depth, _lib.NF_ACT["relu"], _lib.dtype_code(w_in.dtype), _lib.dtype_code(x.dtype),
        ws.data_ptr(), ws_bytes, _lib.current_stream(x.device),
    )
    if rc == _lib.NF_EUNSUPPORTED:
        return None
    _lib.check(rc, "nf_mlp_bwd_rounded")
    g = [None if t is None else flat.as_strided(t.shape, t.stride(), o) if t.is_contiguous() else flat[o:o + t.numel()].view(t.shape)
         for t, o in zip(like, offsets)]
    dw_in, db_in, dw_out, db_out, dw_hid, db_hid = g
    return dx, dw_in, db_in, dw_out, db_out, dw_hid, db_hid, None, None


def fully_fused_mlp(
    x: Tensor,
    w_in: Tensor, b_in: Optional[Tensor],
    w_out: Tensor, b_out: Optional[Tensor],
    w_hid: Optional[Tensor] = None, b_hid: Optional[Tensor] = None,
    activation: str = "relu",
    fp16_acc: bool = False,
) -> Tensor:
    r"""Fully fused forward pass of a small MLP (reference kernel.py:640-686).

    Shapes:
        - x: :math:`(B, L, D_{in})`
        - w_in: :math:`(D_{hidden}, D_{in})`, b_in: :math:`(D_{hidden},)` or ``None``
        - w_out: :math:`(D_{out}, D_{hidden})`, b_out: :math:`(D_{out},)` or ``None``
        - w_hid: :math:`((depth-1) \cdot D_{hidden}, D_{hidden})`, b_hid: :math:`(depth-1, D_{hidden})` or ``None``
        - Output: :math:`(B, L, D_{out})`

    ``activation`` is one of ``"relu"``, ``"relu2"``, ``"silu"``, ``"none"`` and is applied after every
    layer but the last.
    """
    return _fully_fused_mlp.apply(x, w_in, b_in, w_out, b_out, w_hid, b_hid, activation, fp16_acc)
