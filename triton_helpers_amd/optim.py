"""Fused Adam step for hash tables (``nf_table_adam_step``).

The reference ships no optimiser.  This one is the neighbour of the encoder's backward: it consumes the float32
gradient table that ``hash_encoding_table_grad`` accumulates, so a training loop keeps ONE persistent float32 gradient
buffer -- cleared by the optimiser step itself -- instead of allocating, zero-filling and down-casting a gradient per step.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _lib


class TableAdam:
    """Adam over one table (any float dtype) with float32 moments and an optional float32 master copy.

    ``step(grad)`` takes the float32 gradient ``(E, F)`` (e.g. the ``out=`` buffer of ``hash_encoding_table_grad``), divides it
    by ``grad_scale`` (the loss scale), applies ``torch.optim.Adam``'s update and, by default, zeroes ``grad`` in the same pass.

    ``skip_nonfinite=True`` (the default) leaves the parameter and the moments of an element untouched when its
    gradient is inf or NaN -- an overflowed loss-scaled step; the encoder's backward marks the rows of an overflowed
    level with NaN -- and ``found_nonfinite`` (a device int32 tensor, cleared by ``step`` before the launch) tells whether
    any element was: the signal ``torch.amp.GradScaler`` uses to lower the loss scale.  (``GradScaler`` skips the whole
    step; here the finite elements are still updated.)
    """

    def __init__(self, table: Tensor, lr: float = 1e-3, betas: Tuple[float, float] = (0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 0.0, master: Optional[bool] = None):
        assert table.is_contiguous() and table.device.type == "cuda", "the table must be a contiguous GPU tensor"
        self.table = table
        self.lr, self.betas, self.eps, self.weight_decay = lr, betas, eps, weight_decay
        if master is None:
            master = table.dtype != torch.float32
        self.master = table.detach().float().clone() if master else None
        self.exp_avg = torch.zeros(table.shape, dtype=torch.float32, device=table.device)
        self.exp_avg_sq = torch.zeros_like(self.exp_avg)
        self.found_nonfinite = torch.zeros(1, dtype=torch.int32, device=table.device)
        self.steps = 0

    @torch.no_grad()
    def step(self, grad: Tensor, grad_scale: float = 1.0, clear_grad: bool = True, skip_nonfinite: bool = True) -> None:
        assert grad.dtype == torch.float32 and grad.is_contiguous() and grad.shape == self.table.shape and grad.device == self.table.device
        self.steps += 1
        lib = _lib.load()
        self.found_nonfinite.zero_()
        flags = (_lib.NF_ADAM_CLEAR_GRAD if clear_grad else 0) | (_lib.NF_ADAM_SKIP_NONFINITE if skip_nonfinite else 0)
        rc = lib.nf_table_adam_step(
            self.table.data_ptr(), _lib.dtype_code(self.table.dtype), _lib.ptr(self.master), grad.data_ptr(), self.exp_avg.data_ptr(),
            self.exp_avg_sq.data_ptr(), self.table.numel(), self.steps, float(self.lr), float(self.betas[0]), float(self.betas[1]),
            float(self.eps), float(self.weight_decay), float(grad_scale), flags, self.found_nonfinite.data_ptr(), _lib.current_stream(self.table.device))
        _lib.check(rc, "nf_table_adam_step")
