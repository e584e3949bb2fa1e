"""The hash-encoding oracle under the reference's private names (test infrastructure only).

The reference's tests import ``_cpu_create_corner_offsets``, ``_cpu_embedding_lookup``, ``_cpu_interpolate`` and
``_cpu_hash_encoding`` from ``triton_helpers/layers/hash_encoding/kernel.py`` (``:443-502``; imported at
``tests/test_layers/test_hash_encoding.py:13-26``).  A test suite written against those names finds them here, with the
reference's argument order, evaluated by ``oracle.hash_encoding``.  The shipped package does not carry them: it has no
CPU path.
"""
from __future__ import annotations

import torch
from torch import Tensor

from . import hash_encoding as O


def _cpu_create_corner_offsets(d: int, **kwargs) -> Tensor:
    """Corner ``j`` has offset bit ``(j >> dim) & 1`` (reference kernel.py:443-445)."""
    return O.corner_offsets(d).to(**kwargs)


@torch.no_grad()
def _cpu_embedding_lookup(x: Tensor, pi: Tensor, D: int, T_l: int, N_l: int) -> Tensor:
    """Level-local rows ``[N, 2**D]`` (reference kernel.py:448-462)."""
    return O.corner_rows(x, pi.to(torch.int64), D, T_l, N_l)


def _cpu_interpolate(x: Tensor, e: Tensor, D: int, N_l: int) -> Tensor:
    """``sum_j w_j e[:, j]`` for gathered corner rows ``e [N, 2**D, F]`` (reference kernel.py:465-479)."""
    return O.interpolate(x, e, D, N_l)


def _cpu_hash_encoding(x: Tensor, e: Tensor, pi: Tensor, o: Tensor, D: int, F: int, T: int, L: int, N_min: int, N_max: int) -> Tensor:
    """The per-level loop writing into ``o`` (reference kernel.py:482-502)."""
    assert 1 <= D <= 3, "D must be 1, 2, or 3"
    o[..., : L * F] = O.encode_forward(x, e, pi.to(torch.int64), T, L, N_min, N_max).to(o.dtype)
    return o
