"""CPU oracle for the multiresolution hash encoding (test infrastructure only).

Restates, with plain torch on the CPU, the PyTorch path of the reference:
``triton_helpers/layers/hash_encoding/helpers.py`` (level geometry) and
``triton_helpers/layers/hash_encoding/kernel.py:443-502`` (corner offsets,
index lookup, D-linear interpolation, per-level loop).  The backward is the
textbook scatter-add that autograd derives from that forward.

All index arithmetic is int64 and all value arithmetic is float32, like the
reference's CPU functions.
"""
from __future__ import annotations

import math
from typing import List, Sequence, Tuple

import torch
from torch import Tensor

# One prime per spatial dimension (reference kernel.py:24-27).
PRIMES: Tuple[int, int, int] = (1, 2_654_435_761, 805_459_861)


# --------------------------------------------------------------------------
# Level geometry (reference helpers.py)
# --------------------------------------------------------------------------
def growth_factor(min_res: int, max_res: int, levels: int) -> float:
    """Per-level growth ``exp((ln max - ln min)/(levels-1)) + 1e-5`` (helpers.py:12-23)."""
    return float(math.exp((math.log(max_res) - math.log(min_res)) / (levels - 1))) + 1e-5


def level_resolutions(levels: int, min_res: int, max_res: int) -> List[int]:
    """``floor(b**l * min_res)`` evaluated in float32 (helpers.py:26-39).

    The reference builds ``b`` as a default-dtype (float32) 0-dim tensor and
    raises it to an int64 ``arange``; the result is float32.
    """
    b = torch.tensor(growth_factor(min_res, max_res, levels), dtype=torch.float32)
    exponents = torch.arange(levels)
    return torch.floor(torch.pow(b, exponents) * min_res).to(torch.int64).tolist()


def level_row_counts(levels: int, max_rows: int, dims: int, min_res: int, max_res: int) -> List[int]:
    """Rows of each level's table: ``min((N_l+1)**D, T)`` (helpers.py:42-57)."""
    return [min((n + 1) ** dims, max_rows) for n in level_resolutions(levels, min_res, max_res)]


def first_hashed_level(min_res: int, max_res: int, levels: int, max_rows: int, dims: int) -> int:
    """First level with ``(N_l+1)**D > T``; ``levels + 1`` when none (helpers.py:60-73)."""
    for i, n in enumerate(level_resolutions(levels, min_res, max_res)):
        if (n + 1) ** dims > max_rows:
            return i
    return levels + 1


def level_row_offsets(levels: int, max_rows: int, dims: int, min_res: int, max_res: int) -> List[int]:
    """Exclusive prefix sum of the row counts, length ``levels + 1`` (helpers.py:76-115)."""
    out = [0]
    for c in level_row_counts(levels, max_rows, dims, min_res, max_res):
        out.append(out[-1] + c)
    return out


# --------------------------------------------------------------------------
# Per-level pieces (reference kernel.py:443-479)
# --------------------------------------------------------------------------
def corner_offsets(dims: int) -> Tensor:
    """``[2**D, D]`` int64; corner ``j`` has bit ``(j >> d) & 1`` in dim ``d`` (kernel.py:443-445)."""
    j = torch.arange(2 ** dims, dtype=torch.int64)[:, None]
    d = torch.arange(dims, dtype=torch.int64)[None, :]
    return (j >> d) & 1


def corner_rows(x: Tensor, primes: Tensor, dims: int, rows_l: int, res_l: int) -> Tensor:
    """Table row of every cell corner, ``[N, 2**D]`` int64 (kernel.py:448-462).

    cell = floor(x * N_l) in float32.  Dense levels (``(N_l+1)**D <= T_l``) use
    ``sum_d corner_d * N_l**d`` -- the stride is ``N_l``, not ``N_l + 1``.
    Hashed levels use ``(xor_d corner_d * pi_d) mod T_l`` with exact 64-bit products.
    """
    cell = torch.floor(x.to(torch.float32) * res_l).to(torch.int64)
    corners = cell[:, None, :] + corner_offsets(dims)[None]
    if (res_l + 1) ** dims <= rows_l:
        stride = torch.tensor([res_l ** d for d in range(dims)], dtype=torch.int64)
        return (corners * stride).sum(-1)
    prod = corners * primes.to(torch.int64)[:dims]
    h = prod[..., 0]
    for d in range(1, dims):
        h = torch.bitwise_xor(h, prod[..., d])
    return h % rows_l


def corner_weights(x: Tensor, dims: int, res_l: int) -> Tensor:
    """D-linear weights ``[N, 2**D]`` float32 (kernel.py:465-477).

    ``frac = x*N_l - floor(x*N_l)``; the weight of corner ``j`` is the product
    over dims of ``frac_d`` (offset bit set) or ``1 - frac_d`` (clear).
    """
    pos = x.to(torch.float32) * res_l
    frac = (pos - torch.floor(pos))[:, None, :]
    off = corner_offsets(dims)[None]
    w = torch.where(off == 0, 1 - frac, frac)
    return w.prod(-1)


def interpolate(x: Tensor, gathered: Tensor, dims: int, res_l: int) -> Tensor:
    """``sum_j w_j * e_j`` in float32, ``[N, F]`` (kernel.py:479)."""
    w = corner_weights(x, dims, res_l)
    return (w[..., None] * gathered).sum(1)


# --------------------------------------------------------------------------
# Whole encode (reference kernel.py:482-502) and its gradient
# --------------------------------------------------------------------------
def encode_forward(
    x: Tensor,
    table: Tensor,
    primes: Tensor | Sequence[int] | None,
    max_rows: int,
    levels: int,
    min_res: int,
    max_res: int,
    out_dtype: torch.dtype | None = None,
) -> Tensor:
    """Encode ``x [N, D]`` (coordinates in [0, 1]) with ``table [E, F]`` -> ``[N, levels*F]``.

    Float32 accumulation, result stored in ``out_dtype`` (default: the table's
    dtype, as the reference writes into a buffer of the table's dtype).
    """
    n, dims = x.shape
    feat = table.shape[-1]
    assert dims >= 1 and (dims <= 3 or primes is not None), "more than three dimensions need their own primes (kernel.py:537-540)"
    if primes is None:
        primes = PRIMES
    primes = torch.as_tensor(primes, dtype=torch.int64)
    res = level_resolutions(levels, min_res, max_res)
    rows = level_row_counts(levels, max_rows, dims, min_res, max_res)
    offs = level_row_offsets(levels, max_rows, dims, min_res, max_res)
    out = torch.empty(n, levels * feat, dtype=out_dtype or table.dtype)
    for l in range(levels):
        idx = corner_rows(x, primes, dims, rows[l], res[l])
        level_tab = table[offs[l] : offs[l + 1]]
        out[:, l * feat : (l + 1) * feat] = interpolate(x, level_tab[idx], dims, res[l])
    return out


def encode_indices(
    x: Tensor, primes, max_rows: int, levels: int, min_res: int, max_res: int
) -> Tensor:
    """Level-local corner rows for every level, ``[N, levels, 2**D]`` int64."""
    n, dims = x.shape
    if primes is None:
        primes = PRIMES
    primes = torch.as_tensor(primes, dtype=torch.int64)
    res = level_resolutions(levels, min_res, max_res)
    rows = level_row_counts(levels, max_rows, dims, min_res, max_res)
    return torch.stack([corner_rows(x, primes, dims, rows[l], res[l]) for l in range(levels)], 1)


def encode_backward(
    x: Tensor,
    dout: Tensor,
    table_rows: int,
    feat: int,
    primes,
    max_rows: int,
    levels: int,
    min_res: int,
    max_res: int,
) -> Tensor:
    """Gradient of ``encode_forward`` w.r.t. the table, float32 ``[E, F]``.

    ``d_table[offs_l + idx_j, f] += w_j * dout[n, l*F + f]`` (the scatter-add the
    reference's ``_bwd_kernel`` performs, kernel.py:417-432, here with a float32
    product and float32 accumulation).
    """
    n, dims = x.shape
    if primes is None:
        primes = PRIMES
    primes = torch.as_tensor(primes, dtype=torch.int64)
    res = level_resolutions(levels, min_res, max_res)
    rows = level_row_counts(levels, max_rows, dims, min_res, max_res)
    offs = level_row_offsets(levels, max_rows, dims, min_res, max_res)
    grad = torch.zeros(table_rows, feat, dtype=torch.float32)
    g = dout.to(torch.float32)
    for l in range(levels):
        idx = corner_rows(x, primes, dims, rows[l], res[l]) + offs[l]  # [N, C]
        w = corner_weights(x, dims, res[l])  # [N, C]
        contrib = w[..., None] * g[:, None, l * feat : (l + 1) * feat]  # [N, C, F]
        grad.index_add_(0, idx.reshape(-1), contrib.reshape(-1, feat))
    return grad
