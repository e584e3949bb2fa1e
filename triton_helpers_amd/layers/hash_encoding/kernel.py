"""Instant-NGP multiresolution hash encoding on MI355X.

Drop-in for ``triton_helpers/layers/hash_encoding/kernel.py`` of the reference:
same ``hash_encoding(...)`` functional, same ``HashEncoding`` autograd Function
(argument order of ``forward``, 11-tuple returned by ``backward``), same
assertions.  The Triton launches are replaced by ``nf_hash_encode_fwd`` /
``nf_hash_encode_bwd`` of ``libnf_cdna4.so``.

Differences, all supersets or accuracy improvements:
  * the level scaling follows the reference's PyTorch path (``x * N_l`` per
    level, reference kernel.py:450,466) rather than the Triton kernel's
    cumulative rescale, so corner indices equal the CPU reference bit for bit;
  * the table gradient is accumulated in float32 and rounded once to the
    table's dtype (the reference adds in the table's dtype, kernel.py:432,636);
  * ``divider`` / ``bwd_divider`` are accepted and validated but have no effect:
    one launch covers all levels and keeps L2 locality by itself.
"""
from __future__ import annotations

import math
from typing import Any, Dict, Final, Optional, Tuple

import torch
from torch import Tensor

from ... import _lib
from .helpers import (
    compute_b,
    compute_embedding_counts,
    compute_level_embedding_offset,
    compute_resolutions,
    get_first_hash_level,
    level_geometry,
    seek_to_level_embeddings,
    total_rows,
)

# One prime per spatial dimension, as in the paper (reference kernel.py:24-27)
PI_1: Final = 1
PI_2: Final = 2_654_435_761
PI_3: Final = 805_459_861

# Kept for API presence; the launch here does not depend on them.
DIVIDER_CONFIGS: Dict[Any, int] = {}
BWD_DIVIDER_CONFIGS: Dict[Any, int] = {}

_REPACK_MIN_POINTS = 4096  # batches from which misaligned output / gradient rows go through a packed buffer
_FLAGS = 0  # test hook: _lib.NF_HASH_FORCE_GENERIC / NF_HASH_FORCE_ATOMIC / NF_HASH_FORCE_PLANES select other kernels


# ---------------------------------------------------------------------------
# Launch helpers
# ---------------------------------------------------------------------------
_default_primes: Dict[torch.device, Tensor] = {}


def _primes_for(device: torch.device) -> Tensor:
    p = _default_primes.get(device)
    if p is None:
        p = torch.tensor([PI_1, PI_2, PI_3], dtype=torch.int64, device=device)
        _default_primes[device] = p
    return p


def _flat_coords(coords: Tensor) -> Tensor:
    """``(..., D) -> (N, D)`` view when the layout allows, else a copy."""
    return coords.reshape(-1, coords.shape[-1])


def _launch_forward(coords2d: Tensor, embeddings: Tensor, pi: Tensor, out2d: Tensor, T: int, min_res: int,
                    max_res: int, levels: int, scale: float) -> None:
    N, D = coords2d.shape
    F = embeddings.shape[-1]
    geom = level_geometry(T, levels, D, F, min_res, max_res)
    lib = _lib.load()
    rc = lib.nf_hash_encode_fwd(
        coords2d.data_ptr(), _lib.dtype_code(coords2d.dtype), coords2d.stride(0), coords2d.stride(1),
        embeddings.data_ptr(), _lib.dtype_code(embeddings.dtype), out2d.data_ptr(), out2d.stride(0), N,
        geom, pi.data_ptr(), float(scale), _FLAGS, _lib.current_stream(coords2d.device),
    )
    _lib.check(rc, "nf_hash_encode_fwd")


def _launch_backward(coords2d: Tensor, do2d: Tensor, de: Tensor, pi: Tensor, T: int, min_res: int, max_res: int,
                     levels: int, scale: float) -> None:
    N, D = coords2d.shape
    F = de.shape[-1]
    geom = level_geometry(T, levels, D, F, min_res, max_res)
    lib = _lib.load()
    # scratch for the LDS-tile backward; torch's caching allocator makes this free after the first call
    ws_bytes = lib.nf_hash_encode_bwd_workspace_bytes(N, geom, _lib.dtype_code(do2d.dtype), _FLAGS)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=coords2d.device) if ws_bytes > 0 else None
    rc = lib.nf_hash_encode_bwd(
        coords2d.data_ptr(), _lib.dtype_code(coords2d.dtype), coords2d.stride(0), coords2d.stride(1),
        do2d.data_ptr(), _lib.dtype_code(do2d.dtype), do2d.stride(0), de.data_ptr(), N,
        geom, pi.data_ptr(), float(scale), _lib.ptr(ws), ws_bytes, _FLAGS, _lib.current_stream(coords2d.device),
    )
    _lib.check(rc, "nf_hash_encode_bwd")


def _as_rows(t: Tensor, width: int) -> Tensor:
    """2-D view ``(N, width)`` with unit inner stride (copies only when the layout forces it)."""
    t2 = t.reshape(-1, width)
    # rows that overlap (an expanded / broadcast tensor has row stride 0) or a strided inner dimension: copy
    if t2.stride(1) != 1 or (t2.shape[0] > 1 and t2.stride(0) < width):
        t2 = t2.contiguous()
    return t2


def hash_encoding_table_grad(
    coords: Tensor,
    do: Tensor,
    num_embeddings: int,
    d_embed: int,
    pi: Optional[Tensor] = None,
    max_entries_per_level: int = 2**14,
    min_res: int = 16,
    max_res: int = 512,
    levels: int = 16,
    scale: float = 1.0,
    out: Optional[Tensor] = None,
) -> Tensor:
    """Float32 table gradient ``(E, F)`` for upstream gradient ``do (..., >= levels*F)``.

    This is what ``HashEncoding.backward`` computes before autograd rounds it to
    the table's dtype; callers that keep float32 master gradients use it directly.
    ``out`` (float32, ``(E, F)``) is accumulated into when given.
    """
    if pi is None:
        pi = _primes_for(coords.device)
    assert pi.numel() >= coords.shape[-1], "Pi must have at least D_in elements"
    de = out if out is not None else torch.zeros(num_embeddings, d_embed, dtype=torch.float32, device=coords.device)
    assert de.dtype == torch.float32 and de.is_contiguous() and de.shape == (num_embeddings, d_embed)
    coords2d = _flat_coords(coords)
    do2d = _as_rows(do, do.shape[-1])
    if do2d.shape[0] >= _REPACK_MIN_POINTS and ((do2d.stride(0) * do2d.element_size()) % 16 != 0 or do2d.data_ptr() % 16 != 0):
        # gradient rows off 16-byte boundaries (the output carried appended features): the LDS-tile kernels read whole
        # aligned rows, so the encoding's columns are packed first (one pass instead of scattered atomics per corner)
        do2d = do2d[:, : levels * d_embed].contiguous()
    _launch_backward(coords2d, do2d, de, pi, max_entries_per_level, min_res, max_res, levels, scale)
    return de


class HashEncoding(torch.autograd.Function):
    """Autograd Function with the reference's signature (reference kernel.py:509-675)."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.float16)
    def forward(
        ctx,
        coords: Tensor,
        embeddings: Tensor,
        pi: Optional[Tensor],
        features: Optional[Tensor],
        max_entries_per_level: int,
        min_res: int,
        max_res: int,
        levels: int,
        divider: Optional[int] = None,
        bwd_divider: Optional[int] = None,
        scale: float = 1.0,
    ) -> Tensor:
        D_in = coords.shape[-1]
        D_feature = features.shape[-1] if features is not None else 0
        D_embed = embeddings.shape[-1]

        assert coords.is_floating_point(), "Coords must be float"

        if pi is None:
            if D_in > 3:
                raise ValueError("Pi must be provided for more than 3 dimensions")
            pi = _primes_for(coords.device)

        assert isinstance(pi, Tensor)
        assert pi.ndim == 1, "Pi must be a 1-dimensional tensor"
        assert pi.numel() >= D_in, "Pi must have at least D_in elements"

        if features is not None:
            assert isinstance(features, Tensor)
            assert (
                features.shape[:-1] == coords.shape[:-1]
            ), "Features must have the same shape as coords, except for the last dimension"

        assert not coords.requires_grad, "Gradients not supported for coords"
        assert features is None or not features.requires_grad, "Gradients not supported for features"
        assert not pi.requires_grad, "Gradients not supported for pi"

        devices = {coords.device, embeddings.device, pi.device, features.device if features is not None else None}
        devices = {d for d in devices if d is not None}
        assert len(devices) == 1 and all(
            d.type == "cuda" for d in devices
        ), f"All tensors must be on the same device: {devices}"

        assert levels & (levels - 1) == 0, "Levels must be a power of 2"
        for name, div in (("Divider", divider), ("Backward divider", bwd_divider)):
            if div is not None:
                assert 1 <= div <= levels, f"{name} must be between 1 and {levels}"
                assert div & (div - 1) == 0, f"{name} must be a power of 2"
        assert embeddings.ndim == 2, "Embeddings must have shape (E, D_embed)"
        need = total_rows(max_entries_per_level, levels, D_in, min_res, max_res)
        assert embeddings.shape[0] >= need, f"Embedding table has {embeddings.shape[0]} rows, geometry needs {need}"
        if pi.dtype != torch.int64:
            pi = pi.to(torch.int64)

        D_out = D_embed * levels + D_feature
        table = embeddings.detach()
        if not table.is_contiguous():
            table = table.contiguous()
        coords2d = _flat_coords(coords.detach())
        if features is not None and coords2d.shape[0] >= _REPACK_MIN_POINTS and (D_out * embeddings.element_size()) % 16 != 0:
            # appended features that leave the output rows off 16-byte boundaries (three view-direction components, say):
            # the fast kernels write whole aligned rows, so the encoding goes to a buffer of its own and one
            # concatenation builds the output (a pass over the output instead of the per-(point, level) kernel)
            enc = embeddings.new_empty(*coords.shape[:-1], D_embed * levels)
            _launch_forward(coords2d, table, pi, enc.view(-1, D_embed * levels), max_entries_per_level, min_res, max_res, levels, scale)
            o = torch.cat([enc, features.to(enc.dtype)], dim=-1)
        else:
            o = embeddings.new_empty(*coords.shape[:-1], D_out)
            _launch_forward(coords2d, table, pi, o.view(-1, D_out), max_entries_per_level, min_res, max_res, levels, scale)
            if features is not None:
                o[..., D_embed * levels :] = features

        ctx.save_for_backward(coords, embeddings, pi)
        ctx.max_entries_per_level = max_entries_per_level
        ctx.min_res = min_res
        ctx.max_res = max_res
        ctx.levels = levels
        ctx.scale = scale
        ctx.bwd_divider = bwd_divider
        return o

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    @torch.no_grad()
    def backward(ctx, do: Tensor):
        coords, embeddings, pi = ctx.saved_tensors
        de = hash_encoding_table_grad(
            coords, do, embeddings.shape[0], embeddings.shape[1], pi,
            ctx.max_entries_per_level, ctx.min_res, ctx.max_res, ctx.levels, ctx.scale,
        )
        # float32 accumulators; autograd rounds them once to the table's dtype
        return None, de, None, None, None, None, None, None, None, None, None

    @staticmethod
    def _possible_dividers(levels: int) -> Tuple[int, ...]:
        return tuple(2**i for i in range(int(math.log2(levels)) + 1))


def hash_encoding(
    coord: Tensor,
    embeddings: Tensor,
    features: Optional[Tensor] = None,
    pi: Optional[Tensor] = None,
    max_entries_per_level: int = 2**14,
    min_res: int = 16,
    max_res: int = 512,
    levels: int = 16,
    divider: Optional[int] = None,
    bwd_divider: Optional[int] = None,
    scale: float = 1.0,
) -> Tensor:
    r"""Multi-resolution hash encoding as defined in Instant NGP (reference kernel.py:678-728).

    Args:
        coord: Coordinates on the range :math:`[0, scale]`, shape :math:`(..., D)`.
        embeddings: Stacked per-level tables, shape :math:`(E, D_e)`.
        features: Optional features :math:`(..., D_f)` appended to the output.
        pi: Hashing primes :math:`(D,)` int64; defaults to the paper's for ``D <= 3``.
        max_entries_per_level: Cap ``T`` on the rows of one level.
        min_res, max_res: Coarsest / finest grid resolution.
        levels: Number of levels (a power of two).
        divider, bwd_divider: Accepted for compatibility; no effect.
        scale: Upper end of the coordinate range.

    Returns:
        :math:`(..., L \times D_e + D_f)` tensor of the tables' dtype.
    """
    return HashEncoding.apply(
        coord, embeddings, pi, features, max_entries_per_level, min_res, max_res, levels, divider, bwd_divider, scale
    )


def hash_encoding_indices(
    coord: Tensor,
    pi: Optional[Tensor] = None,
    max_entries_per_level: int = 2**14,
    min_res: int = 16,
    max_res: int = 512,
    levels: int = 16,
    scale: float = 1.0,
    return_weights: bool = False,
    fast: bool = False,
):
    """Level-local table rows ``(N, L, 2**D)`` int64 (and float32 weights) computed by the device code.

    The device-side counterpart of the reference's ``embedding_lookup`` test kernels
    (reference tests/test_layers/test_hash_encoding.py:178-215).  ``fast=True`` evaluates the 32-bit index arithmetic
    of the fast kernels (forward sweep, binned backward; 2-D / 3-D, power-of-two hashed levels) instead of the 64-bit
    form of the per-(point, level) kernels; the two must agree bit for bit.
    """
    coords2d = _flat_coords(coord)
    N, D = coords2d.shape
    if pi is None:
        pi = _primes_for(coord.device)
    assert pi.numel() >= D, "Pi must have at least D_in elements"
    geom = level_geometry(max_entries_per_level, levels, D, 1, min_res, max_res)
    rows = torch.empty(N, levels, 2**D, dtype=torch.int64, device=coord.device)
    w = torch.empty(N, levels, 2**D, dtype=torch.float32, device=coord.device) if return_weights else None
    lib = _lib.load()
    entry = lib.nf_hash_encode_indices_fast if fast else lib.nf_hash_encode_indices
    rc = entry(
        coords2d.data_ptr(), _lib.dtype_code(coords2d.dtype), coords2d.stride(0), coords2d.stride(1),
        rows.data_ptr(), _lib.ptr(w), N, geom, pi.data_ptr(), float(scale), _lib.current_stream(coord.device),
    )
    _lib.check(rc, "nf_hash_encode_indices_fast" if fast else "nf_hash_encode_indices")
    return (rows, w) if return_weights else rows
