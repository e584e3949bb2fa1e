"""Level geometry of the multiresolution hash table.

Same functions (names, arguments, results) as
``triton_helpers/layers/hash_encoding/helpers.py`` of the reference, plus
``level_geometry`` which packs everything the kernels need into one cached
``nf_hash_geom`` so that nothing is recomputed per launch.
"""
from __future__ import annotations

import math
import sys
from functools import lru_cache
from typing import Final, List, Tuple

import torch
from torch import Tensor

from ..._lib import NF_MAX_DIMS, NF_MAX_LEVELS, HashGeom

EPS: Final = 1e-5


def compute_b(N_min: int, N_max: int, L: int) -> float:
    """Growth factor between consecutive levels (reference helpers.py:12-23)."""
    span = math.log(N_max) - math.log(N_min)
    return float(math.exp(span / (L - 1))) + EPS


@lru_cache(maxsize=256)
def _resolutions(num_levels: int, N_min: int, N_max: int) -> Tuple[int, ...]:
    # float32 power, like the reference's default-dtype tensor arithmetic (helpers.py:37-39)
    base = torch.tensor(compute_b(N_min, N_max, num_levels), dtype=torch.float32)
    level = torch.arange(num_levels)
    return tuple(int(v) for v in torch.floor(torch.pow(base, level) * N_min).to(torch.int64).tolist())


def compute_resolutions(num_levels: int, N_min: int, N_max: int) -> List[int]:
    """Grid resolution ``N_l`` of every level (reference helpers.py:26-39)."""
    return list(_resolutions(num_levels, N_min, N_max))


def compute_embedding_counts(L: int, T: int, D: int, N_min: int, N_max: int) -> List[int]:
    """Rows of every level: ``min((N_l+1)**D, T)`` (reference helpers.py:42-57)."""
    return [min((n + 1) ** D, T) for n in _resolutions(L, N_min, N_max)]


def get_first_hash_level(N_min: int, N_max: int, L: int, T: int, D: int) -> int:
    """First level whose full grid exceeds ``T`` rows; ``L + 1`` if none does (reference helpers.py:60-73)."""
    full = compute_embedding_counts(L, sys.maxsize, D, N_min, N_max)
    for i, t in enumerate(full):
        if t > T:
            return i
    return L + 1


@lru_cache(maxsize=256)
def _starts(L: int, T: int, D: int, N_min: int, N_max: int) -> Tuple[int, ...]:
    # cached: the forward checks the table's size against the last entry on every call
    starts = [0]
    for c in compute_embedding_counts(L, T, D, N_min, N_max):
        starts.append(starts[-1] + c)
    return tuple(starts)


def seek_to_level_embeddings(e: Tensor, l_i: int, L: int, T: int, D: int, N_min: int, N_max: int) -> Tensor:
    """View of level ``l_i``'s rows of a stacked table ``(*, E, F)`` (reference helpers.py:76-98)."""
    starts = _starts(L, T, D, N_min, N_max)
    return e[..., starts[l_i] : starts[l_i + 1], :]


def compute_level_embedding_offset(l_i: int, L: int, T: int, D: int, N_min: int, N_max: int) -> int:
    """First row of level ``l_i`` in the stacked table (reference helpers.py:101-115)."""
    return _starts(L, T, D, N_min, N_max)[l_i]


@lru_cache(maxsize=64)
def level_geometry(T: int, L: int, D: int, F: int, N_min: int, N_max: int) -> HashGeom:
    """All per-level constants as one ``nf_hash_geom`` (cached per configuration)."""
    if not 1 <= D <= NF_MAX_DIMS:
        raise ValueError(f"coordinate dimension {D} outside 1..{NF_MAX_DIMS}")
    if not 1 <= L <= NF_MAX_LEVELS:
        raise ValueError(f"levels {L} outside 1..{NF_MAX_LEVELS}")
    geom = HashGeom()
    geom.dims, geom.feat, geom.levels = D, F, L
    geom.first_hash_level = get_first_hash_level(N_min, N_max, L, T, D)
    geom.max_rows = T
    res = _resolutions(L, N_min, N_max)
    counts = compute_embedding_counts(L, T, D, N_min, N_max)
    starts = _starts(L, T, D, N_min, N_max)
    for l in range(L):
        geom.res[l] = res[l]
        geom.rows[l] = counts[l]
        geom.row_offset[l] = starts[l]
    return geom


def total_rows(T: int, L: int, D: int, N_min: int, N_max: int) -> int:
    return _starts(L, T, D, N_min, N_max)[-1]
