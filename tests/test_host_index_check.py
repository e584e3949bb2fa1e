"""CPU-only: the kernels' own index functions, compiled for the host, against the oracle and against adversarial input.

``nf_hash_check_host`` evaluates the inline functions the GPU kernels use (cell clamp, 32-bit wrap-around hashing of the
fast D = 2 / 3 kernels, 64-bit form of the per-(point, level) kernels) on host coordinates.  The reference's counterpart
is its debug build (``tl.device_assert`` under ``TRITON_DEBUG``, hash_encoding/kernel.py:109-122, 151, 227-228, and the
range test tests/test_layers/test_hash_encoding.py:372-392).
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import hash_encoding as O


def _lib():
    from triton_helpers_amd import _lib

    if not _lib.LIB_PATH.exists():
        pytest.skip("libnf_cdna4.so not built (run python -m triton_helpers_amd.build)")
    return _lib, _lib.load()


def _check(x: torch.Tensor, T, L, lo, hi, variant, primes=O.PRIMES, scale=1.0, want_rows=True):
    from triton_helpers_amd.layers.hash_encoding.helpers import level_geometry

    L_, lib = _lib()
    n, D = x.shape
    geom = level_geometry(T, L, D, 2, lo, hi)
    xs = np.ascontiguousarray(x.numpy().astype(np.float32))
    pr = np.asarray(primes[:D] if D <= len(primes) else primes, dtype=np.int64)
    rows = np.empty((n, L, 2**D), dtype=np.int64) if want_rows else None
    bad_rows, bad_coords = ctypes.c_int64(-1), ctypes.c_int64(-1)
    rc = lib.nf_hash_check_host(
        xs.ctypes.data, n, geom, pr.ctypes.data, float(scale), variant,
        None if rows is None else rows.ctypes.data, ctypes.addressof(bad_rows), ctypes.addressof(bad_coords))
    L_.check(rc, "nf_hash_check_host")
    return (None if rows is None else torch.from_numpy(rows)), bad_rows.value, bad_coords.value


GEOMS = [
    # T, L, min_res, max_res, D
    (2**19, 16, 16, 7006, 3),   # BASELINE geometry
    (2**14, 16, 16, 512, 3),    # the reference's default
    (2**14, 8, 4, 256, 2),
    (2**10, 4, 2, 64, 3),
]


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("T,L,lo,hi,D", GEOMS)
def test_rows_equal_the_oracle(T, L, lo, hi, D, variant):
    """Both index forms give the oracle's int64 rows bit for bit (random points plus cell borders and x == 1)."""
    torch.manual_seed(3)
    x = torch.rand(4000, D)
    res = O.level_resolutions(L, lo, hi)
    border = torch.tensor([[k / r] * D for r in res for k in (0, 1, r // 2, r - 1, r)], dtype=torch.float32)
    if D < 3:  # the reference's CPU path indexes one past a dense level at x == 1 in every dimension; keep x < 1 there
        border = border.clamp(max=1.0 - 2**-24)
    x = torch.cat([x, border.clamp(0, 1)])
    got, bad_rows, bad_coords = _check(x, T, L, lo, hi, variant)
    assert bad_rows == 0 and bad_coords == 0
    assert torch.equal(got, O.encode_indices(x, None, T, L, lo, hi))


@pytest.mark.parametrize("T", [7, 1000, 2**19 - 1, 3 * 2**17])
def test_rows_with_level_sizes_that_are_not_powers_of_two(T):
    """Hashed levels of any size take the exact 64-bit remainder (reference ops.py:69-88, kernel.py:147-149)."""
    torch.manual_seed(5)
    x = torch.rand(3000, 3)
    got, bad_rows, _ = _check(x, T, 8, 2, 600, 0)
    assert bad_rows == 0
    assert torch.equal(got, O.encode_indices(x, None, T, 8, 2, 600))
    L_, lib = _lib()
    from triton_helpers_amd.layers.hash_encoding.helpers import level_geometry

    geom = level_geometry(T, 8, 3, 2, 2, 600)
    z = ctypes.c_int64(0)
    xs = np.zeros((1, 3), dtype=np.float32)
    pr = np.asarray(O.PRIMES, dtype=np.int64)
    rc = lib.nf_hash_check_host(xs.ctypes.data, 1, geom, pr.ctypes.data, 1.0, 1, None, ctypes.addressof(z), ctypes.addressof(z))
    assert rc == L_.NF_EUNSUPPORTED and b"power-of-two" in lib.nf_last_error()


def test_reference_literal_tables():
    """The two literal index tables of the reference's tests (tests/test_layers/test_hash_encoding.py:240-251, 285-296)."""
    from tests.test_oracle_hash import DENSE_ROWS, HASHED_ROWS, QUADRANT_X
    from triton_helpers_amd import _lib as L_

    lib = L_.load() if L_.LIB_PATH.exists() else pytest.skip("library not built")
    x = np.asarray(QUADRANT_X, dtype=np.float32)
    pr = np.asarray(O.PRIMES, dtype=np.int64)
    for T, want in ((9, DENSE_ROWS), (7, HASHED_ROWS)):
        geom = L_.HashGeom()
        geom.dims, geom.feat, geom.levels, geom.max_rows = 2, 2, 1, T
        geom.first_hash_level = 0 if T == 7 else 1
        geom.res[0], geom.rows[0], geom.row_offset[0] = 2, T, 0
        rows = np.empty((len(x), 1, 4), dtype=np.int64)
        a, b = ctypes.c_int64(0), ctypes.c_int64(0)
        rc = lib.nf_hash_check_host(x.ctypes.data, len(x), geom, pr.ctypes.data, 1.0, 0, rows.ctypes.data, ctypes.addressof(a), ctypes.addressof(b))
        assert rc == 0 and a.value == 0 and b.value == 0
        assert rows[:, 0, :].tolist() == want


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("T,L,lo,hi,D", GEOMS)
def test_adversarial_coordinates_stay_inside_every_level(T, L, lo, hi, D, variant):
    """Negative, beyond-scale, huge, infinite and NaN coordinates: every corner row stays below its level's size (the
    cell is clamped to [0, N_l]), and the count of out-of-range coordinates is what the reference would assert on."""
    vals = [-1e-7, -0.25, -3.0, 1.0 + 1e-6, 1.5, 17.0, 3e9, -3e9, 1e30, -1e30, float("inf"), float("-inf"), float("nan"), 0.0, 1.0, 0.5]
    g = torch.Generator().manual_seed(1)
    pick = torch.randint(0, len(vals), (5000, D), generator=g)
    x = torch.tensor(vals, dtype=torch.float32)[pick]
    rows, bad_rows, bad_coords = _check(x, T, L, lo, hi, variant)
    assert bad_rows == 0
    inside = (x >= 0) & (x <= 1)
    assert bad_coords == int((~inside).sum())
    counts = torch.tensor(O.level_row_counts(L, T, D, lo, hi))
    assert bool((rows >= 0).all()) and bool((rows < counts[None, :, None]).all())
    # with a scale, the same holds for coordinates in units of the scale
    _, bad_rows, bad_coords = _check(x * 4.0, T, L, lo, hi, variant, scale=4.0, want_rows=False)
    assert bad_rows == 0 and bad_coords == int((~inside).sum())


def test_in_range_cells_are_untouched_by_the_clamp():
    """For coordinates in [0, 1] the clamped cell is floor(x * N_l) itself: x == 1 keeps cell N_l (corner N_l + 1)."""
    x = torch.tensor([[1.0, 1.0, 1.0], [0.0, 0.0, 0.0], [1.0, 0.0, 0.5]])
    rows, bad_rows, bad_coords = _check(x, 2**19, 16, 16, 7006, 1)
    assert bad_rows == 0 and bad_coords == 0
    assert torch.equal(rows, O.encode_indices(x, None, 2**19, 16, 16, 7006))
