"""Pins the hash-encoding oracle (CPU only).

Every check here uses evidence independent of the oracle's own formulas: literal
tables held by the reference's tests, exact rational arithmetic, Python big-int
brute force, a scalar pure-Python trilinear evaluation, torch.autograd, and
invariants of the mathematics.
"""
import json
import math
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import hash_encoding as O

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "hash_geometry.json")))
PI = torch.tensor(O.PRIMES, dtype=torch.int64)

# The six points and both expected tables of the reference
# (tests/test_layers/test_hash_encoding.py:222-251 dense, :285-296 hashed with T=7).
QUADRANT_X = [[0, 0], [0.55, 0.55], [0.45, 0.45], [0.9999, 0.9999], [0.55, 0.45], [0.45, 0.55]]
DENSE_ROWS = [[0, 1, 2, 3], [3, 4, 5, 6], [0, 1, 2, 3], [3, 4, 5, 6], [1, 2, 3, 4], [2, 3, 4, 5]]
HASHED_ROWS = [[0, 1, 5, 4], [4, 0, 4, 1], [0, 1, 5, 4], [4, 0, 4, 1], [1, 2, 4, 0], [5, 4, 3, 4]]


# ---------------------------------------------------------------- geometry
@pytest.mark.parametrize("name", ["bench", "default"])
def test_geometry_golden(name):
    g = GOLDEN[name]
    args = (g["levels"], g["min_res"], g["max_res"])
    assert O.level_resolutions(*args) == g["resolutions"]
    assert O.level_row_counts(g["levels"], g["T"], g["dims"], g["min_res"], g["max_res"]) == g["rows"]
    assert O.first_hashed_level(g["min_res"], g["max_res"], g["levels"], g["T"], g["dims"]) == g["first_hash_level"]
    offs = O.level_row_offsets(g["levels"], g["T"], g["dims"], g["min_res"], g["max_res"])
    assert offs[0] == 0 and offs[-1] == g["total_rows"]
    assert [b - a for a, b in zip(offs, offs[1:])] == g["rows"]


@pytest.mark.parametrize("levels,lo,hi", [(16, 16, 7006), (16, 16, 512), (8, 2, 128), (2, 2, 4), (4, 16, 512)])
def test_resolutions_exact_rational(levels, lo, hi):
    """floor(N_min * b^l) with b rounded to float32, evaluated exactly."""
    b = Fraction(float(np.float32(O.growth_factor(lo, hi, levels))))
    got = O.level_resolutions(levels, lo, hi)
    for l in range(levels):
        v = b**l * lo
        n = v.numerator // v.denominator
        frac = float(v - n)
        if l > 0 and min(frac, 1 - frac) < 2e-6 * float(v):
            continue  # a float32 pow may legitimately land on either side
        assert got[l] == n, (l, got[l], n)
    assert got[0] == lo and got[-1] in (hi, hi - 1, hi + 1)


def test_growth_factor_closed_form():
    assert O.growth_factor(16, 512, 16) == pytest.approx(2 ** (1 / 3) + 1e-5, rel=1e-12)
    assert O.growth_factor(16, 7006, 16) == pytest.approx(1.500005686, abs=1e-8)


def test_no_hash_needed_returns_levels_plus_one():
    # reference helpers.py:70-72
    assert O.first_hashed_level(2, 4, 2, 10**9, 2) == 3


# ---------------------------------------------------------------- corner offsets / rows
def test_corner_offsets_literal():
    # reference tests/test_layers/test_hash_encoding.py:40-45
    assert O.corner_offsets(2).tolist() == [[0, 0], [1, 0], [0, 1], [1, 1]]
    assert O.corner_offsets(3).tolist() == [
        [0, 0, 0], [1, 0, 0], [0, 1, 0], [1, 1, 0], [0, 0, 1], [1, 0, 1], [0, 1, 1], [1, 1, 1]]


def test_rows_dense_literal():
    x = torch.tensor(QUADRANT_X, dtype=torch.float32)
    assert O.corner_rows(x, PI, 2, 9, 2).tolist() == DENSE_ROWS


def test_rows_hashed_literal():
    x = torch.tensor(QUADRANT_X, dtype=torch.float32)
    assert O.corner_rows(x, PI, 2, 7, 2).tolist() == HASHED_ROWS


def _brute_rows(x_np, dims, rows_l, res_l):
    out = []
    for p in x_np:
        cell = [int(math.floor(float(np.float32(c) * np.float32(res_l)))) for c in p]
        r = []
        for j in range(2**dims):
            corner = [cell[d] + ((j >> d) & 1) for d in range(dims)]
            if (res_l + 1) ** dims <= rows_l:
                r.append(sum(corner[d] * res_l**d for d in range(dims)))
            else:
                h = 0
                for d in range(dims):
                    h ^= corner[d] * O.PRIMES[d]
                r.append(h % rows_l)
        out.append(r)
    return out


@pytest.mark.parametrize(
    "dims,res_l,rows_l",
    [(2, 16, 17**2), (3, 16, 17**2), (3, 16, 17**2 - 2), (3, 128, 129**2), (3, 128, 129**2 - 1), (3, 100, 129**2),
     (3, 101, 1048576), (3, 7006, 2**19), (1, 50, 51), (1, 5000, 64), (3, 8, 9**3), (3, 8, 9**3 - 2), (3, 8, 512)],
)
def test_rows_bigint_bruteforce(dims, res_l, rows_l):
    """Cases follow the reference's matrix (test_hash_encoding.py:337-349) plus the bench geometry."""
    torch.manual_seed(0)
    x = torch.rand(64, dims)
    got = O.corner_rows(x, PI, dims, rows_l, res_l)
    assert got.tolist() == _brute_rows(x.numpy(), dims, rows_l, res_l)
    assert int(got.min()) >= 0 and int(got.max()) < rows_l


@pytest.mark.parametrize("prime,cell,m,expected", [(1, 10, 7, 3), (2**10, 2**10, 2**5, 0), (2_654_435_761, 8, 700, 488)])
def test_hashed_row_is_exact_product_mod(prime, cell, m, expected):
    """The reference's (x*y) % m literals (tests/test_ops.py:245-255, e.g. 2654435761*8 % 700 = 488)
    seen through a 1-D hashed level: corner 0 of cell c maps to (c*pi) % T."""
    res = 2048
    x = torch.tensor([[(cell + 0.5) / res]], dtype=torch.float32)
    row = O.corner_rows(x, torch.tensor([prime]), 1, m, res)[0, 0].item()
    assert row == expected == (prime * cell) % m


# ---------------------------------------------------------------- interpolation
@pytest.mark.parametrize("coord,idx", [((0, 0, 0), 0), ((1, 1, 1), 0), ((0.9999, 0.9999, 0.9999), 7), ((0.9999, 0.9999, 0), 3)])
def test_interpolate_corner_pick(coord, idx):
    # reference test_hash_encoding.py:109-134 (res 1; x = 1 lands on corner 0 of the next cell)
    torch.manual_seed(0)
    x = torch.tensor(coord, dtype=torch.float32).repeat(10, 1)
    e = torch.randn(10, 8, 2)
    torch.testing.assert_close(O.interpolate(x, e, 3, 1), e[:, idx], rtol=0, atol=1e-3)


def test_interpolate_mean_at_centre():
    # reference test_hash_encoding.py:136-153
    torch.manual_seed(0)
    e = torch.randn(10, 8, 2)
    x = torch.full((10, 3), 0.5)
    torch.testing.assert_close(O.interpolate(x, e, 3, 1), e.mean(1))


@pytest.mark.parametrize("dims", [1, 2, 3])
def test_weights_partition_of_unity_and_textbook(dims):
    torch.manual_seed(1)
    x = torch.rand(50, dims)
    res = 13
    w = O.corner_weights(x, dims, res)
    torch.testing.assert_close(w.sum(1), torch.ones(50), rtol=1e-6, atol=1e-6)
    assert (w >= 0).all()
    # scalar textbook D-linear weights in float64
    for n in range(50):
        fr = [float(x[n, d]) * res - math.floor(float(x[n, d]) * res) for d in range(dims)]
        for j in range(2**dims):
            ref = 1.0
            for d in range(dims):
                ref *= fr[d] if (j >> d) & 1 else 1 - fr[d]
            assert abs(float(w[n, j]) - ref) < 2e-5


# ---------------------------------------------------------------- whole encode
def _scalar_encode(x, table, T, L, lo, hi):
    """Pure-Python float64 evaluation, independent of the tensor code."""
    n, dims = x.shape
    F = table.shape[1]
    b = Fraction(float(np.float32(O.growth_factor(lo, hi, L))))
    out = np.zeros((n, L * F))
    off = 0
    for l in range(L):
        v = b**l * lo
        res = int(v.numerator // v.denominator)  # exact floor; independent of any float pow
        rows_l = min((res + 1) ** dims, T)
        for i in range(n):
            pos = [float(np.float32(x[i, d]) * np.float32(res)) for d in range(dims)]
            cell = [int(math.floor(p)) for p in pos]
            fr = [p - c for p, c in zip(pos, cell)]
            for j in range(2**dims):
                corner = [cell[d] + ((j >> d) & 1) for d in range(dims)]
                w = 1.0
                for d in range(dims):
                    w *= fr[d] if (j >> d) & 1 else 1 - fr[d]
                if (res + 1) ** dims <= rows_l:
                    r = sum(corner[d] * res**d for d in range(dims))
                else:
                    h = 0
                    for d in range(dims):
                        h ^= corner[d] * O.PRIMES[d]
                    r = h % rows_l
                out[i, l * F : (l + 1) * F] += w * table[off + r]
        off += rows_l
    return out


@pytest.mark.parametrize("dims,T,L,lo,hi", [(2, 25, 2, 2, 4), (2, 81, 8, 2, 128), (3, 2**10, 4, 4, 64), (3, 2**14, 16, 16, 512)])
def test_encode_forward_vs_scalar(dims, T, L, lo, hi):
    torch.manual_seed(0)
    E = O.level_row_offsets(L, T, dims, lo, hi)[-1]
    table = torch.randn(E, 2)
    x = torch.rand(12, dims)
    got = O.encode_forward(x, table, None, T, L, lo, hi)
    ref = _scalar_encode(x.numpy(), table.double().numpy(), T, L, lo, hi)
    np.testing.assert_allclose(got.numpy(), ref, rtol=1e-4, atol=1e-5)


def test_encode_constant_table_gives_constant():
    g = GOLDEN["default"]
    table = torch.full((g["total_rows"], 2), 0.375)
    x = torch.rand(100, 3)
    out = O.encode_forward(x, table, None, g["T"], 16, 16, 512)
    torch.testing.assert_close(out, torch.full_like(out, 0.375), rtol=1e-6, atol=0)


def test_encode_levels_and_features_independent():
    torch.manual_seed(0)
    g = GOLDEN["default"]
    offs = O.level_row_offsets(16, g["T"], 3, 16, 512)
    table = torch.randn(g["total_rows"], 2)
    x = torch.rand(40, 3)
    base = O.encode_forward(x, table, None, g["T"], 16, 16, 512)
    t2 = table.clone()
    t2[offs[5] : offs[6], 1] += 1.0  # touch feature 1 of level 5 only
    out = O.encode_forward(x, t2, None, g["T"], 16, 16, 512)
    changed = (out != base).any(0)
    assert changed.nonzero().flatten().tolist() == [11]
    torch.testing.assert_close(out[:, 11], base[:, 11] + 1.0, rtol=1e-5, atol=1e-5)


def test_encode_fp16_table_output_dtype():
    g = GOLDEN["default"]
    table = (torch.randn(g["total_rows"], 2)).half()
    out = O.encode_forward(torch.rand(8, 3), table, None, g["T"], 16, 16, 512)
    assert out.dtype == torch.float16 and out.shape == (8, 32)


# ---------------------------------------------------------------- backward
@pytest.mark.parametrize("dims,T,L,lo,hi", [(2, 81, 8, 2, 128), (3, 2**10, 4, 4, 64), (3, 2**14, 16, 16, 512)])
def test_encode_backward_vs_autograd(dims, T, L, lo, hi):
    torch.manual_seed(0)
    E = O.level_row_offsets(L, T, dims, lo, hi)[-1]
    table = torch.randn(E, 2, requires_grad=True)
    x = torch.rand(300, dims)
    dout = torch.randn(300, L * 2)
    O.encode_forward(x, table, None, T, L, lo, hi).backward(dout)
    got = O.encode_backward(x, dout, E, 2, None, T, L, lo, hi)
    torch.testing.assert_close(got, table.grad, rtol=1e-5, atol=1e-5)


def test_encode_backward_column_sums():
    """Weights sum to one, so level l / feature f of the table gradient sums to sum_n dout[n, l*F+f]."""
    torch.manual_seed(0)
    g = GOLDEN["default"]
    offs = O.level_row_offsets(16, g["T"], 3, 16, 512)
    x = torch.rand(500, 3)
    dout = torch.randn(500, 32)
    grad = O.encode_backward(x, dout, g["total_rows"], 2, None, g["T"], 16, 16, 512)
    for l in range(16):
        torch.testing.assert_close(grad[offs[l] : offs[l + 1]].sum(0), dout[:, 2 * l : 2 * l + 2].sum(0), rtol=1e-4, atol=1e-4)
