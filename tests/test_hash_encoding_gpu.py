"""GPU parity of the hash-encoding kernels against the CPU oracle (through the C ABI).

Tolerances: corner rows bit-exact; float32 forward rtol 1e-5 (plus an absolute
floor of 1e-5 x the largest table magnitude, for outputs that cancel to ~0);
backward rtol 1e-3 (atomic order differs) with atol 1e-4 for N(0,1) upstream
gradients; 16-bit tables: the reference's own atol 1e-2 and, tighter, one ulp
of the 16-bit result.
"""
import json
import os

import pytest
import torch

from oracle import hash_encoding as O

pytestmark = pytest.mark.gpu

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "hash_geometry.json")))
DEV = "cuda"


def _hk():
    from triton_helpers_amd.layers.hash_encoding import kernel

    return kernel


def _table(T, L, D, lo, hi, F=2, dtype=torch.float32, amp=1e-4, seed=0):
    g = torch.Generator().manual_seed(seed)
    E = O.level_row_offsets(L, T, D, lo, hi)[-1]
    return ((torch.rand(E, F, generator=g) * 2 - 1) * amp).to(dtype)


CASES = [
    # (N, D, F, T, L, lo, hi, scale)  -- the first six follow the reference's matrix
    # (tests/test_layers/test_hash_encoding.py:400-410), the rest add the bench geometry and odd shapes
    (4, 2, 2, 25, 2, 2, 4, 1.0),
    (4, 2, 2, 81, 8, 2, 128, 1.0),
    (4, 3, 2, 2**14, 16, 16, 512, 1.0),
    (100, 3, 2, 2**14, 16, 16, 512, 1.0),
    (100, 3, 2, 2**20, 16, 16, 512, 1.0),
    (100, 3, 2, 2**14, 16, 16, 512, 2.0),
    (4099, 3, 2, 2**19, 16, 16, 7006, 1.0),
    (777, 3, 2, 5000, 8, 4, 300, 1.0),  # T not a power of two: exact 64-bit remainder
    (513, 3, 4, 2**12, 4, 8, 64, 1.0),
    (1000, 3, 8, 2**14, 8, 16, 512, 1.0),     # rows of 4 / 8 features: 8- / 16-byte gathers in the staged forward
    (2049, 3, 4, 2**16, 16, 16, 2048, 2.0),
    (300, 1, 2, 64, 4, 8, 512, 1.0),
    (300, 3, 1, 2**12, 8, 16, 256, 0.5),
]


@pytest.mark.parametrize("N,D,F,T,L,lo,hi,scale", CASES)
def test_corner_rows_bit_exact(N, D, F, T, L, lo, hi, scale):
    torch.manual_seed(0)
    x = torch.rand(N, D)
    want = O.encode_indices(x, None, T, L, lo, hi)
    xs = x * scale if scale != 1.0 else x
    if scale not in (1.0, 2.0):  # keep only points that survive the round trip through the scale exactly
        keep = ((xs / scale) == x).all(1)
        x, xs, want = x[keep], xs[keep], want[keep]
    got, w = _hk().hash_encoding_indices(xs.to(DEV), None, T, lo, hi, L, scale=scale, return_weights=True)
    assert torch.equal(got.cpu(), want)
    res = O.level_resolutions(L, lo, hi)
    wref = torch.stack([O.corner_weights(x, D, r) for r in res], 1)
    torch.testing.assert_close(w.cpu(), wref, rtol=1e-6, atol=1e-7)
    # the 32-bit index arithmetic of the fast kernels, evaluated on the device, where it applies
    if D in (2, 3) and (T & (T - 1)) == 0:
        fast, wf = _hk().hash_encoding_indices(xs.to(DEV), None, T, lo, hi, L, scale=scale, return_weights=True, fast=True)
        assert torch.equal(fast.cpu(), want)
        assert torch.equal(wf, w), "the fast kernels' weights are the generic kernels' weights, bit for bit"


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("D,T,L,lo,hi", [(4, 2**12, 4, 2, 16), (5, 2**12, 4, 2, 12), (6, 2**13, 4, 2, 8), (4, 3000, 2, 3, 9)])
def test_four_to_six_dimensions(D, T, L, lo, hi, dtype):
    """More than three dimensions (the reference takes any D once the caller brings the primes, kernel.py:537-545): the
    per-(point, level) kernels with 16, 32 and 64 corners per cell, dense and hashed levels, one table size that is not a
    power of two.  Corner rows bit for bit, forward and table gradient against the oracle."""
    hk = _hk()
    torch.manual_seed(D)
    N, F = 500, 2
    pi = torch.tensor([1, 2654435761, 805459861, 3674653429, 2097192037, 1434869437], dtype=torch.int64)
    x = torch.rand(N, D)
    x[0] = 0.0
    x[1] = 1.0
    offs = O.level_row_offsets(L, T, D, lo, hi)
    E = offs[-1]
    assert any(offs[i + 1] - offs[i] < T for i in range(L)) and any(offs[i + 1] - offs[i] == T for i in range(L)), "dense and hashed levels"
    keep = torch.ones(N, dtype=torch.bool)
    keep[1] = False  # x == 1 in every dimension: the reference's CPU path indexes one row past a dense level there
    want_rows = O.encode_indices(x[keep], pi, T, L, lo, hi)
    got_rows = hk.hash_encoding_indices(x.to(DEV), pi.to(DEV), T, lo, hi, L)
    assert got_rows.shape == (N, L, 2**D)
    assert torch.equal(got_rows.cpu()[keep], want_rows)
    assert int(got_rows.max()) < T and int(got_rows.min()) >= 0
    table = ((torch.rand(E, F) * 2 - 1)).to(dtype)
    want = O.encode_forward(x[keep], table.float(), pi, T, L, lo, hi)
    got = hk.hash_encoding(x.to(DEV), table.to(DEV), None, pi.to(DEV), T, lo, hi, L)
    rtol, atol = (1e-5, 1e-6) if dtype == torch.float32 else (2.0**-10, 1e-4)
    torch.testing.assert_close(got.cpu().float()[keep], want, rtol=rtol, atol=atol)
    do = torch.randn(N, L * F).to(dtype)
    do[1] = 0
    want_g = O.encode_backward(x[keep], do[keep], E, F, pi, T, L, lo, hi)
    got_g = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, F, pi.to(DEV), T, lo, hi, L)
    torch.testing.assert_close(got_g.cpu(), want_g, rtol=1e-4, atol=1e-5 * max(1.0, float(want_g.abs().max())))


def test_corner_rows_fast_path_upper_edge():
    """x == scale in every dimension: the fast kernels' index functions keep the zero-weight corner inside the level,
    like the 64-bit form."""
    for D in (2, 3):
        x = torch.ones(5, D, device=DEV)
        x[1:] = torch.rand(4, D, device=DEV)
        a = _hk().hash_encoding_indices(x, None, 2**12, 16, 64, 4)
        b = _hk().hash_encoding_indices(x, None, 2**12, 16, 64, 4, fast=True)
        assert torch.equal(a, b)


def test_corner_rows_reference_literals():
    """The reference's literal tables (test_hash_encoding.py:240-251, 285-296) straight from the device code."""
    from tests.test_oracle_hash import DENSE_ROWS, HASHED_ROWS, QUADRANT_X

    x = torch.tensor(QUADRANT_X, dtype=torch.float32, device=DEV)
    # a single level of resolution 2: min_res = max_res is degenerate for the growth factor, so use L=2 and read level 0
    dense = _hk().hash_encoding_indices(x, None, 9, 2, 4, 2)[:, 0]
    hashed = _hk().hash_encoding_indices(x, None, 7, 2, 4, 2)[:, 0]
    assert dense.cpu().tolist() == DENSE_ROWS
    assert hashed.cpu().tolist() == HASHED_ROWS
    # the dense table again from the fast kernels' 32-bit arithmetic: T = 16 leaves level 0 (resolution 2, nine rows)
    # dense and gives the hashed level 1 the power-of-two size that form needs (the hashed literal table uses T = 7,
    # which only the 64-bit remainder form covers)
    dense_fast = _hk().hash_encoding_indices(x, None, 16, 2, 4, 2, fast=True)[:, 0]
    assert dense_fast.cpu().tolist() == DENSE_ROWS


@pytest.mark.parametrize("N,D,F,T,L,lo,hi,scale", CASES)
@pytest.mark.parametrize("force_generic", [False, True])
def test_forward_fp32_tables(N, D, F, T, L, lo, hi, scale, force_generic, monkeypatch):
    hk = _hk()
    monkeypatch.setattr(hk, "_FLAGS", 1 if force_generic else 0)
    torch.manual_seed(0)
    x = torch.rand(N, D)
    table = _table(T, L, D, lo, hi, F)
    want = O.encode_forward(x, table, None, T, L, lo, hi)
    got = hk.hash_encoding(x.to(DEV) * scale, table.to(DEV), None, None, T, lo, hi, L, scale=scale)
    assert got.dtype == torch.float32 and got.shape == (N, L * F)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-5 * 1e-4)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,D,F,T,L,lo,hi,scale", CASES)
def test_forward_16bit_tables(N, D, F, T, L, lo, hi, scale, dtype):
    hk = _hk()
    torch.manual_seed(0)
    x = torch.rand(N, D)
    table = _table(T, L, D, lo, hi, F, dtype=dtype, amp=1.0)
    want32 = O.encode_forward(x, table.float(), None, T, L, lo, hi)
    got = hk.hash_encoding(x.to(DEV) * scale, table.to(DEV), None, None, T, lo, hi, L, scale=scale)
    assert got.dtype == dtype
    # reference tolerance (test_hash_encoding.py:432)
    torch.testing.assert_close(got.cpu().float(), want32, rtol=0, atol=1e-2)
    # tighter: the float32 result rounded once to the 16-bit type, allow one ulp
    eps = 2.0**-10 if dtype == torch.float16 else 2.0**-7
    torch.testing.assert_close(got.cpu().float(), want32, rtol=eps, atol=eps * 1e-3)


def test_tiled_and_generic_agree_bitwise(monkeypatch):
    hk = _hk()
    g = GOLDEN["bench"]
    torch.manual_seed(1)
    x = torch.rand(5000, 3, device=DEV)
    table = _table(g["T"], 16, 3, 16, 7006, dtype=torch.float16, amp=1.0).to(DEV)
    monkeypatch.setattr(hk, "_FLAGS", 0)
    a = hk.hash_encoding(x, table, None, None, g["T"], 16, 7006, 16)
    monkeypatch.setattr(hk, "_FLAGS", 1)
    b = hk.hash_encoding(x, table, None, None, g["T"], 16, 7006, 16)
    assert torch.equal(a, b)


@pytest.mark.parametrize("D,F,dtype,off", [(3, 4, torch.float32, 0), (3, 8, torch.float32, 0), (3, 6, torch.float32, 0), (2, 6, torch.float16, 0),
                                            (4, 2, torch.bfloat16, 0), (1, 2, torch.float32, 0), (3, 24, torch.float16, 0), (3, 4, torch.float32, 2),
                                            (3, 8, torch.float16, 4), (3, 3, torch.float16, 0)])
def test_generic_forward_reads_rows_in_pieces(D, F, dtype, off, monkeypatch):
    """The per-(point, level) forward reads a row in pieces of up to 16 bytes where the row width and the alignment of
    table and output allow it (float32 rows of 4 features: one load per corner instead of four).  Bit-equal to the
    one-feature-at-a-time form (flag 1); `off` elements of misalignment of table and output make it fall back to
    narrower pieces; 1.0e6 points on the float32 four-feature case keep the many-workgroup path covered elsewhere."""
    from triton_helpers_amd import _lib

    hk = _hk()
    torch.manual_seed(9)
    N, T, L, lo, hi = 3001, 2**12, 4, 4, 40
    pi = torch.tensor([1, 2654435761, 805459861, 3674653429], dtype=torch.int64)
    x = torch.rand(N, D)
    E = O.level_row_offsets(L, T, D, lo, hi)[-1]
    store = torch.zeros(E * F + 8, dtype=dtype, device=DEV)
    table = store[off : off + E * F].view(E, F)
    table.copy_((torch.rand(E, F) * 2 - 1).to(dtype))
    outs = {}
    for flag in (0, _lib.NF_HASH_FORCE_GENERIC):
        monkeypatch.setattr(hk, "_FLAGS", flag)
        outs[flag] = hk.hash_encoding(x.to(DEV), table, None, pi.to(DEV), T, lo, hi, L)
    assert torch.equal(outs[0], outs[_lib.NF_HASH_FORCE_GENERIC])
    want = O.encode_forward(x, table.float().cpu(), pi, T, L, lo, hi)
    rtol, atol = (1e-5, 1e-6) if dtype == torch.float32 else ((2.0**-10, 1e-4) if dtype == torch.float16 else (2.0**-7, 1e-3))
    torch.testing.assert_close(outs[0].cpu().float(), want, rtol=rtol, atol=atol)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("N,D", [(5000, 3), (2**18 + 33, 3), (2**18 + 33, 2)])
def test_thirty_two_levels(N, D, dtype, monkeypatch):
    """More than sixteen levels run as one forward call per sixteen levels on their own columns of the output: bit-equal
    to the per-(point, level) kernel (flag 1) and within the storage rounding of the oracle; the backward against the
    oracle on a sample of the batch."""
    from triton_helpers_amd import _lib

    hk = _hk()
    torch.manual_seed(13)
    T, L, lo, hi = 2**15, 32, 4, 4096
    x = torch.rand(N, D, device=DEV)
    table = _table(T, L, D, lo, hi, dtype=dtype, amp=1.0).to(DEV)
    E = table.shape[0]
    outs = {}
    for flag in (0, _lib.NF_HASH_FORCE_GENERIC):
        monkeypatch.setattr(hk, "_FLAGS", flag)
        outs[flag] = hk.hash_encoding(x, table, None, None, T, lo, hi, L)
    assert outs[0].shape == (N, 64) and torch.equal(outs[0], outs[_lib.NF_HASH_FORCE_GENERIC])
    idx = torch.randperm(N)[:3000]
    want = O.encode_forward(x[idx.to(DEV)].cpu(), table.float().cpu(), None, T, L, lo, hi)
    eps = 1e-5 if dtype == torch.float32 else 2.0**-10
    torch.testing.assert_close(outs[0][idx.to(DEV)].cpu().float(), want, rtol=eps, atol=eps * 1e-3 if dtype != torch.float32 else 1e-6)
    monkeypatch.setattr(hk, "_FLAGS", 0)
    xs = x[idx.to(DEV)].contiguous().repeat(4, 1)[:9000]     # 9000 points: the sorted-record backward
    do = torch.randn(xs.shape[0], 64, device=DEV).to(dtype)
    want_g = O.encode_backward(xs.cpu(), do.cpu(), E, 2, None, T, L, lo, hi)
    got_g = hk.hash_encoding_table_grad(xs, do, E, 2, None, T, lo, hi, L).cpu()
    torch.testing.assert_close(got_g, want_g, rtol=1e-3, atol=1e-4 * float(want_g.abs().max()))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,D,T,L,lo,hi", [(1, 3, 2**19, 16, 16, 7006), (257, 3, 2**19, 16, 16, 7006), (5000, 3, 2**17, 2, 16, 700),
                                            (8191, 2, 2**19, 16, 16, 7006), (60001, 3, 2**19, 16, 16, 7006), (100000, 2, 2**15, 8, 8, 300)])
def test_small_batches_one_thread_per_point_and_level(N, D, T, L, lo, hi, dtype, monkeypatch):
    """Batches below the sweep's minimum (forward) and below the sorted-record kernels' minimum (backward) run one
    thread per (point, level) on 16-bit pairs in two and three dimensions.  Forward: bit-equal to
    the generic kernel (flag 1) and, where it applies, to the LDS-staged tile kernel (flag 8), and within one ulp of
    the oracle.  Backward: against the oracle and the generic kernel, a coordinate scale included."""
    from triton_helpers_amd import _lib

    hk = _hk()
    torch.manual_seed(8)
    scale = 2.5
    x = torch.rand(N, D)
    x[: N // 8, 0] = 1.0
    table = _table(T, L, D, lo, hi, 2, dtype=dtype, amp=1.0)
    E = table.shape[0]
    xs = (x * scale).to(DEV)
    outs = {}
    for flag in (0, _lib.NF_HASH_FORCE_GENERIC, _lib.NF_HASH_FWD_STAGED):
        monkeypatch.setattr(hk, "_FLAGS", flag)
        outs[flag] = hk.hash_encoding(xs, table.to(DEV), None, None, T, lo, hi, L, scale=scale)
    assert torch.equal(outs[0], outs[_lib.NF_HASH_FORCE_GENERIC]) and torch.equal(outs[0], outs[_lib.NF_HASH_FWD_STAGED])
    want = O.encode_forward(xs.cpu() / scale, table.float(), None, T, L, lo, hi)
    eps = 2.0**-10 if dtype == torch.float16 else 2.0**-7
    torch.testing.assert_close(outs[0].cpu().float(), want, rtol=eps, atol=eps * 1e-3)

    do = torch.randn(N, L * 2).to(dtype)
    do[::7] = 0  # rows of zero gradient are skipped
    want_g = O.encode_backward(xs.cpu() / scale, do, E, 2, None, T, L, lo, hi)
    grads = {}
    for flag in (_lib.NF_HASH_FORCE_ATOMIC, _lib.NF_HASH_FORCE_GENERIC):
        monkeypatch.setattr(hk, "_FLAGS", flag)
        grads[flag] = hk.hash_encoding_table_grad(xs, do.to(DEV), E, 2, None, T, lo, hi, L, scale=scale).cpu()
    peak = float(want_g.abs().max())
    for got in grads.values():
        torch.testing.assert_close(got, want_g, rtol=1e-4, atol=1e-5 * peak)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("L,hi", [(16, 7006), (8, 512), (4, 64)])
def test_forward_kernels_agree_bitwise_at_sweep_sizes(L, hi, dtype, monkeypatch):
    """From 2^18 points on the forward takes the register-resident level sweep; flag 8 selects the LDS-staged
    tile kernel (16-bit tables) and flag 1 the per-(point, level) kernel: all three must produce the same bits, also
    for a ragged last workgroup and a coordinate scale."""
    hk = _hk()
    g = GOLDEN["bench"]
    N = 2**18 + 77
    torch.manual_seed(2)
    x = torch.rand(N, 3, device=DEV) * 2.5
    table = _table(g["T"], L, 3, 16, hi, dtype=dtype, amp=1.0).to(DEV)
    outs = []
    for flags in (0, 8, 1):
        monkeypatch.setattr(hk, "_FLAGS", flags)
        outs.append(hk.hash_encoding(x, table, None, None, g["T"], 16, hi, L, scale=2.5))
    assert torch.equal(outs[0], outs[1])
    assert torch.equal(outs[0], outs[2])
    idx = torch.randperm(N)[:2048]
    want = O.encode_forward(x[idx.to(DEV)].cpu() / 2.5, table.float().cpu(), None, g["T"], L, 16, hi)
    eps = {torch.float16: 2.0**-10, torch.bfloat16: 2.0**-7, torch.float32: 1e-5}[dtype]
    # (float32: sums of eight products of order one cancel to anything; 1e-6 is a few of their roundings)
    torch.testing.assert_close(outs[0][idx.to(DEV)].cpu().float(), want, rtol=eps, atol=1e-6 if dtype == torch.float32 else eps * 1e-3)


@pytest.mark.parametrize("dtype,N", [(torch.float16, 2**20 + 1537), (torch.float32, 2**19 + 1537)])
def test_forward_sweep_in_several_launches(dtype, N, monkeypatch):
    """Large batches run the level sweep as several launches (2^20 points each with 16-bit tables, 2^19 with float32
    tables): a ragged batch that crosses the boundary, written into rows of a wider output (stride 40), must equal the
    per-(point, level) kernel bit for bit."""
    hk = _hk()
    g = GOLDEN["bench"]
    torch.manual_seed(4)
    x = torch.rand(N, 3, device=DEV)
    feats = torch.randn(N, 8, device=DEV).to(dtype)  # appended columns
    table = _table(g["T"], 16, 3, 16, 7006, dtype=dtype, amp=1.0).to(DEV)
    outs = []
    for flags in (0, 1):
        monkeypatch.setattr(hk, "_FLAGS", flags)
        outs.append(hk.hash_encoding(x, table, feats, None, g["T"], 16, 7006, 16))
    assert outs[0].shape == (N, 40)
    assert torch.equal(outs[0], outs[1])
    edge = N - 1537
    idx = torch.cat([torch.arange(edge - 512, edge + 512), torch.arange(N - 256, N)])
    want = O.encode_forward(x[idx.to(DEV)].cpu(), table.float().cpu(), None, g["T"], 16, 16, 7006)
    rtol, atol = (1e-5, 1e-6) if dtype == torch.float32 else (2.0**-10, 1e-6)
    torch.testing.assert_close(outs[0][idx.to(DEV), :32].cpu().float(), want, rtol=rtol, atol=atol)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("L,hi", [(16, 7006), (8, 512)])
def test_forward_sweep_two_dimensions(L, hi, dtype, monkeypatch):
    """Two-dimensional coordinates take the same level sweep over four corners (16-bit tables): same bits as the
    per-(point, level) kernel (flag 1), ragged last workgroup and a coordinate scale included."""
    hk = _hk()
    g = GOLDEN["bench"]
    N = 2**18 + 77
    torch.manual_seed(3)
    x = torch.rand(N, 2, device=DEV) * 2.5
    table = _table(g["T"], L, 2, 16, hi, dtype=dtype, amp=1.0).to(DEV)
    outs = []
    for flags in (0, 1):
        monkeypatch.setattr(hk, "_FLAGS", flags)
        outs.append(hk.hash_encoding(x, table, None, None, g["T"], 16, hi, L, scale=2.5))
    assert torch.equal(outs[0], outs[1])
    idx = torch.randperm(N)[:2048]
    want = O.encode_forward(x[idx.to(DEV)].cpu() / 2.5, table.float().cpu(), None, g["T"], L, 16, hi)
    eps = {torch.float16: 2.0**-10, torch.bfloat16: 2.0**-7}[dtype]
    torch.testing.assert_close(outs[0][idx.to(DEV)].cpu().float(), want, rtol=eps, atol=eps * 1e-3)


def test_forward_config0_full_size():
    """BASELINE configs[0]: N=65536, L=16, F=2, T=2^19, fp32 table U(-1e-4, 1e-4), seed 0."""
    g = GOLDEN["bench"]
    torch.manual_seed(0)
    x = torch.rand(65536, 3)
    table = (torch.rand(g["total_rows"], 2) * 2 - 1) * 1e-4
    want = O.encode_forward(x, table, None, g["T"], 16, 16, 7006)
    got = _hk().hash_encoding(x.to(DEV), table.to(DEV), None, None, g["T"], 16, 7006, 16)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-9)
    want_rows = O.encode_indices(x, None, g["T"], 16, 16, 7006)
    rows = _hk().hash_encoding_indices(x.to(DEV), None, g["T"], 16, 7006, 16)
    assert torch.equal(rows.cpu(), want_rows)
    fast = _hk().hash_encoding_indices(x.to(DEV), None, g["T"], 16, 7006, 16, fast=True)
    assert torch.equal(fast.cpu(), want_rows), "the fast kernels' device index arithmetic differs from the oracle"


@pytest.mark.parametrize("N,D,F,T,L,lo,hi,scale", CASES + [(65536, 3, 2, 2**20, 16, 16, 512, 1.0), (131072, 3, 2, 2**14, 16, 16, 512, 1.0)])
@pytest.mark.parametrize("do_dtype,flags", [(torch.float32, 1), (torch.float32, 0), (torch.float16, 0), (torch.float16, 1), (torch.float16, 2)])
def test_backward_vs_oracle(N, D, F, T, L, lo, hi, scale, do_dtype, flags, monkeypatch):
    """flags: 0 = default dispatch (LDS-tile kernels from 8192 points), 1 = generic, 2 = scattered atomics."""
    hk = _hk()
    monkeypatch.setattr(hk, "_FLAGS", flags)
    torch.manual_seed(0)
    x = torch.rand(N, D)
    E = O.level_row_offsets(L, T, D, lo, hi)[-1]
    do = torch.randn(N, L * F).to(do_dtype)
    want = O.encode_backward(x, do, E, F, None, T, L, lo, hi)
    got = hk.hash_encoding_table_grad(x.to(DEV) * scale, do.to(DEV), E, F, None, T, lo, hi, L, scale)
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.cpu(), want, rtol=1e-3, atol=1e-4)


@pytest.mark.parametrize("do_dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize(
    "N,T,L,lo,hi",
    [
        (40000, 2**14, 16, 16, 512),    # every hashed level is exactly one LDS tile
        (33000, 2**19, 16, 16, 7006),   # bench geometry: 32 tiles per hashed level, dense levels of 1, 1, 4 and 11 tiles
        (50001, 2**16, 8, 16, 2048),    # 4 tiles per hashed level, ragged point count
        (40000, 2**19, 4, 4096, 30000), # resolutions above the tile size: the x corner moves the tile id
        (45000, 2**12, 4, 8, 64),       # hashed levels smaller than a tile
        (40000, 12345, 8, 16, 512),     # hashed level size not a power of two: exact 64-bit remainder
    ],
)
@pytest.mark.parametrize("variant", [0, 4])  # 0: binned records, 4: bit-planes (NF_HASH_FORCE_PLANES)
def test_backward_lds_tile_path(N, T, L, lo, hi, do_dtype, variant):
    """Both LDS-tile backwards against the oracle and against the scattered-atomic kernel.  A float32 upstream
    gradient takes the binned records with 16-byte records; the bit-plane variant is 16-bit only."""
    hk = _hk()
    if do_dtype == torch.float32 and variant == 4:
        pytest.skip("the bit-plane variant takes 16-bit upstream gradients")
    torch.manual_seed(3)
    x = torch.rand(N, 3)
    x[:7] = torch.tensor([[0.0, 0.0, 0.0], [1.0, 1.0, 1.0], [1.0, 0.0, 0.5], [0.999999, 0.5, 0.25], [0.5, 1.0, 0.0],
                          [0.25, 0.25, 1.0], [1.0, 1.0, 0.0]])
    E = O.level_row_offsets(L, T, 3, lo, hi)[-1]
    do = torch.randn(N, L * 2).to(do_dtype)
    do[100:200] = 0  # rows with no upstream gradient are skipped
    want = O.encode_backward(x, do, E, 2, None, T, L, lo, hi)
    hk._FLAGS = variant
    got = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, 2, None, T, lo, hi, L)
    hk._FLAGS = 2
    try:
        ref = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, 2, None, T, lo, hi, L)
    finally:
        hk._FLAGS = 0
    torch.testing.assert_close(got.cpu(), want, rtol=1e-3, atol=1e-4)
    torch.testing.assert_close(got, ref, rtol=1e-3, atol=1e-4)


@pytest.mark.parametrize("do_dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("N,T,L,lo,hi", [(40000, 2**14, 16, 16, 512), (70001, 2**19, 8, 16, 4096), (33000, 2**12, 4, 8, 64),
                                        (40000, 5000, 4, 8, 256)])
def test_backward_binned_two_dimensions(N, T, L, lo, hi, do_dtype):
    """2-D coordinates take the binned backward too (two x-pairs per point and level): against the oracle and the
    scattered-atomic kernel, with points on the cell borders."""
    hk = _hk()
    torch.manual_seed(4)
    x = torch.rand(N, 2)
    x[:5] = torch.tensor([[0.0, 0.0], [1.0, 1.0], [1.0, 0.0], [0.999999, 0.5], [0.5, 1.0]])
    E = O.level_row_offsets(L, T, 2, lo, hi)[-1]
    do = torch.randn(N, L * 2).to(do_dtype)
    want = O.encode_backward(x, do, E, 2, None, T, L, lo, hi)
    got = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, 2, None, T, lo, hi, L)
    hk._FLAGS = 2
    try:
        ref = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, 2, None, T, lo, hi, L)
    finally:
        hk._FLAGS = 0
    scale = max(1.0, float(want.abs().max()))
    torch.testing.assert_close(got.cpu(), want, rtol=1e-3, atol=1e-4 * scale)
    torch.testing.assert_close(got, ref, rtol=1e-3, atol=1e-4 * scale)


@pytest.mark.parametrize("do_dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("N,D,F,T,L,lo,hi", [(40000, 3, 4, 2**14, 16, 16, 512), (35001, 3, 8, 2**16, 8, 16, 1024),
                                            (40000, 2, 4, 5000, 4, 8, 256), (33000, 3, 6, 2**12, 4, 8, 64),
                                            # one feature, and odd numbers of them: the last feature goes alone
                                            (40000, 3, 1, 2**14, 16, 16, 512), (33000, 3, 3, 2**12, 4, 8, 64),
                                            (35001, 2, 5, 5000, 4, 8, 256), (33000, 3, 1, 2**19, 16, 16, 7006),
                                            # rows of an odd number of elements are not 4-byte aligned: scattered atomics
                                            (33000, 3, 3, 2**12, 5, 8, 64)])
def test_backward_binned_wide_rows(N, D, F, T, L, lo, hi, do_dtype):
    """Tables with 1 to 8 features per row: the binned backward takes the features two at a time (one fill and
    one accumulation per pair).  Against the oracle and the scattered-atomic kernel."""
    hk = _hk()
    from triton_helpers_amd import _lib
    from triton_helpers_amd.layers.hash_encoding.helpers import level_geometry

    # every one of these geometries has a sorted-records plan (the kernel is taken when the rows are 4-byte aligned)
    geom = level_geometry(T, L, D, F, lo, hi)
    assert _lib.load().nf_hash_encode_bwd_workspace_bytes(N, geom, _lib.dtype_code(do_dtype), 0) > 0
    torch.manual_seed(5)
    x = torch.rand(N, D)
    x[0] = 0.0
    x[1] = 1.0
    E = O.level_row_offsets(L, T, D, lo, hi)[-1]
    do = torch.randn(N, L * F).to(do_dtype)
    want = O.encode_backward(x, do, E, F, None, T, L, lo, hi)
    got = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, F, None, T, lo, hi, L)
    hk._FLAGS = 2
    try:
        ref = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, F, None, T, lo, hi, L)
    finally:
        hk._FLAGS = 0
    scale = max(1.0, float(want.abs().max()))
    torch.testing.assert_close(got.cpu(), want, rtol=1e-3, atol=1e-4 * scale)
    torch.testing.assert_close(got, ref, rtol=1e-3, atol=1e-4 * scale)


@pytest.mark.parametrize("do_dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("T,L,lo,hi", [(2**22, 16, 16, 7006), (2**24, 4, 256, 2048)])
def test_backward_binned_large_tables(T, L, lo, hi, do_dtype):
    """Tables with more bins than the count and fill kernels hold counters for: the levels go through the pipeline
    in groups (three groups at 2^22 rows per level, one level per group at 2^24).  Against the oracle."""
    hk = _hk()
    N = 40000
    torch.manual_seed(6)
    x = torch.rand(N, 3)
    x[0] = 0.0
    x[1] = 1.0
    E = O.level_row_offsets(L, T, 3, lo, hi)[-1]
    do = torch.randn(N, L * 2).to(do_dtype)
    want = O.encode_backward(x, do, E, 2, None, T, L, lo, hi)
    got = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, 2, None, T, lo, hi, L)
    scale = max(1.0, float(want.abs().max()))
    torch.testing.assert_close(got.cpu(), want, rtol=1e-3, atol=1e-4 * scale)


@pytest.mark.parametrize("do_dtype", [torch.float16, torch.float32])
def test_backward_binned_clustered_points(do_dtype):
    """Clustered input: a few cells receive everything, so their bins are cut into several accumulation tasks
    (atomic flush), and x = 8191 sits on a bin border of the dense levels / has 13 trailing ones on hashed levels, so
    corner pairs are split into two records."""
    hk = _hk()
    torch.manual_seed(5)
    N, T, L, lo, hi = 150000, 2**19, 16, 16, 16384
    x = torch.rand(N, 3)
    x[: N // 2] = torch.tensor([0.3, 0.6, 0.9]) + 1e-4 * torch.rand(N // 2, 3)       # one cell on the coarse levels
    x[N // 2: N // 2 + 20000, 0] = (8191.0 + 0.5 * torch.rand(20000)) / 16384.0       # x cell 8191 at resolution 16384
    E = O.level_row_offsets(L, T, 3, lo, hi)[-1]
    do = torch.randn(N, L * 2).to(do_dtype)
    want = O.encode_backward(x, do, E, 2, None, T, L, lo, hi)
    got = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, 2, None, T, lo, hi, L)
    # sums of up to 75000 terms: compare with a tolerance scaled to the largest row
    torch.testing.assert_close(got.cpu(), want, rtol=1e-3, atol=1e-4 * float(want.abs().max()))
    # bins cut into several tasks meet in float atomics, so two runs agree to rounding only
    again = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, 2, None, T, lo, hi, L)
    torch.testing.assert_close(got, again, rtol=1e-5, atol=1e-6 * float(want.abs().max()))


@pytest.mark.parametrize("do_dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_backward_binned_dense_levels_of_several_bins(do_dtype):
    """Dense 3-D levels of 2 to 48 bins (resolutions 24 .. 72 in a table of 2^19 rows): with 16-bit gradients a point
    leaves one record per level, and a second one where its cell reaches into the next bin.  Points on grid nodes
    (weights exactly 0 and 1), on the upper edge and clustered in one cell are part of the input."""
    hk = _hk()
    torch.manual_seed(11)
    N, T, L, lo, hi = 120000, 2**19, 6, 24, 72
    x = torch.rand(N, 3)
    x[:5000] = torch.randint(0, 73, (5000, 3)).float() / 72.0          # nodes of the finest level
    x[5000:10000] = torch.randint(0, 25, (5000, 3)).float() / 24.0     # nodes of the coarsest level
    x[10000:30000] = torch.tensor([0.71, 0.33, 0.52]) + 1e-3 * torch.rand(20000, 3)
    x[30000:30100] = 1.0
    offs = O.level_row_offsets(L, T, 3, lo, hi)
    E = offs[-1]
    assert all(offs[i + 1] - offs[i] < T for i in range(L)), "every level is dense"
    do = torch.randn(N, L * 2).to(do_dtype)
    want = O.encode_backward(x, do, E, 2, None, T, L, lo, hi)
    got = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, 2, None, T, lo, hi, L)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-3, atol=1e-4 * float(want.abs().max()))
    # rows that no point's cell touches stay exactly zero
    assert float(got.cpu()[want == 0].abs().max()) == 0.0


@pytest.mark.parametrize(
    "N,D,F,T,L,lo,hi,do_dtype",
    [
        (150001, 3, 2, 2**14, 16, 16, 512, torch.float16),   # the reference's default geometry (kernel.py:682-686)
        (140000, 3, 2, 2**14, 16, 16, 512, torch.float32),
        (131072, 2, 2, 2**13, 8, 16, 512, torch.bfloat16),
        (135000, 3, 4, 12345, 8, 8, 256, torch.float16),     # two passes of feature pairs, exact 64-bit remainder
        (133000, 3, 1, 2**14, 4, 16, 128, torch.float16),    # odd feature counts: the last pair has one feature
        (133000, 3, 3, 2**14, 4, 16, 128, torch.float32),
        (2**21 + 5000, 3, 2, 2**14, 2, 16, 64, torch.float16),  # more than one piece of 2^21 points
        (4099, 3, 2, 2**14, 16, 16, 512, torch.float16),        # batches too small for the record kernels take the walk as well
        (20000, 3, 2, 2**14, 16, 16, 512, torch.float32),
    ],
)
def test_backward_without_records(N, D, F, T, L, lo, hi, do_dtype, monkeypatch):
    """Tables whose levels are at most two bins (2^14 rows) take the walk without records: a workgroup per level and
    feature (or per level, for a level of one bin) hashes a slice of the points and adds every corner to its LDS tile.
    Against the oracle, against the sorted-record kernels (flag NF_HASH_BWD_RECORDS), with a smaller workspace, and
    with rows that no point touches left exactly zero."""
    from triton_helpers_amd import _lib

    hk = _hk()
    torch.manual_seed(5)
    x = torch.rand(N, D)
    x[:500, 0] = 1.0                                   # the upper edge of the first coordinate
    x[500:1000] = torch.randint(0, hi, (500, D)).float() / hi   # grid nodes of the finest level: weights exactly 0 and 1
    k = min(N, 20000)
    x[1000:k] = torch.rand(1, D) * 0.9 + 1e-3 * torch.rand(k - 1000, D)  # a cluster in one cell of the coarse levels
    E = O.level_row_offsets(L, T, D, lo, hi)[-1]
    do = torch.randn(N, L * F).to(do_dtype)
    want = O.encode_backward(x, do, E, F, None, T, L, lo, hi)
    geom = hk.level_geometry(T, L, D, F, lo, hi)
    lib = _lib.load()
    need = lib.nf_hash_encode_bwd_workspace_bytes(N, geom, _lib.dtype_code(do_dtype), 0)
    need_records = lib.nf_hash_encode_bwd_workspace_bytes(N, geom, _lib.dtype_code(do_dtype), _lib.NF_HASH_BWD_RECORDS)
    assert 0 < need and (need < need_records or need_records == 0), (need, need_records)  # (no records below 8192 points)
    got = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, F, None, T, lo, hi, L).cpu()
    monkeypatch.setattr(hk, "_FLAGS", _lib.NF_HASH_BWD_RECORDS)
    records = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, F, None, T, lo, hi, L).cpu()
    peak = float(want.abs().max())
    torch.testing.assert_close(got, want, rtol=1e-3, atol=1e-5 * peak)   # float weights: tighter than the records' bound
    torch.testing.assert_close(records, want, rtol=1e-3, atol=1e-4 * peak)
    touched = O.encode_backward(x, torch.ones_like(do, dtype=torch.float32), E, F, None, T, L, lo, hi) != 0
    assert float(got[~touched].abs().max()) == 0.0 if bool((~touched).any()) else True


@pytest.mark.parametrize(
    "N,D,F,T,L,lo,hi,do_dtype",
    [
        (30000, 1, 2, 2**12, 8, 16, 16000, torch.float16),   # dense and hashed 1-D levels
        (9000, 4, 2, 2**13, 4, 2, 24, torch.float16),        # 4-D: 16 corners per cell
        (12000, 4, 4, 5000, 2, 3, 9, torch.float32),         # a table size that is not a power of two, two feature pairs
        (5000, 4, 1, 2**14, 8, 2, 40, torch.bfloat16),
        # larger 4-D tables: the sorted-record kernels, once per corner of the fourth coordinate
        (9000, 4, 2, 2**17, 4, 4, 40, torch.float16),        # dense levels of several bins and hashed ones
        (40000, 4, 2, 2**19, 8, 2, 64, torch.float16),
        (12000, 4, 4, 50000, 2, 3, 30, torch.float32),       # a size that is not a power of two: exact 64-bit remainder
        (20000, 4, 3, 2**16, 2, 8, 20, torch.bfloat16),
        (9000, 5, 2, 2**16, 2, 2, 8, torch.float16),         # five and six dimensions: four and eight passes
        (8500, 6, 2, 2**15, 2, 2, 5, torch.float32),
    ],
)
def test_backward_without_records_in_one_and_four_dimensions(N, D, F, T, L, lo, hi, do_dtype, monkeypatch):
    """Small tables walk the points without records in one to four dimensions; other tables in four to six dimensions
    run the 3-D record kernels once per corner of the extra coordinates (their term joins the hash, the dense index and
    the weights).  The alternative is scattered atomics (2^20 points: 18 ms in 1-D, 38 ms in 4-D).  Against the oracle
    and against the atomic kernels (flag NF_HASH_FORCE_ATOMIC)."""
    from triton_helpers_amd import _lib

    hk = _hk()
    torch.manual_seed(12)
    pi = torch.tensor([1, 2654435761, 805459861, 3674653429, 2097192037, 1434869437], dtype=torch.int64)
    x = torch.rand(N, D).clamp(max=0.999999)
    x[:300] = (torch.randint(0, hi, (300, D)).float() / hi).clamp(max=0.999999)   # grid nodes: weights exactly 0 and 1
    x[300:3000] = (torch.rand(1, D) * 0.9 + 1e-3 * torch.rand(2700, D)).clamp(max=0.999999)  # a cluster
    x[3000] = 0.0
    E = O.level_row_offsets(L, T, D, lo, hi)[-1]
    do = torch.randn(N, L * F).to(do_dtype)
    want = O.encode_backward(x, do, E, F, pi[:D], T, L, lo, hi)
    geom = hk.level_geometry(T, L, D, F, lo, hi)
    lib = _lib.load()
    assert lib.nf_hash_encode_bwd_workspace_bytes(N, geom, _lib.dtype_code(do_dtype), 0) > 0
    if D == 1:
        assert lib.nf_hash_encode_bwd_workspace_bytes(N, geom, _lib.dtype_code(do_dtype), _lib.NF_HASH_BWD_RECORDS) == 0
    got = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, F, pi[:D].to(DEV), T, lo, hi, L).cpu()
    monkeypatch.setattr(hk, "_FLAGS", _lib.NF_HASH_FORCE_ATOMIC)
    atomic = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, F, pi[:D].to(DEV), T, lo, hi, L).cpu()
    peak = float(want.abs().max())
    records = max(O.level_row_counts(L, T, D, lo, hi)) > 2 * 8192   # more than two bins on some level: sorted records
    torch.testing.assert_close(got, want, rtol=1e-3, atol=(1e-4 if records else 1e-5) * peak)
    torch.testing.assert_close(atomic, want, rtol=1e-3, atol=1e-4 * peak)
    touched = O.encode_backward(x, torch.ones_like(do, dtype=torch.float32), E, F, pi[:D], T, L, lo, hi) != 0
    if bool((~touched).any()):
        assert float(got[~touched].abs().max()) == 0.0


def test_backward_without_records_nonfinite_gradient():
    """An inf in the upstream gradient of one level: that level's touched rows come out NaN, as from the record kernels,
    and every other level is unaffected."""
    from triton_helpers_amd import _lib

    hk = _hk()
    torch.manual_seed(6)
    N, D, F, T, L, lo, hi = 140000, 3, 2, 2**14, 4, 16, 128
    x = torch.rand(N, D)
    offs = O.level_row_offsets(L, T, D, lo, hi)
    E = offs[-1]
    do = torch.randn(N, L * F).half()
    clean = O.encode_backward(x, do, E, F, None, T, L, lo, hi)
    do[777, 2 * 2] = float("inf")
    got = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, F, None, T, lo, hi, L).cpu()
    hk_flags = hk._FLAGS
    try:
        hk._FLAGS = _lib.NF_HASH_BWD_RECORDS
        records = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, F, None, T, lo, hi, L).cpu()
    finally:
        hk._FLAGS = hk_flags
    lvl = slice(offs[2], offs[3])
    assert torch.equal(torch.isnan(got), torch.isnan(records))
    assert bool(torch.isnan(got[lvl]).any()) and not bool(torch.isnan(got[: offs[2]]).any()) and not bool(torch.isnan(got[offs[3] :]).any())
    keep = ~torch.isnan(got)
    torch.testing.assert_close(got[keep], clean[keep], rtol=1e-3, atol=1e-5 * float(clean.abs().max()))


@pytest.mark.parametrize("level", [1, 2])
@pytest.mark.parametrize("do_dtype", [torch.float16, torch.float32])
def test_backward_binned_nonfinite_gradient(do_dtype, level):
    """An inf in one level's upstream gradient turns the rows that level touches into nan and leaves the other
    levels exact (level 1: dense, five bins; level 2: hashed)."""
    hk = _hk()
    torch.manual_seed(6)
    N, T, L, lo, hi = 40000, 2**16, 4, 16, 128
    x = torch.rand(N, 3)
    E = O.level_row_offsets(L, T, 3, lo, hi)[-1]
    offs = O.level_row_offsets(L, T, 3, lo, hi)
    do = torch.randn(N, L * 2).to(do_dtype)
    clean = O.encode_backward(x, do, E, 2, None, T, L, lo, hi)
    do[123, 2 * level] = float("inf")  # feature 0 of the level
    got = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, 2, None, T, lo, hi, L).cpu()
    lvl = slice(offs[level], offs[level + 1])
    assert not torch.isfinite(got[lvl]).all()
    keep = torch.ones(E, dtype=torch.bool)
    keep[lvl] = False
    torch.testing.assert_close(got[keep], clean[keep], rtol=1e-3, atol=1e-4)


@pytest.mark.parametrize("feat", [1, 3])
def test_backward_binned_nonfinite_gradient_odd_feature_count(feat):
    """With an odd number of features the last feature is a pair with an empty partner: an inf in a level's gradient
    must mark that level's rows only -- not feature 0 of the following row, the first row of the next level, or the
    memory behind the table (a guard region after the gradient table stays untouched)."""
    hk = _hk()
    torch.manual_seed(7)
    N, T, L, lo, hi = 40000, 2**16, 4, 16, 256
    x = torch.rand(N, 3)
    offs = O.level_row_offsets(L, T, 3, lo, hi)
    E = offs[-1]
    do = torch.randn(N, L * feat).half()
    clean = O.encode_backward(x, do, E, feat, None, T, L, lo, hi)
    do[123, 3 * feat + feat - 1] = float("inf")  # the last level, its last feature
    guard = 4096
    buf = torch.zeros(E * feat + guard, dtype=torch.float32, device=DEV)
    out = buf[: E * feat].view(E, feat)
    got = hk.hash_encoding_table_grad(x.to(DEV), do.to(DEV), E, feat, None, T, lo, hi, L, out=out).cpu()
    assert torch.count_nonzero(buf[E * feat:]).item() == 0, "wrote behind the gradient table"
    last = slice(offs[3], offs[4])
    assert not torch.isfinite(got[last, feat - 1]).all()
    # the other features of the poisoned level and every other level are exact
    if feat > 1:
        torch.testing.assert_close(got[last, : feat - 1], clean[last, : feat - 1], rtol=1e-3, atol=1e-4)
    torch.testing.assert_close(got[: offs[3]], clean[: offs[3]], rtol=1e-3, atol=1e-4)
    # ... and with the inf in the first level the first row of the next level stays clean
    do2 = torch.randn(N, L * feat).half()
    clean2 = O.encode_backward(x, do2, E, feat, None, T, L, lo, hi)
    do2[77, feat - 1] = float("inf")
    got2 = hk.hash_encoding_table_grad(x.to(DEV), do2.to(DEV), E, feat, None, T, lo, hi, L).cpu()
    torch.testing.assert_close(got2[offs[1]:], clean2[offs[1]:], rtol=1e-3, atol=1e-4)


def test_autograd_round_trip_fp16_table():
    """hash_encoding(...).backward(do) through the autograd Function: grad lands in the table's dtype."""
    hk = _hk()
    g = GOLDEN["default"]
    torch.manual_seed(0)
    x = torch.rand(2, 500, 3)
    table = torch.randn(g["total_rows"], 2).half()
    e = table.to(DEV).requires_grad_(True)
    o = hk.hash_encoding(x.to(DEV), e, max_entries_per_level=g["T"])
    assert o.shape == (2, 500, 32) and o.dtype == torch.float16
    do = torch.randn(2, 500, 32).half()
    o.backward(do.to(DEV))
    assert e.grad is not None and e.grad.dtype == torch.float16
    want = O.encode_backward(x.view(-1, 3), do.view(-1, 32), g["total_rows"], 2, None, g["T"], 16, 16, 512)
    torch.testing.assert_close(e.grad.cpu().float(), want, rtol=2e-3, atol=2e-3)


def test_features_are_appended_and_ignored_in_backward():
    hk = _hk()
    g = GOLDEN["default"]
    torch.manual_seed(0)
    x = torch.rand(333, 3)
    feats = torch.randn(333, 5).half()
    table = torch.randn(g["total_rows"], 2).half()
    e = table.to(DEV).requires_grad_(True)
    o = hk.hash_encoding(x.to(DEV), e, feats.to(DEV), max_entries_per_level=g["T"])
    assert o.shape == (333, 37)
    want = O.encode_forward(x, table.float(), None, g["T"], 16, 16, 512)
    torch.testing.assert_close(o[:, :32].cpu().float(), want, rtol=2.0**-10, atol=1e-3)
    assert torch.equal(o[:, 32:].cpu(), feats)
    do = torch.randn(333, 37).half()
    o.backward(do.to(DEV))
    wantg = O.encode_backward(x, do[:, :32], g["total_rows"], 2, None, g["T"], 16, 16, 512)
    torch.testing.assert_close(e.grad.cpu().float(), wantg, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("dtype,n_feat", [(torch.float16, 3), (torch.float32, 3), (torch.float16, 4), (torch.bfloat16, 1)])
def test_appended_features_off_16_byte_rows_at_large_batches(dtype, n_feat):
    """Three appended features (view directions) leave output and gradient rows off 16-byte boundaries.  From 4096
    points the encoding is then written to a packed buffer and concatenated, and the backward packs the encoding's
    gradient columns first, so both directions keep the fast kernels: same values as the call without features, bit for
    bit in the forward, and the table gradient against the oracle."""
    hk = _hk()
    g = GOLDEN["bench"]
    T, L, lo, hi = g["T"], 16, 16, 7006
    N = 20000 + 3
    torch.manual_seed(4)
    x = torch.rand(2, N, 3, device=DEV)                     # leading batch dimensions as in the reference's shapes
    feats = torch.randn(2, N, n_feat, device=DEV).to(dtype)
    table = _table(T, L, 3, lo, hi, dtype=dtype, amp=1.0).to(DEV)
    e = table.clone().requires_grad_(True)
    o = hk.hash_encoding(x, e, feats, None, T, lo, hi, L)
    plain = hk.hash_encoding(x, table, None, None, T, lo, hi, L)
    assert o.shape == (2, N, 32 + n_feat) and o.dtype == dtype
    assert torch.equal(o[..., :32], plain) and torch.equal(o[..., 32:], feats)
    do = torch.randn(2, N, 32 + n_feat, device=DEV).to(dtype)
    o.backward(do)
    want = O.encode_backward(x.reshape(-1, 3).cpu(), do.reshape(-1, 32 + n_feat)[:, :32].cpu(), table.shape[0], 2, None, T, L, lo, hi)
    tol = 2e-3 if dtype != torch.float32 else 1e-4
    torch.testing.assert_close(e.grad.cpu().float(), want, rtol=max(tol, 2.0**-8 if dtype == torch.bfloat16 else 0), atol=tol * float(want.abs().max()))


def test_module_autocast():
    # reference test_hash_encoding.py:507-530
    from triton_helpers_amd.layers.hash_encoding import HashEncoding

    layer = HashEncoding(2**14, 16, 3, 2, 16, 512).to(DEV)
    x = torch.rand(16, 40, 3, device=DEV)
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        o = layer(x)
    assert o.dtype == torch.float16 and o.shape == (16, 40, 32)
    layer2 = HashEncoding(2**8, 4, 3, 2, 16, 512).to(DEV)
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        o2 = layer2(x)
    o2.sum().backward()
    assert layer2.embeddings.grad is not None
    assert set(layer.state_dict().keys()) == {"embeddings", "pi"}


def test_argument_errors():
    hk = _hk()
    g = GOLDEN["default"]
    table = torch.zeros(g["total_rows"], 2, device=DEV)
    x = torch.rand(10, 3, device=DEV)
    with pytest.raises(AssertionError):
        hk.hash_encoding(x.cpu(), table, max_entries_per_level=g["T"])  # mixed devices
    with pytest.raises(AssertionError):
        hk.hash_encoding(x, table, max_entries_per_level=g["T"], levels=12)  # not a power of two
    with pytest.raises(ValueError):
        hk.hash_encoding(torch.rand(10, 4, device=DEV), table, max_entries_per_level=g["T"])  # D>3 without pi
    with pytest.raises(AssertionError):
        hk.hash_encoding(x.long(), table, max_entries_per_level=g["T"])
    with pytest.raises(AssertionError):
        hk.hash_encoding(x, table[:100], max_entries_per_level=g["T"])  # table too small for the geometry


def test_empty_and_edge_coordinates():
    hk = _hk()
    g = GOLDEN["default"]
    table = _table(g["T"], 16, 3, 16, 512).to(DEV)
    o = hk.hash_encoding(torch.empty(0, 3, device=DEV), table, max_entries_per_level=g["T"])
    assert o.shape == (0, 32)
    # x == scale is legal (cell N_l, corners up to N_l + 1); must match the oracle and stay in range
    x = torch.tensor([[1.0, 1.0, 1.0], [0.0, 0.0, 0.0], [1.0, 0.0, 0.5]])
    got = hk.hash_encoding(x.to(DEV), table, max_entries_per_level=g["T"])
    want = O.encode_forward(x, table.cpu(), None, g["T"], 16, 16, 512)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-9)


@pytest.mark.parametrize("N", [3, 2**18 + 3])
def test_upper_edge_in_two_dimensions(N):
    """x == scale in both of two dimensions: on a dense level the last corner (weight 0) is row (N_l + 1)^2, one past
    the level, where the reference's CPU path raises an IndexError.  The kernels keep that corner inside the level:
    the encoding is the table row of corner 0, whose weight is 1, and the whole upstream gradient lands there.
    Both the small-batch kernels and the sweep / binned kernels are covered."""
    hk = _hk()
    T, L, lo, hi = 2**19, 16, 16, 7006
    offs = O.level_row_offsets(L, T, 2, lo, hi)
    table = _table(T, L, 2, lo, hi, dtype=torch.float16, amp=1.0).to(DEV).requires_grad_(True)
    x = torch.rand(N, 2)
    x[0] = 1.0
    out = hk.hash_encoding(x.to(DEV), table, None, None, T, lo, hi, L)
    rows = hk.hash_encoding_indices(x[:1].to(DEV), None, T, lo, hi, L).cpu()[0]  # (L, 4)
    want_rows = O.encode_indices(x[1:3], None, T, L, lo, hi)
    assert torch.equal(hk.hash_encoding_indices(x[1:3].to(DEV), None, T, lo, hi, L).cpu(), want_rows)
    for l in range(L):
        n_rows = offs[l + 1] - offs[l]
        assert int(rows[l].max()) < n_rows and int(rows[l].min()) >= 0
        assert torch.equal(out[0, 2 * l : 2 * l + 2], table[offs[l] + int(rows[l, 0])]), l
    want = O.encode_forward(x[1:3], table.detach().float().cpu(), None, T, L, lo, hi)
    torch.testing.assert_close(out[1:3].detach().cpu().float(), want, rtol=2.0**-10, atol=1e-6)
    do = torch.zeros(N, 2 * L, dtype=torch.float16)
    do[0] = 1.0
    out.backward(do.to(DEV))
    grad = table.grad.float().cpu()
    for l in range(L):
        level = grad[offs[l] : offs[l + 1]]
        assert abs(float(level[int(rows[l, 0])].min()) - 1.0) < 1e-3  # (the binned backward carries 19-bit weights)
        assert abs(float(level.sum()) - 2.0) < 2e-3, l


def test_upper_edge_in_one_dimension():
    """The same edge with one coordinate: x == scale puts the second corner (weight 0) at row N_l + 1, one past a
    dense level; it is kept at the level's last row, the encoding is the row of corner 0 and the gradient lands there."""
    hk = _hk()
    T, L, lo, hi = 64, 4, 8, 512
    offs = O.level_row_offsets(L, T, 1, lo, hi)
    table = _table(T, L, 1, lo, hi, dtype=torch.float32, amp=1.0).to(DEV).requires_grad_(True)
    x = torch.tensor([[1.0], [0.25], [0.0]])
    out = hk.hash_encoding(x.to(DEV), table, None, None, T, lo, hi, L)
    rows = hk.hash_encoding_indices(x.to(DEV), None, T, lo, hi, L).cpu()
    assert torch.equal(rows[1:], O.encode_indices(x[1:], None, T, L, lo, hi))
    want = O.encode_forward(x[1:], table.detach().cpu(), None, T, L, lo, hi)
    torch.testing.assert_close(out[1:].detach().cpu(), want, rtol=1e-5, atol=1e-9)
    do = torch.zeros(3, 2 * L)
    do[0] = 1.0
    out.backward(do.to(DEV))
    grad = table.grad.cpu()
    for l in range(L):
        n_rows = offs[l + 1] - offs[l]
        assert 0 <= int(rows[0, l].min()) and int(rows[0, l].max()) < n_rows
        assert torch.equal(out[0, 2 * l : 2 * l + 2], table[offs[l] + int(rows[0, l, 0])])
        assert float(grad[offs[l] : offs[l + 1]].sum()) == 2.0


def test_full_size_properties_config1():
    """BASELINE configs[1] at full size (N=2^20): size-independent checks.

    * sum over level l / feature f of the table gradient == sum_n do[n, l*F+f] (weights sum to one);
    * linearity of the backward in do;
    * a constant table encodes to that constant;
    * a 4096-point sample of the full-size forward equals the oracle.
    """
    hk = _hk()
    g = GOLDEN["bench"]
    T, E = g["T"], g["total_rows"]
    torch.manual_seed(0)
    x = torch.rand(2**20, 3)
    table = ((torch.rand(E, 2) * 2 - 1) * 1e-4).half()
    do = torch.randn(2**20, 32).half()
    xd, td, dod = x.to(DEV), table.to(DEV), do.to(DEV)
    out = hk.hash_encoding(xd, td, None, None, T, 16, 7006, 16)
    idx = torch.randperm(2**20)[:4096]
    want = O.encode_forward(x[idx], table.float(), None, T, 16, 16, 7006)
    # table values ~1e-4 sit in fp16's subnormal range: one fp16 step there is 2^-24 = 6e-8
    torch.testing.assert_close(out[idx.to(DEV)].cpu().float(), want, rtol=2.0**-10, atol=2.0**-24)

    grad = hk.hash_encoding_table_grad(xd, dod, E, 2, None, T, 16, 7006, 16)
    offs = O.level_row_offsets(16, T, 3, 16, 7006)
    colsum = dod.float().sum(0).cpu().double()
    for l in range(16):
        s = grad[offs[l] : offs[l + 1]].double().sum(0).cpu()
        torch.testing.assert_close(s, colsum[2 * l : 2 * l + 2], rtol=1e-3, atol=0.5)
    grad2 = hk.hash_encoding_table_grad(xd, (dod * 2), E, 2, None, T, 16, 7006, 16)
    torch.testing.assert_close(grad2, grad * 2, rtol=1e-3, atol=1e-3)

    const = torch.full((E, 2), 0.25, dtype=torch.float16, device=DEV)
    oc = hk.hash_encoding(xd, const, None, None, T, 16, 7006, 16)
    torch.testing.assert_close(oc.float(), torch.full_like(oc, 0.25, dtype=torch.float32), rtol=1e-3, atol=0)


@pytest.mark.parametrize("records", [False, True])
def test_backward_in_pieces_beyond_two_million_points(records, monkeypatch):
    """Batches above 2^21 points run in pieces, through the walk without records (this geometry's default) and through
    the sort-and-accumulate pipeline alike: the workspace stops growing and the gradient equals the sum of the halves'
    gradients computed separately."""
    from triton_helpers_amd import _lib

    hk = _hk()
    flags = _lib.NF_HASH_BWD_RECORDS if records else 0
    monkeypatch.setattr(hk, "_FLAGS", flags)
    T, L, lo, hi = 2**14, 16, 16, 512
    E = O.level_row_offsets(L, T, 3, lo, hi)[-1]
    from triton_helpers_amd.layers.hash_encoding.helpers import level_geometry

    geom = level_geometry(T, L, 3, 2, lo, hi)
    lib = _lib.load()
    assert lib.nf_hash_encode_bwd_workspace_bytes(2**22, geom, _lib.NF_F16, flags) == lib.nf_hash_encode_bwd_workspace_bytes(2**21, geom, _lib.NF_F16, flags)
    N = 2**21 + 12345
    g = torch.Generator().manual_seed(3)
    x = torch.rand(N, 3, generator=g).to(DEV)
    do = torch.randn(N, 32, generator=g).half().to(DEV)
    whole = hk.hash_encoding_table_grad(x, do, E, 2, None, T, lo, hi, L)
    cut = 2**20 + 77
    parts = hk.hash_encoding_table_grad(x[:cut], do[:cut], E, 2, None, T, lo, hi, L)
    hk.hash_encoding_table_grad(x[cut:], do[cut:], E, 2, None, T, lo, hi, L, out=parts)
    torch.testing.assert_close(whole, parts, rtol=1e-4, atol=1e-3 * float(parts.abs().mean()))
