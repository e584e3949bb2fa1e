"""CPU-only checks: the C-ABI library loads and exports every symbol the header declares, the host-side
geometry equals the oracle's, and the operators refuse to run without a GPU (no fallback path exists)."""
import ctypes
import json
import os
import re

import pytest
import torch

from oracle import hash_encoding as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = json.load(open(os.path.join(ROOT, "tests", "golden", "hash_geometry.json")))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "nf_cdna4.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nf_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from triton_helpers_amd import _lib

    if not _lib.LIB_PATH.exists():
        pytest.skip("libnf_cdna4.so not built (run python -m triton_helpers_amd.build)")
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    names = _declared_functions()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/nf_cdna4.h but not exported"
    assert set(names) == set(_lib.EXPORTS), "ctypes binding and header disagree"
    lib.nf_abi_version.restype = ctypes.c_int
    assert lib.nf_abi_version() == _lib.NF_ABI_VERSION
    header = open(os.path.join(ROOT, "include", "nf_cdna4.h")).read()
    assert f"#define NF_ABI_VERSION {_lib.NF_ABI_VERSION}" in header


def test_argument_validation_without_gpu():
    """Entry points validate before touching the device: bad arguments come back as negative codes."""
    from triton_helpers_amd import _lib

    if not _lib.LIB_PATH.exists():
        pytest.skip("libnf_cdna4.so not built")
    lib = _lib.load()
    geom = _lib.HashGeom()
    geom.dims = 7
    rc = lib.nf_hash_encode_fwd(None, 0, 3, 1, None, 0, None, 32, 10, geom, None, 1.0, 0, None)
    assert rc == -1 and b"dims" in lib.nf_last_error()
    rc = lib.nf_mlp_fwd(None, 32, None, 16, None, None, None, None, None, None, 8, 32, 24, 16, 2, 1, _lib.NF_BF16, _lib.NF_BF16, None, 0, None)
    assert rc == -1 and b"d_hidden" in lib.nf_last_error()
    rc = lib.nf_mlp_fwd(None, 32, None, 16, None, None, None, None, None, None, 8, 32, 64, 16, 2, 1, _lib.NF_F32, _lib.NF_BF16, None, 0, None)
    assert rc == -2
    rc = lib.nf_revmlp_fwd(None, 128, None, 128, None, None, None, None, 8, 65, 4, 4, _lib.NF_BF16, None)
    assert rc == -1
    with pytest.raises(RuntimeError):
        _lib.check(rc, "nf_revmlp_fwd")
    # zero rows is a no-op that needs no device
    assert lib.nf_mlp_fwd(None, 32, None, 16, None, None, None, None, None, None, 0, 32, 64, 16, 2, 1, _lib.NF_BF16, _lib.NF_BF16, None, 0, None) == 0


def test_mlp_workspace_sizes_without_gpu():
    """One launch needs no workspace; a chain of n launches keeps two hand-over buffers in the forward and
    n - 1 of them plus two gradient buffers in the backward, each rows * d_hidden 16-bit values (256-byte rounded)."""
    from triton_helpers_amd import _lib

    if not _lib.LIB_PATH.exists():
        pytest.skip("libnf_cdna4.so not built")
    lib = _lib.load()
    relu, silu = _lib.NF_ACT["relu"], _lib.NF_ACT["silu"]
    rows = 1000
    buf = (rows * 64 * 2 + 255) // 256 * 256
    for depth in (1, 2, 4):
        assert lib.nf_mlp_workspace_bytes(rows, 64, depth, relu, 0, _lib.NF_BF16) == 0
        assert lib.nf_mlp_workspace_bytes(rows, 64, depth, relu, 1, _lib.NF_BF16) == 0
    assert lib.nf_mlp_workspace_bytes(rows, 64, 2, silu, 1, _lib.NF_BF16) == 0
    assert lib.nf_mlp_workspace_bytes(rows, 64, 8, relu, 0, _lib.NF_BF16) == 0           # 9 layers of weights fit LDS
    assert lib.nf_mlp_workspace_bytes(rows, 64, 8, relu, 1, _lib.NF_BF16) == (1 + 2) * buf  # 9 linear layers = 5 + 4
    assert lib.nf_mlp_workspace_bytes(rows, 64, 5, silu, 1, _lib.NF_BF16) == (1 + 2) * buf  # 6 linear layers = 3 + 3
    assert lib.nf_mlp_workspace_bytes(rows, 64, 32, relu, 0, _lib.NF_BF16) == 2 * buf
    assert lib.nf_mlp_workspace_bytes(rows, 32, 2, relu, 1, _lib.NF_BF16) == 0
    assert lib.nf_mlp_workspace_bytes(rows, 32, 8, relu, 1, _lib.NF_BF16) == (2 + 2) * ((rows * 32 * 2 + 255) // 256 * 256)  # 9 linear layers = 3 + 3 + 3
    assert lib.nf_mlp_workspace_bytes(0, 64, 32, relu, 1, _lib.NF_BF16) == 0
    # float32: nothing in the forward, every hidden layer's float32 pre-activation in the backward (+ partial dW / db)
    part = 512 * (64 * 64 + 64) * 4
    assert lib.nf_mlp_workspace_bytes(rows, 64, 32, relu, 0, _lib.NF_F32) == 0
    assert lib.nf_mlp_workspace_bytes(rows, 64, 2, relu, 1, _lib.NF_F32) == 2 * rows * 64 * 4 + part
    assert lib.nf_mlp_workspace_bytes(rows, 16, 3, silu, 1, _lib.NF_F32) == 3 * rows * 16 * 4 + part
    rc = lib.nf_mlp_bwd(1, 32, 1, 16, None, 32, 1, None, 1, None, 1, None, 1, None, 1, None, 1, None,
                        rows, 32, 64, 16, 2, relu, _lib.NF_F32, _lib.NF_F32, None, 0, None)
    assert rc == -1 and b"workspace" in lib.nf_last_error()
    # float32 parameters with 16-bit rows (or the reverse) are refused
    rc = lib.nf_mlp_fwd(1, 32, 1, 16, 1, None, 1, None, 1, None, rows, 32, 64, 16, 2, relu, _lib.NF_F32, _lib.NF_F16, None, 0, None)
    assert rc == -2 and b"x_dtype" in lib.nf_last_error()
    # a deep call without the workspace is refused before anything is launched
    rc = lib.nf_mlp_bwd(1, 32, 1, 16, None, 32, 1, None, 1, None, 1, None, 1, None, 1, None, 1, None,
                        rows, 32, 64, 16, 8, relu, _lib.NF_BF16, _lib.NF_BF16, None, 0, None)
    assert rc == -1 and b"workspace" in lib.nf_last_error()


@pytest.mark.parametrize("name", ["bench", "default"])
def test_host_geometry_matches_oracle_and_golden(name):
    from triton_helpers_amd.layers.hash_encoding import helpers as H

    g = GOLDEN[name]
    T, L, D, lo, hi = g["T"], g["levels"], g["dims"], g["min_res"], g["max_res"]
    assert H.compute_resolutions(L, lo, hi) == g["resolutions"] == O.level_resolutions(L, lo, hi)
    assert H.compute_embedding_counts(L, T, D, lo, hi) == g["rows"]
    assert H.get_first_hash_level(lo, hi, L, T, D) == g["first_hash_level"]
    assert H.compute_b(lo, hi, L) == O.growth_factor(lo, hi, L)
    offs = O.level_row_offsets(L, T, D, lo, hi)
    for l in range(L):
        assert H.compute_level_embedding_offset(l, L, T, D, lo, hi) == offs[l]
    e = torch.zeros(g["total_rows"], 2)
    assert H.seek_to_level_embeddings(e, 5, L, T, D, lo, hi).shape[0] == g["rows"][5]
    geom = H.level_geometry(T, L, D, 2, lo, hi)
    assert list(geom.res)[:L] == g["resolutions"] and list(geom.rows)[:L] == g["rows"]
    assert list(geom.row_offset)[:L] == offs[:L] and geom.first_hash_level == g["first_hash_level"]
    assert H.get_first_hash_level(2, 4, 2, 10**9, 2) == 3  # "no hashing" is reported as L + 1


def test_cpu_helpers_with_reference_names_live_with_the_oracle():
    """The reference's private ``_cpu_*`` test helpers exist under ``oracle/`` (its argument order, literal tables
    included); the shipped package carries no CPU path."""
    from oracle import reference_names as R
    from tests.test_oracle_hash import DENSE_ROWS, HASHED_ROWS, QUADRANT_X
    from triton_helpers_amd.layers.hash_encoding import kernel as K

    assert not any(n.startswith("_cpu_") for n in vars(K)), "CPU restatements belong to the oracle, not to the package"

    pi = torch.tensor([K.PI_1, K.PI_2, K.PI_3])
    x = torch.tensor(QUADRANT_X, dtype=torch.float32)
    assert R._cpu_embedding_lookup(x, pi[:2], 2, 9, 2).tolist() == DENSE_ROWS
    assert R._cpu_embedding_lookup(x, pi[:2], 2, 7, 2).tolist() == HASHED_ROWS
    assert R._cpu_create_corner_offsets(2, dtype=torch.int64).tolist() == [[0, 0], [1, 0], [0, 1], [1, 1]]
    g = GOLDEN["default"]
    torch.manual_seed(0)
    xs = torch.rand(50, 3)
    table = torch.randn(g["total_rows"], 2)
    out = R._cpu_hash_encoding(xs, table, pi, torch.zeros(50, 32), 3, 2, g["T"], 16, 16, 512)
    torch.testing.assert_close(out, O.encode_forward(xs, table, None, g["T"], 16, 16, 512))


def test_operators_refuse_cpu_tensors():
    from triton_helpers_amd.layers.fully_fused_mlp import fully_fused_mlp
    from triton_helpers_amd.layers.hash_encoding import hash_encoding
    from triton_helpers_amd.layers.reversible_mlp import reversible_mlp

    g = GOLDEN["default"]
    with pytest.raises(AssertionError):
        hash_encoding(torch.rand(4, 3), torch.zeros(g["total_rows"], 2), max_entries_per_level=g["T"])
    h = torch.zeros
    with pytest.raises(AssertionError):
        fully_fused_mlp(h(1, 4, 8).half(), h(16, 8).half(), None, h(4, 16).half(), None)
    with pytest.raises(AssertionError):
        reversible_mlp(h(4, 128).half(), h(128, 64).half(), None, h(128, 64).half(), None)


def test_drop_in_alias_package():
    import triton_helpers.layers.fully_fused_mlp as a
    import triton_helpers.layers.hash_encoding as b
    from triton_helpers.layers.fully_fused_mlp.kernel import FULLY_FUSED_MAX_DIM, _fully_fused_mlp  # noqa: F401
    from triton_helpers.layers.hash_encoding.helpers import compute_embedding_counts  # noqa: F401
    from triton_helpers.layers.hash_encoding.kernel import PI_2, HashEncoding, compute_resolutions, get_first_hash_level  # noqa: F401

    assert PI_2 == 2_654_435_761
    assert {"fully_fused_mlp", "FullyFusedMLP", "feedforward"} <= set(a.__all__)
    assert {"hash_encoding", "HashEncoding"} <= set(b.__all__)


def test_bench_rejects_more_than_one_gpu():
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_hash_module_seeded_table_is_the_reference_recipe():
    """Same seed, same table: one ``randn`` draw per level, concatenated (reference hash_encoding/module.py:20-21);
    a single draw over the stacked table gives other values."""
    from triton_helpers_amd.layers.hash_encoding import HashEncoding
    from triton_helpers_amd.layers.hash_encoding.helpers import compute_embedding_counts

    for kw in (dict(), dict(max_entries_per_level=2**10, num_levels=4, d_in=2, d_embed=4, min_res=2, max_res=64)):
        torch.manual_seed(123)
        layer = HashEncoding(**kw)
        T, L, D, F = layer.max_entries_per_level, layer.num_levels, kw.get("d_in", 3), kw.get("d_embed", 2)
        counts = compute_embedding_counts(L, T, D, layer.min_res, layer.max_res)
        torch.manual_seed(123)
        want = torch.cat([torch.randn(int(t), F) for t in counts], dim=0)
        assert torch.equal(layer.embeddings.detach(), want)
        torch.manual_seed(123)
        assert not torch.equal(torch.randn(sum(counts), F), want)
        assert set(layer.state_dict().keys()) == {"embeddings", "pi"}
        assert layer.pi.tolist() == [1, 2654435761, 805459861]


def test_row_views_of_broadcast_and_strided_tensors():
    """An expanded upstream gradient (``out.sum(0).backward(g)`` hands the backward ``g.expand(N, W)``, row stride 0)
    or a strided inner dimension must reach the C ABI as rows that do not overlap."""
    from triton_helpers_amd.layers.fully_fused_mlp.kernel import _rows2d as mlp_rows
    from triton_helpers_amd.layers.hash_encoding.kernel import _as_rows
    from triton_helpers_amd.layers.reversible_mlp.kernel import _rows2d as rev_rows

    for fn in (_as_rows, mlp_rows, rev_rows):
        g = torch.arange(32.0)
        e = g.expand(5, 32)
        r = fn(e, 32)
        assert r.shape == (5, 32) and r.stride() == (32, 1) and torch.equal(r, e)
        e3 = g.expand(2, 3, 32)
        r = fn(e3, 32)
        assert r.shape == (6, 32) and r.stride(1) == 1 and r.stride(0) >= 32 and torch.equal(r, e3.reshape(6, 32))
        t = torch.arange(5 * 64.0).view(5, 64)
        v = fn(t[:, :32], 32)  # wider row stride: stays a view
        assert v.data_ptr() == t.data_ptr() and v.stride() == (64, 1)
        s = fn(t[:, ::2], 32)  # strided inner dimension: copied
        assert s.stride() == (32, 1) and torch.equal(s, t[:, ::2])
        one = fn(g.expand(1, 32), 32)  # a single row has nothing to overlap with
        assert one.shape == (1, 32)
