"""Randomized differential runs of the three layers against the CPU oracle (through the C ABI).

Every case draws a configuration from a seeded generator (shapes off the tiles, ragged row counts, all storage
dtypes, table sizes that are not powers of two, clustered points and points on grid nodes and on the upper
edge) and checks it at the tolerances of the fixed-case tests.  A failure names the drawn configuration.
"""
import random

import pytest
import torch

from oracle import hash_encoding as O
from oracle import mlp as M
from oracle import reversible as R

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rel(got, want):
    got, want = got.detach().cpu().float(), want.float()
    d = (got - want).abs()
    peak = max(float(want.abs().max()) if want.numel() else 0.0, 1e-30)
    return d, peak


@pytest.mark.parametrize("seed", range(6))
def test_hash_encoding_random_configurations(seed):
    """Forward: float32 tables to 1e-5 of the largest output, 16-bit tables to the storage rounding.  Backward: rtol
    1e-3 plus 2e-4 of the largest gradient entry (atomic order, and the 16-bit cell fractions of dense 3-D levels)."""
    from triton_helpers_amd.layers.hash_encoding import kernel as hk

    for it in range(25):
        rng = random.Random(seed * 100003 + it)
        D = rng.choice([1, 2, 2, 3, 3, 3, 3])
        F = rng.choice([1, 2, 2, 2, 3, 4, 8])
        L = rng.choice([2, 4, 8, 16])  # one level has no growth factor (helpers.py:12-23 divides by levels - 1)
        lo = rng.choice([2, 3, 4, 8, 16, 24])
        hi = max(lo, rng.choice([4, 16, 40, 64, 72, 89, 90, 128, 300, 512, 2048, 7006]))
        T = rng.choice([2**10, 2**12, 2**14, 2**16, 2**19, 2**20, 5000, 12345, 3 * 2**15])
        N = rng.choice([1, 63, 1000, 4099, 32768, 33001, 70001])
        scale = rng.choice([1.0, 1.0, 2.0, 0.5])
        do_dtype = rng.choice([torch.float16, torch.bfloat16, torch.float32])
        tab_dtype = rng.choice([torch.float16, torch.bfloat16, torch.float32])
        dist = rng.choice(["uniform", "uniform", "cluster", "nodes", "edge"])
        tag = f"seed={seed} it={it} D={D} F={F} L={L} lo={lo} hi={hi} T={T} N={N} scale={scale} do={do_dtype} table={tab_dtype} {dist}"
        torch.manual_seed(seed * 7919 + it)
        x = torch.rand(N, D)
        if dist == "cluster":
            x[: N // 2] = torch.rand(1, D) * 0.9 + 1e-3 * torch.rand(N // 2, D)
        elif dist == "nodes":  # weights exactly 0 and 1 on the finest level (the corner (1, .., 1) itself is outside the oracle's tables)
            x[: N // 2] = torch.randint(0, hi, (N // 2, D)).float() / hi
        elif dist == "edge":
            x[: N // 3, 0] = 1.0
            x[N // 3 : N // 2] = 0.0
            if D > 1:
                x[: N // 3, 1:] = x[: N // 3, 1:].clamp(max=0.999)
        if D == 1:
            x = x.clamp(max=0.999999)  # x == 1 puts the upper corner one past a dense 1-D level
        E = O.level_row_offsets(L, T, D, lo, hi)[-1]
        g = torch.Generator().manual_seed(it)
        table = (torch.rand(E, F, generator=g) * 2 - 1).to(tab_dtype)
        do = torch.randn(N, L * F).to(do_dtype)
        want = O.encode_forward(x, table.float(), None, T, L, lo, hi)
        got = hk.hash_encoding(x.to(DEV) * scale, table.to(DEV), None, None, T, lo, hi, L, scale=scale)
        assert got.dtype == tab_dtype, tag
        d, peak = _rel(got, want)
        tol = {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 1e-2}[tab_dtype]
        assert float(d.max()) <= tol * max(1.0, peak), f"forward: {tag}"
        want = O.encode_backward(x, do, E, F, None, T, L, lo, hi)
        got = hk.hash_encoding_table_grad(x.to(DEV) * scale, do.to(DEV), E, F, None, T, lo, hi, L, scale).cpu()
        d, peak = _rel(got, want)
        assert bool(torch.isfinite(got).all()) and not bool((d > 1e-3 * want.abs() + 2e-4 * peak).any()), f"backward: {tag}"


@pytest.mark.parametrize("seed", range(3))
def test_hash_encoding_random_configurations_in_one_and_four_to_six_dimensions(seed):
    """The same differential run where the caller brings the primes: one dimension and four to six (the walk without
    records, the record passes per corner of the extra coordinates, the per-(point, level) kernels below their
    minimum batch), forward and backward."""
    from triton_helpers_amd.layers.hash_encoding import kernel as hk

    primes = torch.tensor([1, 2654435761, 805459861, 3674653429, 2097192037, 1434869437], dtype=torch.int64)
    for it in range(12):
        rng = random.Random(seed * 100019 + it)
        D = rng.choice([1, 4, 4, 4, 5, 6])
        F = rng.choice([1, 2, 2, 3, 4])
        L = rng.choice([2, 4, 8])
        lo = rng.choice([2, 3, 4, 8])
        hi = max(lo, rng.choice([4, 6, 9, 16, 24, 40] if D > 1 else [64, 512, 5000, 40000]))
        T = rng.choice([2**10, 2**13, 2**14, 2**15, 2**17, 2**19, 5000, 50000, 3 * 2**15])
        N = rng.choice([63, 4099, 8192, 9001, 20000])
        if D >= 5:
            N = min(N, 9001)
        scale = rng.choice([1.0, 2.0])
        do_dtype = rng.choice([torch.float16, torch.bfloat16, torch.float32])
        tab_dtype = rng.choice([torch.float16, torch.float32])
        tag = f"seed={seed} it={it} D={D} F={F} L={L} lo={lo} hi={hi} T={T} N={N} scale={scale} do={do_dtype} table={tab_dtype}"
        E = O.level_row_offsets(L, T, D, lo, hi)[-1]
        if E > 20_000_000:
            continue
        torch.manual_seed(seed * 7927 + it)
        x = torch.rand(N, D).clamp(max=0.999999)  # (1, .., 1) is outside the oracle's dense tables
        x[: N // 4] = (torch.randint(0, hi, (N // 4, D)).float() / hi).clamp(max=0.999999)
        x[N // 4 : N // 2] = (torch.rand(1, D) * 0.9 + 1e-3 * torch.rand(N // 2 - N // 4, D)).clamp(max=0.999999)
        pi = primes[:D]
        g = torch.Generator().manual_seed(it)
        table = (torch.rand(E, F, generator=g) * 2 - 1).to(tab_dtype)
        do = torch.randn(N, L * F).to(do_dtype)
        want = O.encode_forward(x, table.float(), pi, T, L, lo, hi)
        got = hk.hash_encoding(x.to(DEV) * scale, table.to(DEV), None, pi.to(DEV), T, lo, hi, L, scale=scale)
        d, peak = _rel(got, want)
        tol = {torch.float32: 1e-5, torch.float16: 2e-3}[tab_dtype]
        assert float(d.max()) <= tol * max(1.0, peak), f"forward: {tag}"
        want = O.encode_backward(x, do, E, F, pi, T, L, lo, hi)
        got = hk.hash_encoding_table_grad(x.to(DEV) * scale, do.to(DEV), E, F, pi.to(DEV), T, lo, hi, L, scale).cpu()
        d, peak = _rel(got, want)
        assert bool(torch.isfinite(got).all()) and not bool((d > 1e-3 * want.abs() + 2e-4 * peak).any()), f"backward: {tag}"


@pytest.mark.parametrize("seed", range(4))
def test_fused_mlp_random_configurations(seed):
    """Errors relative to each tensor's largest magnitude: 2e-2 for 16-bit storage (x depth / 4 beyond four layers),
    2e-4 for float32 with smooth activations.  ReLU nets are compared at the 16-bit tolerance in float32 too and
    with 2e-3 of the dx elements left out: a pre-activation within rounding of zero switches its gate in one of the
    two summation orders and moves that row's gradients by whole weights."""
    from triton_helpers_amd.layers.fully_fused_mlp import kernel as mk

    for it in range(40):
        rng = random.Random(seed * 100003 + it)
        dtype = rng.choice([torch.bfloat16, torch.float16, torch.float32])
        d_hidden = rng.choice([16, 32, 64, 64, 64])
        d_in = rng.choice([1, 2, 3, 8, 16, 17, 31, 32, 33, 48, 63, 64])
        d_out = rng.choice([1, 3, 4, 5, 16, 17, 32, 40, 64])
        depth = rng.choice([1, 2, 2, 2, 3, 4, 5, 7, 9])
        act = rng.choice(["relu", "relu", "silu", "none", "relu2"])
        if act == "relu2" and depth > 3:
            act = "relu"
        bias = rng.choice([True, False])
        rows = rng.choice([1, 31, 32, 33, 255, 1000, 4099, 32768])
        gain = {"relu": 6**0.5, "silu": 3.0, "none": 3**0.5, "relu2": 1.0}[act]
        tag = f"seed={seed} it={it} {dtype} in={d_in} hidden={d_hidden} out={d_out} depth={depth} {act} bias={bias} rows={rows}"
        g = torch.Generator().manual_seed(it)

        def u(shape, fan_in):
            return ((torch.rand(*shape, generator=g) * 2 - 1) * gain / fan_in**0.5).to(dtype)

        p = dict(w_in=u((d_hidden, d_in), d_in), w_out=u((d_out, d_hidden), d_hidden))
        p["b_in"] = u((d_hidden,), d_in) if bias else None
        p["b_out"] = u((d_out,), d_hidden) if bias else None
        p["w_hid"] = u(((depth - 1) * d_hidden, d_hidden), d_hidden) if depth > 1 else None
        p["b_hid"] = u((depth - 1, d_hidden), d_hidden) if depth > 1 and bias else None
        torch.manual_seed(it)
        x = torch.randn(1, rows, d_in).to(dtype)
        dy = torch.randn(1, rows, d_out).to(dtype)
        args = (p["w_in"], p["b_in"], p["w_out"], p["b_out"], p["w_hid"], p["b_hid"], act)
        kw = {} if dtype == torch.float32 else dict(round_to=dtype)
        want_y = M.mlp_forward(x.float().view(-1, d_in), *args, **kw)
        want = M.mlp_backward(x.view(-1, d_in), dy.view(-1, d_out), *args, **kw)
        leaves = {k: (None if v is None else v.to(DEV).requires_grad_(True)) for k, v in p.items()}
        xd = x.to(DEV).requires_grad_(True)
        y = mk.fully_fused_mlp(xd, leaves["w_in"], leaves["b_in"], leaves["w_out"], leaves["b_out"], leaves["w_hid"], leaves["b_hid"], act)
        y.backward(dy.to(DEV))
        gated = act in ("relu", "relu2")
        tol = (2e-4 if dtype == torch.float32 and not gated else 2e-2) * max(1.0, depth / 4)
        d, peak = _rel(y.view(-1, d_out), want_y)
        assert float(d.max()) <= tol * peak, f"y: {tag}"
        d, peak = _rel(xd.grad.view(-1, d_in), want["dx"])
        assert float((d > tol * peak).float().mean()) <= (2e-3 if gated else 0.0), f"dx: {tag}"
        for k in ("w_in", "b_in", "w_out", "b_out", "w_hid", "b_hid"):
            if leaves[k] is not None:
                d, peak = _rel(leaves[k].grad, want["d" + k])
                assert float(d.max()) <= 1.5 * tol * peak, f"d{k}: {tag}"


@pytest.mark.parametrize("seed", range(4))
def test_reversible_mlp_random_configurations(seed):
    """rtol 2e-2 / atol 1e-2 plus half a storage ulp of the stream's peak per coupling, weight gradients relative to
    their largest entry; ReLU is checked in the forward only (its backward rebuilds the gates from 16-bit outputs)."""
    from triton_helpers_amd.layers.reversible_mlp import kernel as rk

    eps = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}

    def bad(got, want, blocks, dtype, scale_rel=False):
        d, peak = _rel(got, want)
        atol = 1e-2 + blocks * 0.5 * eps[dtype] * peak
        if scale_rel:
            atol = max(atol, 2e-2 * peak)
        return bool((d > atol + 2e-2 * want.float().abs()).any()) or not bool(torch.isfinite(got).all())

    for it in range(40):
        rng = random.Random(seed * 100003 + it)
        dtype = rng.choice([torch.bfloat16, torch.float16])
        H = rng.choice([8, 16, 20, 32, 32, 48, 64, 64, 64])
        blocks = rng.choice([1, 2, 3, 4, 4, 5, 6, 8])
        act = rng.choice(["gelu", "gelu", "silu", "none", "relu"])
        bias = rng.choice([True, False])
        rows = rng.choice([1, 31, 32, 33, 96, 1000, 1024, 4099, 32768])
        tag = f"seed={seed} it={it} {dtype} H={H} blocks={blocks} {act} bias={bias} rows={rows}"
        g = torch.Generator().manual_seed(it)
        u = lambda *s: ((torch.rand(*s, generator=g) * 2 - 1) / H**0.5).to(dtype)  # noqa: E731
        w1, b1, w2, b2 = u(blocks * 2 * H, H), (u(blocks * 2, H) if bias else None), u(blocks * 2 * H, H), (u(blocks * 2, H) if bias else None)
        torch.manual_seed(it)
        x = torch.randn(rows, 2 * H).to(dtype)
        dy = torch.randn(rows, 2 * H).to(dtype)
        want_y = R.rev_forward(x, w1, b1, w2, b2, act, round_to=dtype, stream_round_every=4).to(dtype)
        want = R.rev_backward(x, dy, w1, b1, w2, b2, act, round_to=dtype)
        leaves = [None if t is None else t.to(DEV).requires_grad_(True) for t in (w1, b1, w2, b2)]
        xd = x.to(DEV).requires_grad_(True)
        y = rk.reversible_mlp(xd, *leaves, act)
        y.backward(dy.to(DEV))
        assert not bad(y, want_y, (blocks + 3) // 4, dtype), f"y: {tag}"
        if act == "relu":
            continue
        assert not bad(xd.grad, want["dx"], blocks, dtype), f"dx: {tag}"
        for name, leaf in zip(("dw1", "db1", "dw2", "db2"), leaves):
            if leaf is not None:
                assert not bad(leaf.grad, want[name], blocks, dtype, scale_rel=True), f"{name}: {tag}"
