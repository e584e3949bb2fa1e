"""GPU parity of the fused MLP against the CPU oracle (through the C ABI).

Tolerance: rtol 2e-2 / atol 1e-2 on y, dx and every dw/db for 16-bit storage, against the oracle
evaluated on the 16-bit-rounded inputs and weights with float32 arithmetic and the layer outputs
rounded to the storage dtype (what an ``nn.Linear`` chain in that dtype does; the reference's tests
compare with such chains at tolerance 1e-2, tests/test_layers/test_fully_fused_mlp.py:253-289,
372-415).  The rounding matters for ReLU: a unit whose pre-activation is within rounding of zero
switches its gate, which moves dx by a whole weight, not by a rounding error.  Weight gradients summed over many rows are compared relative to
their scale (rtol on the tensor's max magnitude).  Nets deeper than the BASELINE one (depth 2) round
to 16 bit once per layer in both directions while the oracle never rounds, so their absolute tolerance
grows with depth / 2.
"""
import pytest
import torch
import torch.nn as nn

from oracle import mlp as M

pytestmark = pytest.mark.gpu
DEV = "cuda"
RTOL, ATOL = 2e-2, 1e-2


def _mk():
    from triton_helpers_amd.layers.fully_fused_mlp import kernel

    return kernel


def _params(d_in, d_hidden, d_out, depth, bias, dtype, seed=0, gain=1.0):
    g = torch.Generator().manual_seed(seed)

    def u(shape, fan_in):
        return ((torch.rand(*shape, generator=g) * 2 - 1) * gain / fan_in**0.5).to(dtype)

    p = dict(w_in=u((d_hidden, d_in), d_in), w_out=u((d_out, d_hidden), d_hidden))
    p["b_in"] = u((d_hidden,), d_in) if bias else None
    p["b_out"] = u((d_out,), d_hidden) if bias else None
    if depth > 1:
        p["w_hid"] = u(((depth - 1) * d_hidden, d_hidden), d_hidden)
        p["b_hid"] = u((depth - 1, d_hidden), d_hidden) if bias else None
    else:
        p["w_hid"] = p["b_hid"] = None
    return p


def _dev(t):
    return None if t is None else t.to(DEV)


def _close(got, want, what, scale_rel=False, depth=2, outliers=0.0):
    """``outliers``: fraction of elements allowed outside the tolerance.  Only used for dx of ReLU nets
    on many rows: accumulation order moves a pre-activation that is within 1e-7 of zero across it, the
    gate flips and that row's dx moves by a whole weight (about 1e-5 of the elements at 2^16 rows)."""
    got, want = got.detach().cpu().float(), want.float()
    atol = ATOL * max(1.0, depth / 2)
    if scale_rel:
        atol = max(atol, RTOL * max(1.0, depth / 2) * float(want.abs().max()))
    if outliers > 0.0:
        bad = ((got - want).abs() > atol + RTOL * want.abs()).float().mean().item()
        assert bad <= outliers, f"{what}: {bad:.2e} of the elements outside tolerance (allowed {outliers:.0e})"
        return
    torch.testing.assert_close(got, want, rtol=RTOL, atol=atol, msg=lambda m: f"{what}: {m}")


SHAPES = [
    # rows(B,L), d_in, d_hidden, d_out, depth
    ((3, 40), 1, 32, 5, 1),     # reference test_forward_shallow
    ((3, 40), 1, 32, 5, 8),     # reference test_forward_deep
    ((2, 2), 8, 16, 4, 1),      # reference test_backward_shallow
    ((2, 2), 8, 16, 4, 3),      # reference test_backward_deep
    ((2, 2), 8, 16, 4, 8),
    ((1, 1000), 32, 64, 16, 2),  # BASELINE configs[2] geometry
    ((1, 4097), 32, 64, 4, 2),   # BASELINE configs[4] geometry, ragged rows
    ((5, 77), 64, 64, 64, 4),
    ((2, 33), 17, 32, 33, 2),
    # one hidden-to-hidden layer with a 64-wide input and / or output (ReLU: chain and gradient waves), ragged rows,
    # widths padded up to the tile, more rows than one round of the grid covers
    ((5, 77), 64, 64, 64, 2),    # the reference's benchmark shape (fully_fused_mlp/__main__.py:16-23)
    ((1, 4099), 64, 64, 16, 2),
    ((2, 1000), 32, 64, 64, 2),
    ((1, 200), 48, 64, 40, 2),
    # one hidden layer of width 64: the ReLU backward runs the two-layer kernels behind an identity layer
    ((1, 1000), 32, 64, 16, 1),
    ((1, 4099), 64, 64, 64, 1),
    ((2, 77), 27, 64, 3, 1),
    # two or three hidden-to-hidden layers of width 64: ReLU takes the register-resident backward for deeper nets
    ((1, 1000), 32, 64, 16, 4),
    ((1, 1000), 32, 64, 16, 3),
    ((3, 100), 64, 64, 64, 3),
    ((2, 77), 40, 64, 20, 3),
    # deeper than one launch covers: a chain of launches handing pre-activations over through the workspace
    ((1, 300), 32, 64, 16, 5),
    ((2, 100), 64, 64, 64, 8),
    ((1, 203), 32, 64, 3, 12),
    ((1, 100), 8, 32, 4, 12),
    ((1, 64), 32, 64, 16, 32),   # the forward, too, splits (the weights of 33 layers do not fit LDS)
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("act", ["relu", "silu", "relu2", "none"])
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("shape,d_in,d_hidden,d_out,depth", SHAPES)
def test_forward_backward(shape, d_in, d_hidden, d_out, depth, bias, act, dtype):
    mk = _mk()
    if act == "relu2" and depth > 3:
        pytest.skip("relu2 squares the activations at every layer: an 8-deep net overflows in any precision")
    torch.manual_seed(0)
    p = _params(d_in, d_hidden, d_out, depth, bias, dtype)
    x = torch.randn(*shape, d_in).to(dtype)
    dy = torch.randn(*shape, d_out).to(dtype)
    want_y = M.mlp_forward(x.float().view(-1, d_in), p["w_in"], p["b_in"], p["w_out"], p["b_out"], p["w_hid"], p["b_hid"], act, round_to=dtype)
    want = M.mlp_backward(x.view(-1, d_in), dy.view(-1, d_out), p["w_in"], p["b_in"], p["w_out"], p["b_out"], p["w_hid"], p["b_hid"], act, round_to=dtype)

    leaves = {k: (None if v is None else v.to(DEV).requires_grad_(True)) for k, v in p.items()}
    xd = x.to(DEV).requires_grad_(True)
    y = mk.fully_fused_mlp(xd, leaves["w_in"], leaves["b_in"], leaves["w_out"], leaves["b_out"], leaves["w_hid"], leaves["b_hid"], act)
    assert y.shape == (*shape, d_out) and y.dtype == dtype
    _close(y.view(-1, d_out), want_y, "y", depth=depth)
    y.backward(dy.to(DEV))
    _close(xd.grad.view(-1, d_in), want["dx"], "dx", depth=depth)
    for k in ("w_in", "b_in", "w_out", "b_out", "w_hid", "b_hid"):
        if leaves[k] is None:
            continue
        _close(leaves[k].grad, want["d" + k], "d" + k, scale_rel=True, depth=depth)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("d_in,d_out", [(64, 64), (64, 16), (32, 64)])
def test_wide_one_hidden_layer_many_rows(d_in, d_out, bias, dtype):
    """More rows than one round of the grid covers (ragged), through autograd: forward, dx and the rounded weight
    gradients of the chain / gradient wave kernels against the oracle's 16-bit mode.  A handful of dx rows may differ by
    a flipped ReLU gate (a pre-activation within rounding of zero and another order of the sum)."""
    mk = _mk()
    rows = 70001
    torch.manual_seed(11)
    p = _params(d_in, 64, d_out, 2, bias, dtype, seed=11)
    x = torch.randn(1, rows, d_in).to(dtype)
    dy = torch.randn(1, rows, d_out).to(dtype)
    args = (p["w_in"], p["b_in"], p["w_out"], p["b_out"], p["w_hid"], p["b_hid"], "relu")
    want_y = M.mlp_forward(x.float().view(-1, d_in), *args, round_to=dtype)
    want = M.mlp_backward(x.view(-1, d_in), dy.view(-1, d_out), *args, round_to=dtype)
    leaves = {k: (None if v is None else v.to(DEV).requires_grad_(True)) for k, v in p.items()}
    xd = x.to(DEV).requires_grad_(True)
    y = mk.fully_fused_mlp(xd, leaves["w_in"], leaves["b_in"], leaves["w_out"], leaves["b_out"], leaves["w_hid"], leaves["b_hid"], "relu")
    _close(y.view(-1, d_out), want_y, "y")
    y.backward(dy.to(DEV))
    _close(xd.grad.view(-1, d_in), want["dx"], "dx", outliers=1e-3)
    for k in ("w_in", "b_in", "w_out", "b_out", "w_hid", "b_hid"):
        if leaves[k] is not None:
            _close(leaves[k].grad, want["d" + k], "d" + k, scale_rel=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
    "act,gain,d_in,d_hidden,d_out,depth",
    [
        ("relu", 6**0.5, 32, 64, 16, 5),
        ("relu", 6**0.5, 32, 64, 16, 9),
        ("relu", 6**0.5, 64, 64, 3, 12),
        ("relu", 6**0.5, 16, 32, 8, 11),
        ("silu", 3.0, 32, 64, 16, 3),
        ("silu", 3.0, 32, 64, 16, 6),
        ("none", 3**0.5, 32, 64, 16, 7),
    ],
)
def test_chained_launches_keep_signal(act, gain, d_in, d_hidden, d_out, depth, dtype):
    """Deep nets with variance-preserving weights: activations and gradients stay O(1) through every launch
    boundary, so a wrong hand-over (activation applied twice or not at all, a missing act'(x) on the gradient,
    a weight slice off by one layer) shows at full size instead of drowning in a shrinking signal."""
    mk = _mk()
    rows = 777
    torch.manual_seed(1)
    p = _params(d_in, d_hidden, d_out, depth, True, dtype, seed=3, gain=gain)
    x = torch.randn(1, rows, d_in).to(dtype)
    dy = torch.randn(1, rows, d_out).to(dtype)
    want_y = M.mlp_forward(x.float().view(-1, d_in), p["w_in"], p["b_in"], p["w_out"], p["b_out"], p["w_hid"], p["b_hid"], act, round_to=dtype)
    want = M.mlp_backward(x.view(-1, d_in), dy.view(-1, d_out), p["w_in"], p["b_in"], p["w_out"], p["b_out"], p["w_hid"], p["b_hid"], act, round_to=dtype)
    assert float(want_y.abs().mean()) > 0.05 and float(want["dx"].abs().mean()) > 0.05, "the signal must survive the depth"
    leaves = {k: v.to(DEV).requires_grad_(True) for k, v in p.items()}
    xd = x.to(DEV).requires_grad_(True)
    y = mk.fully_fused_mlp(xd, leaves["w_in"], leaves["b_in"], leaves["w_out"], leaves["b_out"], leaves["w_hid"], leaves["b_hid"], act)
    y.backward(dy.to(DEV))

    def rel(got, ref):  # error relative to the tensor's scale: deep 16-bit chains accumulate rounding layer by layer
        got, ref = got.detach().cpu().float(), ref.float()
        return float((got - ref).abs().max() / ref.abs().max())

    tol = RTOL * max(1.0, depth / 4)
    assert rel(y.view(-1, d_out), want_y) <= tol
    # ReLU: rows whose gate flips on a rounding difference move by a whole weight; compare the bulk
    dxe = (xd.grad.view(-1, d_in).cpu().float() - want["dx"].float()).abs() / want["dx"].float().abs().max()
    assert float((dxe > tol).float().mean()) <= (2e-3 if act == "relu" else 0.0), f"dx: max rel {float(dxe.max()):.3g}"
    for k in ("w_in", "b_in", "w_out", "b_out", "w_hid", "b_hid"):
        assert rel(leaves[k].grad, want["d" + k]) <= tol, k


@pytest.mark.parametrize("depth", [1, 2, 6])
def test_step_replays_from_a_hip_graph(depth):
    """The library only enqueues kernels on the caller's stream (no allocation, no synchronisation, no memset), so a
    forward + backward step can be captured once and replayed.  Every replay, with new inputs copied into the captured
    tensors and eager work in between, must give what the eager step gives."""
    mk = _mk()
    dtype = torch.bfloat16
    rows, d_in, H, d_out = 3000, 32, 64, 16
    p = {k: (None if v is None else v.to(DEV).requires_grad_(True)) for k, v in _params(d_in, H, d_out, depth, True, dtype, gain=6**0.5).items()}
    x = torch.randn(1, rows, d_in).to(dtype).to(DEV).requires_grad_(True)
    dy = torch.randn(1, rows, d_out).to(dtype).to(DEV)
    leaves = [x] + [t for t in p.values() if t is not None]

    def step():
        for t in leaves:
            t.grad = None
        y = mk.fully_fused_mlp(x, p["w_in"], p["b_in"], p["w_out"], p["b_out"], p["w_hid"], p["b_hid"], "relu")
        y.backward(dy)
        return y

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        y_static = step()
    grads_static = [t.grad for t in leaves]
    for seed in (1, 2, 3):
        torch.manual_seed(seed)
        x_new = torch.randn(1, rows, d_in).to(dtype).to(DEV)
        dy_new = torch.randn(1, rows, d_out).to(dtype).to(DEV)
        with torch.no_grad():
            x.copy_(x_new)
            dy.copy_(dy_new)
        g.replay()
        torch.cuda.synchronize()
        got_y = y_static.clone()
        got = [t.clone() for t in grads_static]
        # the same step eagerly, on fresh leaves holding the same values
        xe = x_new.clone().requires_grad_(True)
        pe = {k: (None if v is None else v.detach().clone().requires_grad_(True)) for k, v in p.items()}
        ye = mk.fully_fused_mlp(xe, pe["w_in"], pe["b_in"], pe["w_out"], pe["b_out"], pe["w_hid"], pe["b_hid"], "relu")
        ye.backward(dy_new)
        torch.cuda.synchronize()
        assert torch.equal(got_y, ye)
        want = [xe.grad] + [t.grad for t in pe.values() if t is not None]
        assert torch.equal(got[0], want[0])  # dx: no atomics, bitwise
        for a, b in zip(got[1:], want[1:]):  # dW: float atomics, order may differ
            torch.testing.assert_close(a.float(), b.float(), rtol=2e-2, atol=1e-2 * float(b.float().abs().max()))


def test_backward_without_workspace_takes_the_one_launch_kernel():
    """A C caller that passes no workspace still gets the gradients of a narrow deep net (slower kernel); a net that
    fits no single launch is refused with the size it needs."""
    from triton_helpers_amd import _lib

    lib = _lib.load()
    rows, d_in, H, d_out, depth = 500, 8, 32, 4, 4
    dtype = torch.bfloat16
    p = {k: _dev(v) for k, v in _params(d_in, H, d_out, depth, True, dtype, seed=7, gain=6**0.5).items()}
    torch.manual_seed(2)
    x = torch.randn(rows, d_in).to(dtype).to(DEV)
    dy = torch.randn(rows, d_out).to(dtype).to(DEV)
    relu = _lib.NF_ACT["relu"]
    code = _lib.dtype_code(dtype)
    stream = _lib.current_stream(x.device)

    def run(ws):
        dx = torch.empty_like(x)
        g = {k: torch.zeros(v.shape, dtype=torch.float32, device=DEV) for k, v in p.items()}
        rc = lib.nf_mlp_bwd(
            x.data_ptr(), d_in, dy.data_ptr(), d_out, dx.data_ptr(), d_in,
            p["w_in"].data_ptr(), p["b_in"].data_ptr(), p["w_hid"].data_ptr(), p["b_hid"].data_ptr(), p["w_out"].data_ptr(), p["b_out"].data_ptr(),
            g["w_in"].data_ptr(), g["b_in"].data_ptr(), g["w_hid"].data_ptr(), g["b_hid"].data_ptr(), g["w_out"].data_ptr(), g["b_out"].data_ptr(),
            rows, d_in, H, d_out, depth, relu, code, code, _lib.ptr(ws), 0 if ws is None else ws.numel(), stream)
        _lib.check(rc, "nf_mlp_bwd")
        torch.cuda.synchronize()
        return dx, g

    n = lib.nf_mlp_workspace_bytes(rows, H, depth, relu, 1, code)
    assert n > 0
    dx_a, g_a = run(torch.empty(n, dtype=torch.uint8, device=DEV))
    dx_b, g_b = run(None)
    for k in g_a:
        scale = float(g_a[k].abs().max())
        assert float((g_a[k] - g_b[k]).abs().max()) <= 2e-2 * scale, k
    bad = ((dx_a.float() - dx_b.float()).abs() > 2e-2 * float(dx_a.float().abs().max())).float().mean().item()
    assert bad <= 2e-3
    # width 64, depth 8: no single launch holds it
    rc = lib.nf_mlp_bwd(1, 32, 1, 16, None, 32, 1, None, 1, None, 1, None, 1, None, 1, None, 1, None,
                        rows, 32, 64, 16, 8, relu, code, code, None, 0, stream)
    assert rc == -1 and b"workspace" in lib.nf_last_error()


@pytest.mark.parametrize("act", ["relu", "silu", "none"])
@pytest.mark.parametrize("shape,d_in,d_hidden,d_out,depth", [((3, 40), 1, 32, 5, 1), ((2, 2), 8, 16, 4, 3), ((1, 1000), 32, 64, 16, 2)])
def test_float32_storage(shape, d_in, d_hidden, d_out, depth, act):
    """float32 tensors with ``set_float32_operands("float16")``: the reference multiplies them in TF32 (10-bit
    mantissa) and its tests allow 1e-3 forward, 1e-2 backward (tests/test_layers/test_fully_fused_mlp.py:42-46,
    235-239); this mode multiplies float16 roundings of the same values with float32 accumulation and returns
    float32.  Checked against the float32 oracle on the unrounded values at those tolerances (relative to each
    tensor's scale), and the results must be float32.  (The default float32 mode: test_fused_mlp_f32_gpu.py.)"""
    mk = _mk()
    previous = mk.set_float32_operands("float16")
    try:
        _float32_storage_half_operands(mk, shape, d_in, d_hidden, d_out, depth, act)
    finally:
        mk.set_float32_operands(previous)


def _float32_storage_half_operands(mk, shape, d_in, d_hidden, d_out, depth, act):
    torch.manual_seed(0)
    p = _params(d_in, d_hidden, d_out, depth, True, torch.float32)
    x = torch.randn(*shape, d_in)
    dy = torch.randn(*shape, d_out)
    if act == "relu":
        # a unit within float16 rounding of zero switches its gate and moves dx by a whole weight: compare with the
        # oracle evaluated at the same rounding points (float16 operands), as the 16-bit tests do
        h = {k: (None if v is None else v.half()) for k, v in p.items()}
        args = (h["w_in"], h["b_in"], h["w_out"], h["b_out"], h["w_hid"], h["b_hid"], act)
        want_y = M.mlp_forward(x.half().float().view(-1, d_in), *args, round_to=torch.float16)
        want = M.mlp_backward(x.half().view(-1, d_in), dy.half().view(-1, d_out), *args, round_to=torch.float16)
    else:
        args = (p["w_in"], p["b_in"], p["w_out"], p["b_out"], p["w_hid"], p["b_hid"], act)
        want_y = M.mlp_forward(x.view(-1, d_in), *args)
        want = M.mlp_backward(x.view(-1, d_in), dy.view(-1, d_out), *args)
    leaves = {k: (None if v is None else v.to(DEV).requires_grad_(True)) for k, v in p.items()}
    xd = x.to(DEV).requires_grad_(True)
    y = mk.fully_fused_mlp(xd, leaves["w_in"], leaves["b_in"], leaves["w_out"], leaves["b_out"], leaves["w_hid"], leaves["b_hid"], act)
    assert y.dtype == torch.float32 and y.shape == (*shape, d_out)

    def close(got, ref, tol, what):
        ref = ref.float()
        scale = max(1.0, float(ref.abs().max()))
        tol = max(tol, 1e-2) if act == "relu" else tol
        torch.testing.assert_close(got.detach().cpu(), ref, rtol=tol, atol=tol * scale, msg=lambda m: f"{what}: {m}")

    close(y.view(-1, d_out), want_y, 2e-3 * depth, "y")
    y.backward(dy.to(DEV))
    assert xd.grad.dtype == torch.float32
    close(xd.grad.view(-1, d_in), want["dx"], 1e-2, "dx")
    for k in ("w_in", "b_in", "w_out", "b_out", "w_hid", "b_hid"):
        if leaves[k] is not None:
            assert leaves[k].grad.dtype == torch.float32
            close(leaves[k].grad, want["d" + k], 1e-2, "d" + k)


def test_config2_sample_vs_oracle():
    """BASELINE configs[2] (32->64->64->16, ReLU, bf16, no bias) on 65536 rows against the oracle."""
    mk = _mk()
    torch.manual_seed(0)
    p = _params(32, 64, 16, 2, False, torch.bfloat16)
    rows = 65536
    x = torch.randn(1, rows, 32).bfloat16()
    dy = torch.randn(1, rows, 16).bfloat16()
    want_y = M.mlp_forward(x.view(-1, 32), p["w_in"], None, p["w_out"], None, p["w_hid"], None, "relu", round_to=torch.bfloat16)
    want = M.mlp_backward(x.view(-1, 32), dy.view(-1, 16), p["w_in"], None, p["w_out"], None, p["w_hid"], None, "relu", round_to=torch.bfloat16)
    leaves = {k: (None if v is None else v.to(DEV).requires_grad_(True)) for k, v in p.items()}
    xd = x.to(DEV).requires_grad_(True)
    y = mk.fully_fused_mlp(xd, leaves["w_in"], None, leaves["w_out"], None, leaves["w_hid"], None)
    _close(y.view(-1, 16), want_y, "y")
    y.backward(dy.to(DEV))
    _close(xd.grad.view(-1, 32), want["dx"], "dx", outliers=1e-4)
    for k in ("w_in", "w_out", "w_hid"):
        _close(leaves[k].grad, want["d" + k], "d" + k, scale_rel=True)


def test_full_size_properties_config2():
    """configs[2] at 2^20 rows: linearity of the backward in dy, additivity of dW over row halves,
    and forward agreement of a 4096-row sample with the oracle."""
    mk = _mk()
    torch.manual_seed(0)
    p = {k: _dev(v) for k, v in _params(32, 64, 16, 2, False, torch.bfloat16).items()}
    rows = 2**20
    x = torch.randn(1, rows, 32, device=DEV).bfloat16()
    dy = torch.randn(1, rows, 16, device=DEV).bfloat16()

    def grads(xx, dd):
        leaves = {k: (None if v is None else v.detach().clone().requires_grad_(True)) for k, v in p.items()}
        xr = xx.detach().clone().requires_grad_(True)
        y = mk.fully_fused_mlp(xr, leaves["w_in"], None, leaves["w_out"], None, leaves["w_hid"], None)
        y.backward(dd)
        return y, xr.grad, {k: leaves[k].grad.float() for k in ("w_in", "w_out", "w_hid")}

    y, dx, dw = grads(x, dy)
    idx = torch.randperm(rows)[:4096]
    cpu = {k: (None if v is None else v.cpu()) for k, v in p.items()}
    want = M.mlp_forward(x[0, idx.to(DEV)].cpu(), cpu["w_in"], None, cpu["w_out"], None, cpu["w_hid"], None, "relu", round_to=torch.bfloat16)
    _close(y[0, idx.to(DEV)], want, "y sample")
    half = rows // 2
    _, _, dwa = grads(x[:, :half], dy[:, :half])
    _, _, dwb = grads(x[:, half:], dy[:, half:])
    for k in dw:
        s = dwa[k] + dwb[k]
        torch.testing.assert_close(dw[k], s, rtol=RTOL, atol=RTOL * float(s.abs().max()))
    _, dx2, _ = grads(x, dy * 2)
    torch.testing.assert_close(dx2.float(), dx.float() * 2, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("depth", [1, 4, 8])
def test_module_autocast(depth):
    # reference test_module (test_fully_fused_mlp.py:372-415): same seed => same init as an nn.Linear chain
    from triton_helpers_amd.layers.fully_fused_mlp import FullyFusedMLP

    torch.manual_seed(0)
    x = torch.randn(2, 2, 8, device=DEV, requires_grad=True)
    torch.manual_seed(0)
    lin_in = nn.Linear(8, 16)
    lin_hid = [nn.Linear(16, 16) for _ in range(depth - 1)]
    lin_out = nn.Linear(16, 4)
    torch.manual_seed(0)
    layer = FullyFusedMLP(8, 16, 4, depth=depth).to(DEV)
    assert torch.equal(layer.w_in.cpu(), lin_in.weight) and torch.equal(layer.b_out.cpu(), lin_out.bias)
    if depth > 1:
        assert torch.equal(layer.w_hid.cpu(), torch.cat([l.weight for l in lin_hid], 0))
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        y = layer(x)
    assert y.dtype == torch.float16
    y.sum().backward()
    ref_net = nn.Sequential(lin_in, nn.ReLU(), *[m for l in lin_hid for m in (l, nn.ReLU())], lin_out)
    xc = x.detach().cpu().requires_grad_(True)
    yr = ref_net(xc)
    yr.sum().backward()
    _close(y, yr.detach(), "y")
    _close(x.grad, xc.grad, "dx")
    _close(layer.w_in.grad, lin_in.weight.grad, "dw_in", scale_rel=True)
    _close(layer.b_in.grad, lin_in.bias.grad, "db_in", scale_rel=True)
    _close(layer.w_out.grad, lin_out.weight.grad, "dw_out", scale_rel=True)
    _close(layer.b_out.grad, lin_out.bias.grad, "db_out", scale_rel=True)
    expect = {"w_in", "b_in", "w_out", "b_out"} | ({"w_hid", "b_hid"} if depth > 1 else set())
    assert set(layer.state_dict().keys()) == expect


@pytest.mark.parametrize("x_dtype,w_dtype", [(torch.float16, torch.bfloat16), (torch.bfloat16, torch.float16)])
@pytest.mark.parametrize("depth,bias", [(2, True), (2, False), (3, True), (1, True)])
def test_input_in_the_other_16bit_dtype(x_dtype, w_dtype, depth, bias):
    """x stored in the other 16-bit dtype than the parameters (an fp16 encoder output in front of bf16 weights): the
    result is bit-identical to casting x first, y comes in the parameters' dtype and dx in x's."""
    mk = _mk()
    torch.manual_seed(11)
    p = {k: _dev(v) for k, v in _params(32, 64, 16, depth, bias, w_dtype, seed=5).items()}
    rows = 4099
    x = torch.randn(1, rows, 32).to(x_dtype).to(DEV)
    dy = torch.randn(1, rows, 16).to(w_dtype).to(DEV)

    def run(xin):
        xin = xin.clone().requires_grad_(True)
        ws = {k: (None if v is None else v.clone().requires_grad_(True)) for k, v in p.items()}
        y = mk.fully_fused_mlp(xin, ws["w_in"], ws["b_in"], ws["w_out"], ws["b_out"], ws["w_hid"], ws["b_hid"], "relu")
        y.backward(dy)
        return y, xin.grad, {k: v.grad for k, v in ws.items() if v is not None}

    y_mixed, dx_mixed, g_mixed = run(x)
    y_cast, dx_cast, g_cast = run(x.to(w_dtype))
    assert y_mixed.dtype == w_dtype and dx_mixed.dtype == x_dtype
    assert torch.equal(y_mixed, y_cast)
    # dx is rounded once from float32 to x's dtype instead of to the parameters' dtype and then again by autograd
    torch.testing.assert_close(dx_mixed.float(), dx_cast.float(), rtol=1e-2, atol=1e-3)
    for k in g_cast:
        torch.testing.assert_close(g_mixed[k].float(), g_cast[k].float(), rtol=2e-2, atol=2e-2 * float(g_cast[k].float().abs().max()))


def test_argument_errors():
    mk = _mk()
    p = {k: _dev(v) for k, v in _params(8, 16, 4, 1, True, torch.float16).items()}
    x = torch.randn(2, 3, 8, device=DEV).half()
    with pytest.raises(AssertionError):
        mk.fully_fused_mlp(x[..., :7], p["w_in"], p["b_in"], p["w_out"], p["b_out"])  # input dim mismatch
    with pytest.raises(AssertionError):
        mk.fully_fused_mlp(x, p["w_in"], p["b_in"], p["w_out"], p["b_out"], activation="tanh")
    with pytest.raises(ValueError):
        mk.fully_fused_mlp(x[0], p["w_in"], p["b_in"], p["w_out"], p["b_out"])  # x must be 3-D
    with pytest.raises(NotImplementedError):
        mk.fully_fused_mlp(x.double(), *(p[k].double() for k in ("w_in", "b_in", "w_out", "b_out")))
    with pytest.raises(AssertionError):
        mk.fully_fused_mlp(x, *(p[k].float() for k in ("w_in", "b_in", "w_out", "b_out")))  # float32 parameters, 16-bit input
    w24 = torch.zeros(24, 8, device=DEV).half()
    with pytest.raises(AssertionError):
        mk.fully_fused_mlp(x, w24, None, torch.zeros(4, 24, device=DEV).half(), None)  # hidden not a power of 2
    y = mk.fully_fused_mlp(x[:, :0], p["w_in"], p["b_in"], p["w_out"], p["b_out"])
    assert y.shape == (2, 0, 4)


def test_relu2_gradients_far_above_unit_scale():
    """A randomly drawn shape (1 -> 16 -> 16 -> 33, ReLU^2, 70001 rows) on which 1.1e-3 of the dx elements once fell
    outside rtol 2e-2 / atol 1e-2.  ReLU^2 squares the activations at every layer: with a single N(0,1) input the
    outputs reach the thousands, and dx of a row is a sum of products of that size, each carrying the 16-bit rounding
    of its operands (the kernel rounds act'(z) and dz of every layer to the storage dtype, half an ulp = 2^-9 each in
    bfloat16).  An element whose terms cancel keeps an absolute error proportional to the TERMS.  The guaranteed
    bound is therefore the running error bound of the back-propagation,

        |dx - dx_oracle| <= rtol |dx_oracle| + atol + n 2^-9 |W_in|^T (|act'(z1)| . |W_hid|^T (|act'(z2)| . |W_out|^T |dy|)),

    with n = 2 roundings per layer; no element of this case is outside it."""
    mk = _mk()
    case, rows, d_in, H, d_out, depth, dtype = 190, 70001, 1, 16, 33, 2, torch.bfloat16
    torch.manual_seed(case)
    p = _params(d_in, H, d_out, depth, False, dtype, seed=case)
    x = torch.randn(1, rows, d_in).to(dtype)
    dy = torch.randn(1, rows, d_out).to(dtype)
    want_y = M.mlp_forward(x.float().view(-1, d_in), p["w_in"], None, p["w_out"], None, p["w_hid"], None, "relu2", round_to=dtype)
    want = M.mlp_backward(x.view(-1, d_in), dy.view(-1, d_out), p["w_in"], None, p["w_out"], None, p["w_hid"], None, "relu2", round_to=dtype)
    leaves = {k: (None if v is None else v.to(DEV).requires_grad_(True)) for k, v in p.items()}
    xd = x.to(DEV).requires_grad_(True)
    y = mk.fully_fused_mlp(xd, leaves["w_in"], None, leaves["w_out"], None, leaves["w_hid"], None, "relu2")
    y.backward(dy.to(DEV))

    # the absolute-value back-propagation (relu2'(z) = 2 max(z, 0))
    w_in, w_hid, w_out = (p[k].float() for k in ("w_in", "w_hid", "w_out"))
    rnd = lambda t: t.to(dtype).float()  # noqa: E731
    z1 = x.float().view(-1, d_in) @ w_in.t()
    z2 = rnd(z1.clamp_min(0) * z1) @ w_hid.t()
    a = (dy.float().view(-1, d_out).abs() @ w_out.abs()) * (2 * z2.clamp_min(0))
    a = (a @ w_hid.abs()) * (2 * z1.clamp_min(0))
    terms = a @ w_in.abs()
    got, ref = xd.grad.view(-1, d_in).cpu().float(), want["dx"]
    excess = (got - ref).abs() - (RTOL * ref.abs() + ATOL + 2 * (depth + 1) * 2.0**-9 * terms)
    assert float(excess.max()) <= 0.0, f"{int((excess > 0).sum())} elements of dx outside the running error bound"
    ref = want_y
    floor = ATOL * max(1.0, float(ref.pow(2).mean().sqrt()))
    assert not bool(((y.view(-1, d_out).cpu().float() - ref).abs() > floor + RTOL * ref.abs()).any())
    for k in ("w_in", "w_out", "w_hid"):
        _close(leaves[k].grad, want["d" + k], "d" + k, scale_rel=True)


@pytest.mark.parametrize("rows,d_in,d_out,bias,dtype,x_other,pad", [
    (1, 32, 16, False, torch.bfloat16, False, 0),
    (33, 4, 4, True, torch.float16, False, 4),
    (383, 12, 8, False, torch.bfloat16, True, 8),
    (385, 20, 12, True, torch.float16, True, 0),
    (4097, 28, 16, True, torch.bfloat16, True, 4),
    (70001, 32, 4, False, torch.bfloat16, False, 8),
    (200003, 24, 16, True, torch.float16, False, 0),
])
def test_decoder_shape_kernels(rows, d_in, d_out, bias, dtype, x_other, pad):
    """d_in <= 32 -> 64 -> 64 -> d_out <= 16 with ReLU takes kernels of its own in both directions (twelve / eight waves per
    workgroup, rows behind buffer descriptors): row counts around the 32-row chunk and the 384 / 256 rows of a workgroup's
    pass, widths that are multiples of four, x as a column slice of a wider tensor and stored in the other 16-bit type,
    with and without biases."""
    mk = _mk()
    xdt = dtype if not x_other else (torch.float16 if dtype == torch.bfloat16 else torch.bfloat16)
    torch.manual_seed(rows)
    p = _params(d_in, 64, d_out, 2, bias, dtype, seed=rows)
    xs = torch.randn(1, rows, d_in + pad).to(xdt)
    dy = torch.randn(1, rows, d_out).to(dtype)
    xr = xs[..., :d_in].to(dtype)  # what a cast in front of the kernel would hand over
    args = (p["w_in"], p["b_in"], p["w_out"], p["b_out"], p["w_hid"], p["b_hid"], "relu")
    want_y = M.mlp_forward(xr.float().reshape(-1, d_in), *args, round_to=dtype)
    want = M.mlp_backward(xr.reshape(-1, d_in), dy.view(-1, d_out), *args, round_to=dtype)
    leaves = {k: (None if v is None else v.to(DEV).requires_grad_(True)) for k, v in p.items()}
    xsd = xs.to(DEV).requires_grad_(True)
    y = mk.fully_fused_mlp(xsd[..., :d_in], leaves["w_in"], leaves["b_in"], leaves["w_out"], leaves["b_out"], leaves["w_hid"], leaves["b_hid"], "relu")
    assert y.dtype == dtype
    _close(y.view(-1, d_out), want_y, "y")
    y.backward(dy.to(DEV))
    assert xsd.grad.dtype == xdt
    if pad:
        assert float(xsd.grad[..., d_in:].abs().max()) == 0.0
    _close(xsd.grad[..., :d_in].reshape(-1, d_in), want["dx"], "dx", outliers=1e-3)
    for k in ("w_in", "b_in", "w_out", "b_out", "w_hid", "b_hid"):
        if leaves[k] is not None:
            _close(leaves[k].grad, want["d" + k], "d" + k, scale_rel=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("d_in,d_out", [(32, 16), (64, 64), (64, 16), (32, 64), (48, 40)])
def test_rounded_weight_gradients_entry_point(dtype, bias, d_in, d_out):
    """nf_mlp_bwd_rounded against nf_mlp_bwd on the same inputs: the same dx bit for bit, weight and bias gradients equal to
    the float32 accumulators rounded once (one unit in the last place for the order of the sums), written into buffers
    that held garbage, and the same bits on a second call."""
    from triton_helpers_amd import _lib

    lib = _lib.load()
    rows, H = 50000, 64
    code = _lib.dtype_code(dtype)
    relu = _lib.NF_ACT["relu"]
    p = {k: (None if v is None else v.to(DEV)) for k, v in _params(d_in, H, d_out, 2, bias, dtype, seed=5).items()}
    torch.manual_seed(5)
    x = torch.randn(rows, d_in, device=DEV).to(dtype)
    dy = torch.randn(rows, d_out, device=DEV).to(dtype)
    stream = _lib.current_stream(x.device)
    names = ("w_in", "b_in", "w_hid", "b_hid", "w_out", "b_out")
    acc = {k: (None if p[k] is None else torch.zeros(p[k].shape, dtype=torch.float32, device=DEV)) for k in names}
    dx_a = torch.empty_like(x)
    rc = lib.nf_mlp_bwd(x.data_ptr(), d_in, dy.data_ptr(), d_out, dx_a.data_ptr(), d_in,
                        *(_lib.ptr(p[k]) for k in names), *(_lib.ptr(acc[k]) for k in names),
                        rows, d_in, H, d_out, 2, relu, code, code, None, 0, stream)
    _lib.check(rc, "nf_mlp_bwd")
    n = lib.nf_mlp_bwd_rounded_workspace_bytes(d_in, H, d_out)
    ws = torch.empty(n, dtype=torch.uint8, device=DEV)
    runs = []
    for _ in range(2):
        out = {k: (None if p[k] is None else torch.full(p[k].shape, float("nan"), dtype=dtype, device=DEV)) for k in names}
        dx_b = torch.empty_like(x)
        rc = lib.nf_mlp_bwd_rounded(x.data_ptr(), d_in, dy.data_ptr(), d_out, dx_b.data_ptr(), d_in,
                                    *(_lib.ptr(p[k]) for k in names), *(_lib.ptr(out[k]) for k in names),
                                    rows, d_in, H, d_out, 2, relu, code, code, ws.data_ptr(), n, stream)
        _lib.check(rc, "nf_mlp_bwd_rounded")
        torch.cuda.synchronize()
        runs.append((dx_b, out))
    dx_b, out = runs[0]
    assert torch.equal(dx_a, dx_b)
    # one unit in the last place of the storage type: at most 2^-7 (bfloat16) / 2^-10 (float16) of a value's magnitude
    eps = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    for k in names:
        if p[k] is None:
            continue
        want = acc[k].to(dtype).float()
        got = out[k].float()
        assert torch.isfinite(got).all(), k
        assert float((got - want).abs().max()) <= eps * float(want.abs().max()), k
        assert torch.equal(out[k], runs[1][1][k]), f"{k}: two calls differ"
    # shapes it is not built for are refused before anything runs
    rc = lib.nf_mlp_bwd_rounded(x.data_ptr(), d_in, dy.data_ptr(), d_out, None, d_in,
                                *(_lib.ptr(p[k]) for k in names), *(_lib.ptr(out[k]) for k in names),
                                rows, d_in, H, d_out, 2, _lib.NF_ACT["silu"], code, code, ws.data_ptr(), n, stream)
    assert rc == _lib.NF_EUNSUPPORTED
