"""GPU parity of the fused MLP on float32 tensors (float32 matrix products) against the CPU oracle.

The reference multiplies float32 tensors in TF32 and tests them at 1e-3 forward / 1e-2 backward
(tests/test_layers/test_fully_fused_mlp.py:38-46, 231-239).  These kernels multiply in float32, so the bound here is
the accumulation-order one: rtol 1e-4 with an absolute floor of 1e-5 times the tensor's largest magnitude (weight
gradients are sums over all rows).  ReLU gates cannot flip against the float32 oracle except for pre-activations
within ~1e-6 of zero, which the seeded inputs do not produce at these sizes.
"""
import pytest
import torch

from oracle import mlp as M
pytestmark = pytest.mark.gpu
DEV = "cuda"
RTOL = 1e-4


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


def _close(got, want, what):
    got, want = got.detach().cpu().float(), want.float()
    atol = 1e-5 * float(want.abs().max())
    torch.testing.assert_close(got, want, rtol=RTOL, atol=atol, msg=lambda m: f"{what}: {m}")


SHAPES = [
    # rows(B,L), d_in, d_hidden, d_out, depth
    ((3, 40), 1, 32, 5, 1),      # reference test_forward_shallow
    ((3, 40), 1, 32, 5, 8),      # reference test_forward_deep: nine layers, staged one at a time
    ((2, 2), 8, 16, 4, 1),       # reference test_backward_shallow
    ((2, 2), 8, 16, 4, 3),       # reference test_backward_deep
    ((1, 1000), 32, 64, 16, 2),  # benchmark geometry
    ((1, 4097), 32, 64, 4, 2),   # ragged rows
    ((5, 77), 64, 64, 64, 4),
    ((2, 33), 17, 32, 33, 2),    # widths that are no multiple of 4: scalar loads and stores
    ((1, 203), 32, 64, 3, 12),   # deeper than the weights LDS holds at once
    ((1, 1), 3, 16, 1, 2),
]


@pytest.mark.parametrize("act", ["relu", "silu", "relu2", "none"])
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("shape,d_in,d_hidden,d_out,depth", SHAPES)
def test_forward_backward_float32(shape, d_in, d_hidden, d_out, depth, bias, act):
    mk = _mk()
    assert mk.get_float32_operands() == "float32"
    if act == "relu2" and depth > 3:
        pytest.skip("relu2 squares the activations at every layer: an 8-deep net overflows in any precision")
    torch.manual_seed(0)
    p = _params(d_in, d_hidden, d_out, depth, bias, torch.float32, gain=2.0)
    x = torch.randn(*shape, d_in)
    dy = torch.randn(*shape, d_out)
    args = (p["w_in"], p["b_in"], p["w_out"], p["b_out"], p["w_hid"], p["b_hid"], act)
    want_y = M.mlp_forward(x.view(-1, d_in), *args)
    want = M.mlp_backward(x.view(-1, d_in), dy.view(-1, d_out), *args)
    leaves = {k: (None if v is None else v.to(DEV).requires_grad_(True)) for k, v in p.items()}
    xd = x.to(DEV).requires_grad_(True)
    y = mk.fully_fused_mlp(xd, leaves["w_in"], leaves["b_in"], leaves["w_out"], leaves["b_out"], leaves["w_hid"], leaves["b_hid"], act)
    assert y.shape == (*shape, d_out) and y.dtype == torch.float32
    _close(y.view(-1, d_out), want_y, "y")
    y.backward(dy.to(DEV))
    assert xd.grad.dtype == torch.float32
    _close(xd.grad.view(-1, d_in), want["dx"], "dx")
    for k in ("w_in", "b_in", "w_out", "b_out", "w_hid", "b_hid"):
        if leaves[k] is not None:
            assert leaves[k].grad.dtype == torch.float32
            _close(leaves[k].grad, want["d" + k], "d" + k)


def test_float32_range_beyond_float16():
    """Inputs of 1e6 and weights of 1e-4 .. 1e5: every operand and most hidden values are outside what float16 holds
    (65504 above, 6e-8 below); the float32 path must agree with the oracle where the float16-operand mode overflows."""
    mk = _mk()
    torch.manual_seed(1)
    d_in, H, d_out, depth = 32, 64, 16, 2
    p = _params(d_in, H, d_out, depth, True, torch.float32)
    p["w_in"] = p["w_in"] * 1e-4
    p["w_hid"] = p["w_hid"] * 1e5
    p["w_out"] = p["w_out"] * 1e-7
    x = torch.randn(1, 515, d_in) * 1e6
    dy = torch.randn(1, 515, d_out)
    args = (p["w_in"], p["b_in"], p["w_out"], p["b_out"], p["w_hid"], p["b_hid"], "relu")
    want_y = M.mlp_forward(x.view(-1, d_in), *args)
    want = M.mlp_backward(x.view(-1, d_in), dy.view(-1, d_out), *args)
    assert float(x.abs().max()) > 65504 and float(p["w_hid"].abs().max()) > 1e4
    leaves = {k: v.to(DEV).requires_grad_(True) for k, v in p.items()}
    xd = x.to(DEV).requires_grad_(True)
    y = mk.fully_fused_mlp(xd, leaves["w_in"], leaves["b_in"], leaves["w_out"], leaves["b_out"], leaves["w_hid"], leaves["b_hid"], "relu")
    assert torch.isfinite(y).all()
    _close(y.view(-1, d_out), want_y, "y")
    y.backward(dy.to(DEV))
    _close(xd.grad.view(-1, d_in), want["dx"], "dx")
    for k in leaves:
        _close(leaves[k].grad, want["d" + k], "d" + k)
    previous = mk.set_float32_operands("float16")
    try:
        y16 = mk.fully_fused_mlp(xd.detach(), *(leaves[k].detach() for k in ("w_in", "b_in", "w_out", "b_out", "w_hid", "b_hid")), "relu")
    finally:
        mk.set_float32_operands(previous)
    err16 = (y16.cpu().view(-1, d_out) - want_y).abs()
    assert not bool(torch.isfinite(err16).all()) or float(err16.max()) > 0.1 * float(want_y.abs().max()), \
        "the float16-operand mode cannot represent 1e6: this input does not tell the two modes apart"


def test_float32_gradients_accumulate_and_strided_rows():
    """Gradient buffers are added to (two backward calls double them); x, dy, y and dx may be row-strided views."""
    from triton_helpers_amd import _lib

    lib = _lib.load()
    torch.manual_seed(2)
    rows, d_in, H, d_out, depth = 300, 12, 32, 7, 3
    p = {k: (None if v is None else v.to(DEV)) for k, v in _params(d_in, H, d_out, depth, True, torch.float32).items()}
    xs = torch.randn(rows, d_in + 4, device=DEV)
    dys = torch.randn(rows, d_out + 1, device=DEV)
    x, dy = xs[:, :d_in], dys[:, :d_out]
    ys = torch.full((rows, d_out + 5), 7.0, device=DEV)
    dxs = torch.full((rows, d_in + 4), 7.0, device=DEV)
    stream = _lib.current_stream(x.device)
    relu = _lib.NF_ACT["relu"]
    rc = lib.nf_mlp_fwd(x.data_ptr(), xs.stride(0), ys.data_ptr(), ys.stride(0), p["w_in"].data_ptr(), p["b_in"].data_ptr(),
                        p["w_hid"].data_ptr(), p["b_hid"].data_ptr(), p["w_out"].data_ptr(), p["b_out"].data_ptr(), rows, d_in, H,
                        d_out, depth, relu, _lib.NF_F32, _lib.NF_F32, None, 0, stream)
    _lib.check(rc, "nf_mlp_fwd")
    n = lib.nf_mlp_workspace_bytes(rows, H, depth, relu, 1, _lib.NF_F32)
    ws = torch.empty(n, dtype=torch.uint8, device=DEV)
    g = {k: torch.zeros(v.shape, dtype=torch.float32, device=DEV) for k, v in p.items()}
    for _ in range(2):
        rc = lib.nf_mlp_bwd(
            x.data_ptr(), xs.stride(0), dy.data_ptr(), dys.stride(0), dxs.data_ptr(), dxs.stride(0),
            p["w_in"].data_ptr(), p["b_in"].data_ptr(), p["w_hid"].data_ptr(), p["b_hid"].data_ptr(), p["w_out"].data_ptr(), p["b_out"].data_ptr(),
            g["w_in"].data_ptr(), g["b_in"].data_ptr(), g["w_hid"].data_ptr(), g["b_hid"].data_ptr(), g["w_out"].data_ptr(), g["b_out"].data_ptr(),
            rows, d_in, H, d_out, depth, relu, _lib.NF_F32, _lib.NF_F32, ws.data_ptr(), n, stream)
        _lib.check(rc, "nf_mlp_bwd")
    torch.cuda.synchronize()
    c = {k: v.cpu() for k, v in p.items()}
    args = (c["w_in"], c["b_in"], c["w_out"], c["b_out"], c["w_hid"], c["b_hid"], "relu")
    want_y = M.mlp_forward(x.cpu(), *args)
    want = M.mlp_backward(x.cpu(), dy.cpu(), *args)
    _close(ys[:, :d_out], want_y, "y")
    assert bool((ys[:, d_out:] == 7.0).all()) and bool((dxs[:, d_in:] == 7.0).all()), "columns past the row width were written"
    _close(dxs[:, :d_in], want["dx"], "dx")
    for k in g:
        _close(g[k], 2 * want["d" + k], "d" + k)


def _float64_relu_net(p, x, dy):
    """float64 evaluation of the ReLU network written out with torch ops: gradients, and per row the smallest
    |pre-activation| relative to the row's largest one (a row whose smallest is ~1e-7 has a gate that float32
    rounding, i.e. the order of a sum, can flip)."""
    H = p["w_in"].shape[0]
    depth = 1 if p["w_hid"] is None else p["w_hid"].shape[0] // H + 1
    leaves = {k: (None if v is None else v.double().clone().requires_grad_(True)) for k, v in p.items()}
    xx = x.double().clone().requires_grad_(True)
    margin = None
    h = xx
    for k in range(depth):
        w = leaves["w_in"] if k == 0 else leaves["w_hid"][(k - 1) * H:k * H]
        b = leaves["b_in"] if k == 0 else (None if leaves["b_hid"] is None else leaves["b_hid"][k - 1])
        z = h @ w.t() if b is None else h @ w.t() + b
        rel = (z.detach().abs() / z.detach().abs().amax(1, keepdim=True).clamp_min(1e-300)).amin(1)
        margin = rel if margin is None else torch.minimum(margin, rel)
        h = torch.relu(z)
    y = h @ leaves["w_out"].t() if leaves["b_out"] is None else h @ leaves["w_out"].t() + leaves["b_out"]
    y.backward(dy.double())
    out = {"y": y.detach(), "dx": xx.grad}
    out.update({"d" + k: v.grad for k, v in leaves.items() if v is not None})
    return out, margin


@pytest.mark.parametrize("case,rows,d_in,d_hidden,depth,d_out,bias", [
    (67, 33333, 25, 64, 9, 50, False),
    (141, 4097, 45, 64, 4, 21, True),
])
def test_deep_relu_float32_many_rows(case, rows, d_in, d_hidden, depth, d_out, bias):
    """The two cases of a randomized sweep in which 33 % / 49 % of the elements of dW_in missed rtol 1e-4.  Cause: ONE
    row of the batch has a pre-activation within float32 rounding of zero, its ReLU gate opens or closes with the order
    of the sum, and a single row carries more than 1e-4 of every weight-gradient element.  On the CPU, float32 against
    float64 reproduces the same fraction for the second case (0.4906 of dW_in) and a permuted float32 summation makes it
    vanish.  So the kernels are held to: (1) rows whose dx is grossly off are rows with such a pre-activation, and
    there are only a handful; (2) with those rows taken out of the batch every gradient matches float64 at rtol 1e-4
    with no outlier."""
    mk = _mk()
    torch.manual_seed(case)
    p = _params(d_in, d_hidden, d_out, depth, bias, torch.float32, seed=case, gain=1.7)
    x = torch.randn(rows, d_in)
    dy = torch.randn(rows, d_out)

    def run(xr, dyr):
        leaves = {k: (None if v is None else v.to(DEV).requires_grad_(True)) for k, v in p.items()}
        xd = xr.view(1, -1, d_in).to(DEV).requires_grad_(True)
        y = mk.fully_fused_mlp(xd, leaves["w_in"], leaves["b_in"], leaves["w_out"], leaves["b_out"], leaves["w_hid"], leaves["b_hid"], "relu")
        y.backward(dyr.view(1, -1, d_out).to(DEV))
        out = {"y": y.detach().view(-1, d_out), "dx": xd.grad.view(-1, d_in)}
        out.update({"d" + k: v.grad for k, v in leaves.items() if v is not None})
        return {k: v.cpu() for k, v in out.items()}

    want, margin = _float64_relu_net(p, x, dy)
    got = run(x, dy)
    _close(got["y"], want["y"], "y")
    gross = (got["dx"].double() - want["dx"]).abs().amax(1) > 1e-3 * float(want["dx"].abs().max())
    fragile = margin < 1e-5
    assert int(gross.sum()) <= 8, f"{int(gross.sum())} rows with a gross dx error"
    assert bool((fragile | ~gross).all()), "a row without a pre-activation near zero has a gross dx error"
    keep = ~fragile
    assert int(keep.sum()) >= 0.98 * rows  # nine layers x 64 units x 33333 rows: a few hundred rows come that close
    want2, _ = _float64_relu_net(p, x[keep], dy[keep])
    got2 = run(x[keep].contiguous(), dy[keep].contiguous())
    for k in want2:
        _close(got2[k], want2[k], k)
