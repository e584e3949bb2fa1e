"""Pins the MLP and reversible-MLP oracles (CPU only).

MLP: against a chain of ``nn.Linear`` modules with autograd -- the baseline the reference's own
tests use (tests/test_layers/test_fully_fused_mlp.py:21-35, 253-260).
Reversible: no reference exists ("parity unpinned"); pinned by inverse(forward(x)) == x, by autograd
through an independently written plain composition, and by a finite-difference check.
"""
import pytest
import torch
import torch.nn as nn

from oracle import mlp as M
from oracle import reversible as R


class RefMLP(nn.Module):
    """Same structure as the reference tests' baseline module."""

    def __init__(self, d_in, d_hidden, d_out, depth=1, act=nn.ReLU()):
        super().__init__()
        self.first = nn.Linear(d_in, d_hidden)
        self.mid = nn.ModuleList([nn.Linear(d_hidden, d_hidden) for _ in range(depth - 1)])
        self.last = nn.Linear(d_hidden, d_out)
        self.act = act

    def forward(self, x):
        x = self.act(self.first(x))
        for l in self.mid:
            x = self.act(l(x))
        return self.last(x)


ACTS = {"relu": nn.ReLU(), "silu": nn.SiLU(), "none": nn.Identity(), "gelu": nn.GELU()}


def _stack(net):
    if len(net.mid) == 0:
        return None, None
    return torch.cat([l.weight for l in net.mid], 0), torch.stack([l.bias for l in net.mid], 0)


@pytest.mark.parametrize("act", ["relu", "silu", "none", "gelu"])
@pytest.mark.parametrize("depth", [1, 3, 8])
def test_mlp_forward_backward_vs_linear_chain(act, depth):
    torch.manual_seed(0)
    net = RefMLP(8, 16, 4, depth, ACTS[act]).double()
    x = torch.randn(6, 8, dtype=torch.double, requires_grad=True)
    y = net(x)
    dy = torch.randn_like(y)
    y.backward(dy)
    w_hid, b_hid = _stack(net)
    f = lambda t: None if t is None else t.detach().float()  # noqa: E731
    got = M.mlp_forward(f(x), f(net.first.weight), f(net.first.bias), f(net.last.weight), f(net.last.bias), f(w_hid), f(b_hid), act)
    torch.testing.assert_close(got, y.detach().float(), rtol=1e-5, atol=1e-5)
    g = M.mlp_backward(f(x), f(dy), f(net.first.weight), f(net.first.bias), f(net.last.weight), f(net.last.bias), f(w_hid), f(b_hid), act)
    torch.testing.assert_close(g["dx"], x.grad.float(), rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(g["dw_in"], net.first.weight.grad.float(), rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(g["db_in"], net.first.bias.grad.float(), rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(g["dw_out"], net.last.weight.grad.float(), rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(g["db_out"], net.last.bias.grad.float(), rtol=1e-4, atol=1e-5)
    if depth > 1:
        torch.testing.assert_close(g["dw_hid"], torch.cat([l.weight.grad for l in net.mid], 0).float(), rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(g["db_hid"], torch.stack([l.bias.grad for l in net.mid], 0).float(), rtol=1e-4, atol=1e-5)


def test_relu2_matches_definition():
    # reference ops.py:58-66: relu2(x) = max(x,0)*x ; tests/test_ops.py compares with F.relu(x)**2
    z = torch.linspace(-3, 3, 101)
    torch.testing.assert_close(M.activation(z, "relu2"), torch.relu(z) ** 2)


def test_mlp_no_bias_and_rounding_variant():
    torch.manual_seed(1)
    x = torch.randn(5, 32)
    w_in, w_hid, w_out = torch.randn(64, 32) / 6, torch.randn(64, 64) / 8, torch.randn(16, 64) / 8
    ref = torch.relu(torch.relu(x @ w_in.t()) @ w_hid.t()) @ w_out.t()
    torch.testing.assert_close(M.mlp_forward(x, w_in, None, w_out, None, w_hid, None, "relu"), ref)
    r = M.mlp_forward(x, w_in, None, w_out, None, w_hid, None, "relu", round_to=torch.bfloat16)
    assert torch.equal(r, r.bfloat16().float())
    torch.testing.assert_close(r, ref, rtol=3e-2, atol=3e-2)


# ----------------------------------------------------------------------------- reversible
def _rev_params(blocks, H, bias=True, seed=0, dtype=torch.double):
    g = torch.Generator().manual_seed(seed)
    w1 = (torch.rand(blocks * 2 * H, H, generator=g, dtype=dtype) * 2 - 1) / H**0.5
    w2 = (torch.rand(blocks * 2 * H, H, generator=g, dtype=dtype) * 2 - 1) / H**0.5
    b1 = (torch.rand(blocks * 2, H, generator=g, dtype=dtype) * 2 - 1) / H**0.5 if bias else None
    b2 = (torch.rand(blocks * 2, H, generator=g, dtype=dtype) * 2 - 1) / H**0.5 if bias else None
    return w1, b1, w2, b2


def _plain_composition(x, w1, b1, w2, b2, act):
    """Independent restatement with explicit nn.functional calls and slicing per block."""
    H = x.shape[-1] // 2
    fn = {"gelu": torch.nn.functional.gelu, "relu": torch.relu, "silu": torch.nn.functional.silu, "none": lambda t: t}[act]
    a, b = x[:, :H], x[:, H:]
    for k in range(w1.shape[0] // (2 * H)):
        wf1, wf2 = w1[2 * k * H : (2 * k + 1) * H], w2[2 * k * H : (2 * k + 1) * H]
        wg1, wg2 = w1[(2 * k + 1) * H : (2 * k + 2) * H], w2[(2 * k + 1) * H : (2 * k + 2) * H]
        bf1 = 0 if b1 is None else b1[2 * k]
        bf2 = 0 if b2 is None else b2[2 * k]
        bg1 = 0 if b1 is None else b1[2 * k + 1]
        bg2 = 0 if b2 is None else b2[2 * k + 1]
        a = a + fn(b @ wf1.t() + bf1) @ wf2.t() + bf2
        b = b + fn(a @ wg1.t() + bg1) @ wg2.t() + bg2
    return torch.cat([a, b], 1)


@pytest.mark.parametrize("act", ["gelu", "relu", "silu"])
@pytest.mark.parametrize("bias", [True, False])
def test_reversible_forward_inverse_and_grads(act, bias):
    torch.manual_seed(0)
    H, blocks = 8, 3
    w1, b1, w2, b2 = _rev_params(blocks, H, bias, dtype=torch.float32)
    x = torch.randn(7, 2 * H)
    y = R.rev_forward(x, w1, b1, w2, b2, act)
    torch.testing.assert_close(y, _plain_composition(x, w1, b1, w2, b2, act), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(R.rev_inverse(y, w1, b1, w2, b2, act), x, rtol=1e-4, atol=1e-5)
    dy = torch.randn_like(y)
    g = R.rev_backward(x, dy, w1, b1, w2, b2, act)
    leaves = [t.clone().requires_grad_(True) if t is not None else None for t in (x, w1, b1, w2, b2)]
    _plain_composition(*leaves, act).backward(dy)
    for name, leaf in zip(("dx", "dw1", "db1", "dw2", "db2"), leaves):
        if leaf is None:
            assert g[name] is None
        else:
            torch.testing.assert_close(g[name], leaf.grad, rtol=1e-4, atol=1e-5)


def test_reversible_finite_difference():
    torch.manual_seed(0)
    H, blocks = 4, 2
    w1, b1, w2, b2 = _rev_params(blocks, H, True)
    x = torch.randn(3, 2 * H, dtype=torch.double)
    dy = torch.randn(3, 2 * H, dtype=torch.double)

    def loss(w1_):
        return (_plain_composition(x, w1_, b1, w2, b2, "gelu") * dy).sum()

    g = R.rev_backward(x.float(), dy.float(), w1.float(), b1.float(), w2.float(), b2.float(), "gelu")
    eps = 1e-6
    for idx in [(0, 0), (5, 2), (13, 3)]:
        wp, wm = w1.clone(), w1.clone()
        wp[idx] += eps
        wm[idx] -= eps
        fd = (loss(wp) - loss(wm)) / (2 * eps)
        assert abs(fd.item() - g["dw1"][idx].item()) < 1e-3 * max(1.0, abs(fd.item()))


# ----------------------------------------------------------------------------- the 16-bit (``round_to=``) mode
# ``round_to`` is the mode every 16-bit GPU comparison uses, so it is pinned on its own, four ways:
#   (1) against a chain of ``nn.Linear`` modules whose parameters and activations ARE bfloat16 / float16 tensors under
#       CPU autograd (a library routine; what the reference's half-precision tests run on the GPU,
#       tests/test_layers/test_fully_fused_mlp.py:72-107, 292-369);
#   (2) against a hand-written float64 back-propagation through the rounded activations (no autograd, no ste_round);
#   (3) on integer-valued inputs where nothing rounds: the mode must then be invisible, forward and backward;
#   (4) on a known answer where one rounding happens at a known place.
EPS = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("act", ["relu", "silu", "none"])
@pytest.mark.parametrize("depth", [1, 2, 3])
def test_round_to_matches_a_16bit_linear_chain(depth, act, dtype):
    torch.manual_seed(0)
    d_in, H, d_out, rows = 32, 64, 16, 4096
    net = RefMLP(d_in, H, d_out, depth, ACTS[act]).to(dtype)
    x = torch.randn(rows, d_in).to(dtype).requires_grad_(True)
    y = net(x)
    dy = torch.randn(rows, d_out).to(dtype)
    y.backward(dy)
    w_hid, b_hid = _stack(net)
    d = lambda t: None if t is None else t.detach()  # noqa: E731
    args = (d(net.first.weight), d(net.first.bias), d(net.last.weight), d(net.last.bias), d(w_hid), d(b_hid), act)
    got = M.mlp_forward(x.detach(), *args, round_to=dtype)
    want = y.detach().float()
    assert torch.equal(got, got.to(dtype).float()), "the result must be representable in the storage dtype"
    # forward: the chain rounds each layer's float32-accumulated result once, exactly where round_to does; only the
    # order of the float32 additions differs, so all but a few results agree bit for bit.  SiLU rounds twice in the
    # chain (pre-activation, then activation) and once here and in the kernels (reference kernel.py:34-47).
    if act != "silu":
        assert float((got == want).float().mean()) >= 0.999
    assert float((got - want).abs().max()) <= 4 * EPS[dtype] * float(want.abs().max())
    # backward: the chain also rounds every gradient it hands down to 16 bit; the oracle keeps them float32
    g = M.mlp_backward(x.detach(), dy, *args, round_to=dtype)
    bound = 4 * EPS[dtype]  # of the tensor's largest magnitude
    pairs = [("dx", x.grad), ("dw_in", net.first.weight.grad), ("db_in", net.first.bias.grad),
             ("dw_out", net.last.weight.grad), ("db_out", net.last.bias.grad)]
    if depth > 1:
        pairs += [("dw_hid", torch.cat([l.weight.grad for l in net.mid], 0)), ("db_hid", torch.stack([l.bias.grad for l in net.mid], 0))]
    for name, ref in pairs:
        ref = ref.float()
        assert float((g[name] - ref).abs().max()) <= bound * float(ref.abs().max()), name
    # and no element of dx is outside the tolerance the GPU tests use
    ref = x.grad.float()
    assert not bool(((g["dx"] - ref).abs() > 1e-2 + 2e-2 * ref.abs()).any())


def _round16(t, dtype):
    return t.to(torch.float32).to(dtype).to(torch.float64)


def _manual_backprop(x, dy, ws, bs, act, dtype):
    """float64 forward over 16-bit-rounded activations and the textbook backward, written out layer by layer:
    z_k = h_{k-1} W_k^T + b_k,  h_k = round(act(z_k));  dz_k = dh_k * act'(z_k),  dW_k = dz_k^T h_{k-1},  dh_{k-1} = dz_k W_k."""
    f = {"relu": lambda z: z.clamp_min(0), "silu": lambda z: z * torch.sigmoid(z), "none": lambda z: z}[act]
    df = {"relu": lambda z: (z > 0).to(z.dtype), "silu": lambda z: torch.sigmoid(z) * (1 + z * (1 - torch.sigmoid(z))), "none": torch.ones_like}[act]
    hs, zs = [x.double()], []
    for k, (w, b) in enumerate(zip(ws, bs)):
        z = hs[-1] @ w.double().t() + b.double()
        zs.append(z)
        hs.append(_round16(f(z) if k < len(ws) - 1 else z, dtype))
    dh = dy.double()
    dws, dbs = [None] * len(ws), [None] * len(ws)
    for k in reversed(range(len(ws))):
        dz = dh if k == len(ws) - 1 else dh * df(zs[k])
        dws[k], dbs[k] = dz.t() @ hs[k], dz.sum(0)
        dh = dz @ ws[k].double()
    return hs[-1], dh, dws, dbs


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("act", ["relu", "silu", "none"])
def test_round_to_equals_manual_backprop_through_rounded_activations(act, dtype):
    torch.manual_seed(2)
    d_in, H, d_out, rows, depth = 8, 16, 4, 64, 3
    ws = [(torch.randn(H, d_in) / d_in**0.5).to(dtype)] + [(torch.randn(H, H) / H**0.5).to(dtype) for _ in range(depth - 1)] + [(torch.randn(d_out, H) / H**0.5).to(dtype)]
    bs = [(torch.randn(w.shape[0]) / 4).to(dtype) for w in ws]
    x = torch.randn(rows, d_in).to(dtype)
    dy = torch.randn(rows, d_out).to(dtype)
    y, dx, dws, dbs = _manual_backprop(x, dy, ws, bs, act, dtype)
    args = (ws[0], bs[0], ws[-1], bs[-1], torch.cat(ws[1:-1], 0), torch.stack(bs[1:-1], 0), act)
    got = M.mlp_forward(x, *args, round_to=dtype)
    # float32 against float64 sums: a result within float32 rounding of a 16-bit tie may land on the other neighbour
    assert float((got.double() == y).float().mean()) >= 0.995
    torch.testing.assert_close(got.double(), y, rtol=2 * EPS[dtype], atol=1e-6)
    g = M.mlp_backward(x, dy, *args, round_to=dtype)
    # gradients differ only where such a tie moved an activation, and by float32 rounding: bound relative to each tensor's scale
    def close(a, b, what):
        assert float((a.double() - b).abs().max()) <= 2 * EPS[dtype] * float(b.abs().max()), what
    close(g["dx"], dx, "dx")
    close(g["dw_in"], dws[0], "dw_in")
    close(g["db_in"], dbs[0], "db_in")
    close(g["dw_hid"], torch.cat(dws[1:-1], 0), "dw_hid")
    close(g["db_hid"], torch.stack(dbs[1:-1], 0), "db_hid")
    close(g["dw_out"], dws[-1], "dw_out")
    close(g["db_out"], dbs[-1], "db_out")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_round_to_is_invisible_when_nothing_rounds(dtype):
    """Small integer inputs and weights: every activation is an integer below 256, exact in both 16-bit types, so the
    rounding mode must give the plain float32 results bit for bit -- forward and all gradients (a straight-through
    rounding that scaled, dropped or doubled the gradient would show here)."""
    g = torch.Generator().manual_seed(4)
    ri = lambda *s: torch.randint(-1, 2, s, generator=g).float()  # noqa: E731
    x, dy = ri(50, 8), ri(50, 4)
    w_in, w_hid, w_out = ri(8, 8), ri(16, 8), ri(4, 8)
    b_in, b_hid, b_out = ri(8), ri(2, 8), ri(4)
    for act in ("relu", "none"):
        plain = M.mlp_forward(x, w_in, b_in, w_out, b_out, w_hid, b_hid, act)
        assert float(plain.abs().max()) < 256 and torch.equal(plain, plain.round())
        assert torch.equal(M.mlp_forward(x, w_in, b_in, w_out, b_out, w_hid, b_hid, act, round_to=dtype), plain)
        a = M.mlp_backward(x, dy, w_in, b_in, w_out, b_out, w_hid, b_hid, act)
        b = M.mlp_backward(x, dy, w_in, b_in, w_out, b_out, w_hid, b_hid, act, round_to=dtype)
        for k in a:
            assert torch.equal(a[k], b[k]), k


def test_round_to_known_answer():
    """One unit per layer, bfloat16: x = w_in = 1 + 2^-7 gives z = 1 + 2^-6 + 2^-14, stored as 1 + 2^-6; the second
    layer (weight 3) therefore returns 3 + 3 * 2^-6 exactly, where the float32 chain returns 3 + 3 * 2^-6 + 3 * 2^-14.
    The straight-through gradients are those of the float32 chain evaluated at the stored activation:
    dx = w_in * w_out, dw_in = x * w_out, dw_out = stored activation."""
    a = 1 + 2.0**-7
    x, w_in, w_out, dy = (torch.tensor([[v]]) for v in (a, a, 3.0, 1.0))
    y32 = M.mlp_forward(x, w_in, None, w_out, None, None, None, "relu")
    y16 = M.mlp_forward(x, w_in, None, w_out, None, None, None, "relu", round_to=torch.bfloat16)
    assert y32.item() == 3 * (1 + 2.0**-6 + 2.0**-14)
    assert y16.item() == 3 * (1 + 2.0**-6)
    g = M.mlp_backward(x, dy, w_in, None, w_out, None, None, None, "relu", round_to=torch.bfloat16)
    assert g["dx"].item() == a * 3 and g["dw_in"].item() == a * 3 and g["dw_out"].item() == 1 + 2.0**-6
    # a negative pre-activation closes the ReLU gate in both modes
    g = M.mlp_backward(-x, dy, w_in, None, w_out, None, None, None, "relu", round_to=torch.bfloat16)
    assert g["dx"].item() == 0 and g["dw_in"].item() == 0 and g["dw_out"].item() == 0


# ----------------------------------------------------------------------------- reversible, 16-bit mode
class _RoundSTE(torch.autograd.Function):
    """Rounding with an identity backward, as an explicit autograd Function (the oracle uses a detach expression)."""

    @staticmethod
    def forward(ctx, t, dtype):
        return t.to(dtype).to(torch.float32)

    @staticmethod
    def backward(ctx, g):
        return g, None


def _plain_composition_rounded(x, w1, b1, w2, b2, act, dtype, every):
    """The plain composition with the 16-bit rounding points written out: every matmul operand (the input of a
    sub-network and its hidden activation) is rounded; the two residual streams themselves stay float32 and are
    rounded after every ``every``-th coupling (0: never)."""
    H = x.shape[-1] // 2
    r = lambda t: _RoundSTE.apply(t, dtype)  # noqa: E731
    fn = {"gelu": torch.nn.functional.gelu, "relu": torch.relu, "silu": torch.nn.functional.silu, "none": lambda t: t}[act]
    a, b = x[:, :H].float(), x[:, H:].float()
    for k in range(w1.shape[0] // (2 * H)):
        def sub(u, i):
            bb1 = 0 if b1 is None else b1[i].float()
            bb2 = 0 if b2 is None else b2[i].float()
            t = r(fn(r(u) @ w1[i * H : (i + 1) * H].float().t() + bb1))
            return t @ w2[i * H : (i + 1) * H].float().t() + bb2
        a = a + sub(b, 2 * k)
        b = b + sub(a, 2 * k + 1)
        if every and (k + 1) % every == 0:
            a, b = r(a), r(b)
    return torch.cat([a, b], 1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("act", ["gelu", "relu", "none"])
@pytest.mark.parametrize("every", [0, 1, 2, 4])
def test_reversible_round_to_vs_written_out_rounding_points(every, act, dtype):
    torch.manual_seed(1)
    H, blocks = 16, 4
    w1, b1, w2, b2 = (t.to(dtype) for t in _rev_params(blocks, H, True, dtype=torch.float32))
    x = torch.randn(40, 2 * H).to(dtype)
    dy = torch.randn(40, 2 * H).to(dtype)
    got = R.rev_forward(x, w1, b1, w2, b2, act, round_to=dtype, stream_round_every=every)
    leaves = [t.clone().float().requires_grad_(True) for t in (x, w1, b1, w2, b2)]
    want = _plain_composition_rounded(*leaves, act, dtype, every)
    assert torch.equal(got, want.detach())
    if every == 1:  # rev_backward differentiates the default rounding schedule
        want.backward(dy.float())
        g = R.rev_backward(x, dy, w1, b1, w2, b2, act, round_to=dtype)
        for name, leaf in zip(("dx", "dw1", "db1", "dw2", "db2"), leaves):
            torch.testing.assert_close(g[name], leaf.grad, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_reversible_round_to_vs_16bit_module_chain(dtype):
    """Couplings built from ``nn.Linear`` modules holding 16-bit parameters, run on 16-bit tensors under CPU autograd
    (each matmul result, activation and residual sum rounded by the library), against ``round_to`` with the stream
    rounded after every coupling."""
    torch.manual_seed(3)
    H, blocks, rows = 64, 4, 2048
    w1, b1, w2, b2 = (t.to(dtype) for t in _rev_params(blocks, H, True, dtype=torch.float32))
    x = torch.randn(rows, 2 * H).to(dtype).requires_grad_(True)
    subs = []
    for i in range(2 * blocks):
        l1, l2 = nn.Linear(H, H).to(dtype), nn.Linear(H, H).to(dtype)
        with torch.no_grad():
            l1.weight.copy_(w1[i * H : (i + 1) * H]); l1.bias.copy_(b1[i])
            l2.weight.copy_(w2[i * H : (i + 1) * H]); l2.bias.copy_(b2[i])
        subs.append(nn.Sequential(l1, nn.GELU(), l2))
    a, b = x[:, :H], x[:, H:]
    for k in range(blocks):
        a = a + subs[2 * k](b)
        b = b + subs[2 * k + 1](a)
    y = torch.cat([a, b], 1)
    dy = torch.randn(rows, 2 * H).to(dtype)
    y.backward(dy)
    got = R.rev_forward(x.detach(), w1, b1, w2, b2, "gelu", round_to=dtype, stream_round_every=1)
    want = y.detach().float()
    # the module chain rounds three more times per coupling half (pre-activation, sub-network output, sum)
    assert float((got - want).abs().max()) <= 8 * EPS[dtype] * float(want.abs().max())
    assert float((got - want).abs().mean()) <= EPS[dtype] * float(want.abs().mean())
    g = R.rev_backward(x.detach(), dy, w1, b1, w2, b2, "gelu", round_to=dtype)
    ref = x.grad.float()
    assert float((g["dx"] - ref).abs().max()) <= 8 * EPS[dtype] * float(ref.abs().max())
    gw = torch.cat([s[0].weight.grad for s in subs], 0).float()
    assert float((g["dw1"] - gw).abs().max()) <= 8 * EPS[dtype] * float(gw.abs().max())
    gw = torch.cat([s[2].weight.grad for s in subs], 0).float()
    assert float((g["dw2"] - gw).abs().max()) <= 8 * EPS[dtype] * float(gw.abs().max())


def test_reversible_round_to_is_invisible_when_nothing_rounds():
    g = torch.Generator().manual_seed(6)
    ri = lambda *s: torch.randint(-1, 2, s, generator=g).float()  # noqa: E731
    H, blocks = 4, 2
    x, dy = ri(30, 2 * H), ri(30, 2 * H)
    w1, w2, b1, b2 = ri(blocks * 2 * H, H), ri(blocks * 2 * H, H), ri(blocks * 2, H), ri(blocks * 2, H)
    plain = R.rev_forward(x, w1, b1, w2, b2, "relu")
    assert float(plain.abs().max()) < 256
    for every in (0, 1, 2):
        assert torch.equal(R.rev_forward(x, w1, b1, w2, b2, "relu", round_to=torch.bfloat16, stream_round_every=every), plain)
    a = R.rev_backward(x, dy, w1, b1, w2, b2, "relu")
    b = R.rev_backward(x, dy, w1, b1, w2, b2, "relu", round_to=torch.bfloat16)
    for k in a:
        assert torch.equal(a[k], b[k]), k


def test_reversible_round_to_known_answer():
    """Half width 1, identity activation, one coupling, bfloat16.  x = (0, a) with a = 1 + 2^-7, F = (w1 = 1, w2 = a),
    G = (w1 = 1, w2 = 1):  y1 = a * a = 1 + 2^-6 + 2^-14 stays float32 in the stream, but G multiplies its 16-bit image
    1 + 2^-6, so y2 = a + 1 + 2^-6 = 2 * (1 + 2^-7 + 2^-8).  Rounding the stream after the coupling stores y1 as
    1 + 2^-6 and y2, a tie between two 8-bit significands, as the even one: 2 * (1 + 2^-6)."""
    a = 1 + 2.0**-7
    x = torch.tensor([[0.0, a]])
    w1 = torch.tensor([[1.0], [1.0]])
    w2 = torch.tensor([[a], [1.0]])
    y = R.rev_forward(x, w1, None, w2, None, "none", round_to=torch.bfloat16, stream_round_every=0)
    assert y[0, 0].item() == 1 + 2.0**-6 + 2.0**-14 and y[0, 1].item() == a + 1 + 2.0**-6
    y = R.rev_forward(x, w1, None, w2, None, "none", round_to=torch.bfloat16, stream_round_every=1)
    assert y[0, 0].item() == 1 + 2.0**-6 and y[0, 1].item() == 2 * (1 + 2.0**-6)
    y = R.rev_forward(x, w1, None, w2, None, "none")
    assert y[0, 1].item() == torch.tensor(a + 1 + 2.0**-6 + 2.0**-14).item()
