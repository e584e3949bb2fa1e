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
