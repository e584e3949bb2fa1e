"""GPU: tensors whose rows overlap or are strided reach the kernels as proper rows.

``out.sum(0).backward(g)`` hands the backward an upstream gradient expanded over the batch (row stride 0); an expanded
input does the same in the forward.  The reference's strided Triton loads accept both; here the Python layer copies
such tensors into rows before the C ABI sees them.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def test_hash_encoding_backward_of_a_broadcast_gradient():
    from oracle import hash_encoding as O
    from triton_helpers_amd.layers.hash_encoding import hash_encoding

    T, L, lo, hi = 2**14, 16, 16, 512
    E = O.level_row_offsets(L, T, 3, lo, hi)[-1]
    torch.manual_seed(0)
    x = torch.rand(300, 3)
    table = torch.randn(E, 2)
    g = torch.randn(32)
    e = table.to(DEV).requires_grad_(True)
    out = hash_encoding(x.to(DEV), e, max_entries_per_level=T, min_res=lo, max_res=hi, levels=L)
    out.sum(0).backward(g.to(DEV))
    want = O.encode_backward(x, g.expand(300, 32), E, 2, None, T, L, lo, hi)
    torch.testing.assert_close(e.grad.cpu(), want, rtol=1e-3, atol=1e-4)


def test_fused_mlp_with_broadcast_gradient_and_input():
    from oracle import mlp as M
    from triton_helpers_amd.layers.fully_fused_mlp import fully_fused_mlp

    torch.manual_seed(1)
    dtype = torch.bfloat16
    u = lambda *s: ((torch.rand(*s) * 2 - 1) / s[-1] ** 0.5).to(dtype)  # noqa: E731
    w_in, w_hid, w_out = u(64, 32), u(64, 64), u(16, 64)
    x = torch.randn(1, 200, 32).to(dtype)
    g = torch.randn(16).to(dtype)
    leaves = [t.to(DEV).requires_grad_(True) for t in (w_in, w_out, w_hid)]
    xd = x.to(DEV).requires_grad_(True)
    y = fully_fused_mlp(xd, leaves[0], None, leaves[1], None, leaves[2], None, "relu")
    y.sum((0, 1)).backward(g.to(DEV))
    want = M.mlp_backward(x.view(-1, 32), g.expand(200, 16), w_in, None, w_out, None, w_hid, None, "relu", round_to=dtype)
    torch.testing.assert_close(xd.grad.view(-1, 32).cpu().float(), want["dx"], rtol=2e-2, atol=1e-2)
    for name, leaf in zip(("dw_in", "dw_out", "dw_hid"), leaves):
        ref = want[name]
        torch.testing.assert_close(leaf.grad.cpu().float(), ref, rtol=2e-2, atol=2e-2 * float(ref.abs().max()))
    # an input expanded over the batch (every row the same vector)
    row = torch.randn(32).to(dtype)
    xe = row.to(DEV).expand(1, 50, 32)
    ye = fully_fused_mlp(xe, leaves[0].detach(), None, leaves[1].detach(), None, leaves[2].detach(), None, "relu")
    want_y = M.mlp_forward(row.expand(50, 32), w_in, None, w_out, None, w_hid, None, "relu", round_to=dtype)
    torch.testing.assert_close(ye.view(-1, 16).cpu().float(), want_y, rtol=2e-2, atol=1e-2)


def test_reversible_mlp_with_broadcast_gradient():
    from oracle import reversible as R
    from triton_helpers_amd.layers.reversible_mlp import reversible_mlp

    torch.manual_seed(2)
    dtype = torch.bfloat16
    H, blocks, rows = 64, 2, 96
    u = lambda *s: ((torch.rand(*s) * 2 - 1) / H**0.5).to(dtype)  # noqa: E731
    w1, w2 = u(blocks * 2 * H, H), u(blocks * 2 * H, H)
    x = torch.randn(rows, 2 * H).to(dtype)
    g = torch.randn(2 * H).to(dtype)
    xd = x.to(DEV).requires_grad_(True)
    y = reversible_mlp(xd, w1.to(DEV), None, w2.to(DEV), None, "gelu")
    y.sum(0).backward(g.to(DEV))
    want = R.rev_backward(x, g.expand(rows, 2 * H), w1, None, w2, None, "gelu", round_to=dtype)
    torch.testing.assert_close(xd.grad.cpu().float(), want["dx"], rtol=2e-2, atol=2e-2)
