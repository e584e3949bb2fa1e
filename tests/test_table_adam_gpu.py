"""GPU: the fused table optimiser step against ``torch.optim.Adam`` on the CPU (the reference has no optimiser; the
checker is the library routine whose arithmetic the kernel states)."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("dtype,master", [(torch.float32, False), (torch.float16, True), (torch.bfloat16, True), (torch.float16, False)])
@pytest.mark.parametrize("weight_decay", [0.0, 1e-2])
def test_steps_match_torch_adam(dtype, master, weight_decay):
    from triton_helpers_amd.optim import TableAdam

    torch.manual_seed(0)
    n, scale = (100003, 2), 1024.0
    p0 = (torch.rand(n) * 2 - 1) * 1e-2
    ref = p0.to(dtype).float().clone().requires_grad_(True)
    opt = torch.optim.Adam([ref], lr=1e-3, betas=(0.9, 0.99), eps=1e-10, weight_decay=weight_decay)
    table = p0.to(dtype).to(DEV)
    mine = TableAdam(table, lr=1e-3, betas=(0.9, 0.99), eps=1e-10, weight_decay=weight_decay, master=master)
    grad = torch.zeros(n, dtype=torch.float32, device=DEV)
    for step in range(5):
        g = torch.randn(n) * (0.1 if step != 2 else 0.0)  # one step with an all-zero gradient
        grad += (g * scale).to(DEV)
        mine.step(grad, grad_scale=scale)
        assert not bool(grad.any()), "the step clears the gradient for the next backward"
        ref.grad = g.clone()
        opt.step()
        if not master and dtype != torch.float32:
            # without a master copy the parameter is re-read from its 16-bit storage every step, so the checker does the same
            with torch.no_grad():
                ref.copy_(ref.to(dtype).float())
        want = ref.detach()
        if master or dtype == torch.float32:
            params = mine.master if master else table
            torch.testing.assert_close(params.cpu().float(), want, rtol=1e-5, atol=1e-8)
        eps16 = {torch.float32: 1e-6, torch.float16: 2.0**-10, torch.bfloat16: 2.0**-7}[dtype]
        if master or dtype == torch.float32:
            torch.testing.assert_close(table.cpu().float(), want, rtol=eps16, atol=1e-7)
        else:  # a last-bit difference in one step is re-read from the 16-bit storage in the next: a few ulps over five steps
            torch.testing.assert_close(table.cpu().float(), want, rtol=4 * eps16, atol=4 * eps16 * 1e-2)
    state = opt.state[ref]
    # torch updates the first moment as m + (g - m) (1 - b1), the kernel as b1 m + (1 - b1) g: moments that nearly cancel
    # differ in their last float32 bits, hence the absolute terms (the moments are ~1e-2 and ~1e-3)
    torch.testing.assert_close(mine.exp_avg.cpu(), state["exp_avg"], rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(mine.exp_avg_sq.cpu(), state["exp_avg_sq"], rtol=1e-5, atol=1e-9)


def test_training_loop_keeps_one_gradient_buffer():
    """encode -> loss -> backward into a persistent float32 buffer -> fused step, three times: the table moves downhill and
    the buffer is clear after every step."""
    from oracle import hash_encoding as O
    from triton_helpers_amd.layers.hash_encoding import kernel as hk
    from triton_helpers_amd.optim import TableAdam

    T, L, lo, hi = 2**14, 16, 16, 512
    E = O.level_row_offsets(L, T, 3, lo, hi)[-1]
    torch.manual_seed(1)
    x = torch.rand(40000, 3, device=DEV)
    table = ((torch.rand(E, 2) * 2 - 1) * 1e-2).half().to(DEV)
    target = torch.rand(40000, 32, device=DEV) * 0.1
    opt = TableAdam(table, lr=1e-2)
    grad = torch.zeros(E, 2, dtype=torch.float32, device=DEV)
    losses = []
    for _ in range(3):
        out = hk.hash_encoding(x, table, None, None, T, lo, hi, L)
        diff = out.float() - target
        losses.append(float(diff.pow(2).mean()))
        do = (2 * diff / diff.numel() * 65536.0).half()
        hk.hash_encoding_table_grad(x, do, E, 2, None, T, lo, hi, L, out=grad)
        opt.step(grad, grad_scale=65536.0)
        assert not bool(grad.any())
    assert losses[2] < losses[1] < losses[0]


def test_nonfinite_gradient_elements_are_skipped_and_reported():
    """An inf and a NaN in the gradient (an overflowed loss-scaled step): those elements keep their parameter and moments,
    the others get the ordinary update, the flag is raised, and the gradient is cleared; without the skip the same
    elements turn non-finite (torch.optim.Adam's behaviour), and the flag is raised all the same."""
    from triton_helpers_amd.optim import TableAdam

    torch.manual_seed(3)
    n = (5000, 2)
    p0 = ((torch.rand(n) * 2 - 1) * 1e-2).half()
    g = torch.randn(n) * 0.1
    bad = g.clone()
    bad[17, 1] = float("inf")
    bad[4000, 0] = float("nan")
    clean_opt = TableAdam(p0.clone().to(DEV), lr=1e-3)
    clean_opt.step(g.to(DEV))
    assert int(clean_opt.found_nonfinite.item()) == 0
    opt = TableAdam(p0.clone().to(DEV), lr=1e-3)
    grad = bad.to(DEV)
    opt.step(grad)
    assert int(opt.found_nonfinite.item()) == 1
    assert not bool(grad.any())
    want = clean_opt.table.cpu().clone()
    want[17, 1] = p0[17, 1]
    want[4000, 0] = p0[4000, 0]
    assert torch.equal(opt.table.cpu(), want)
    assert float(opt.exp_avg[17, 1]) == 0.0 and float(opt.exp_avg_sq[4000, 0]) == 0.0
    assert torch.isfinite(opt.master).all() and torch.isfinite(opt.exp_avg).all() and torch.isfinite(opt.exp_avg_sq).all()
    # a later clean step clears the flag again
    opt.step(g.to(DEV))
    assert int(opt.found_nonfinite.item()) == 0
    raw = TableAdam(p0.clone().to(DEV), lr=1e-3)
    raw.step(bad.to(DEV), skip_nonfinite=False)
    assert int(raw.found_nonfinite.item()) == 1
    assert not torch.isfinite(raw.master[4000, 0]) and torch.isfinite(raw.master[0, 0])
