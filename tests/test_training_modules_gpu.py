"""The modules as a user of the reference trains them: HashEncoding -> FullyFusedMLP under autocast with torch.optim.Adam
(reference modules: hash_encoding/module.py:8-39, fully_fused_mlp/module.py:9-53).  A small field is fitted and the loss
must fall; nothing here compares with the oracle (the parity tests do), it checks that the pieces compose: float32
parameters, autocast to 16 bit, gradients back in float32, state-dict round trip."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _field(x):
    return torch.stack([torch.sin(6.0 * x[:, 0]) * torch.cos(4.0 * x[:, 1]), x[:, 2] ** 2, torch.sin(9.0 * x.sum(1)), x[:, 0] * x[:, 1]], dim=1)


@pytest.mark.parametrize("amp_dtype", [torch.float16, torch.bfloat16])
def test_fit_a_small_field(amp_dtype):
    from triton_helpers.layers.fully_fused_mlp import FullyFusedMLP
    from triton_helpers.layers.hash_encoding import HashEncoding

    torch.manual_seed(0)
    enc = HashEncoding(2**12, 8, 3, 2, 8, 128).to(DEV)
    with torch.no_grad():
        enc.embeddings.uniform_(-1e-2, 1e-2)
    mlp = FullyFusedMLP(16, 64, 4, 2).to(DEV)
    opt = torch.optim.Adam(list(enc.parameters()) + list(mlp.parameters()), lr=1e-2)
    scaler = torch.amp.GradScaler("cuda", enabled=amp_dtype == torch.float16)
    losses = []
    for step in range(150):
        x = torch.rand(4096, 3, device=DEV)
        y = _field(x)
        with torch.autocast("cuda", dtype=amp_dtype):
            h = enc(x)
            out = mlp(h.view(1, -1, 16)).view(-1, 4)
        loss = torch.nn.functional.mse_loss(out.float(), y)
        opt.zero_grad(set_to_none=True)
        scaler.scale(loss).backward()
        assert enc.embeddings.grad.dtype == torch.float32 and mlp.w_in.grad.dtype == torch.float32
        scaler.step(opt)
        scaler.update()
        losses.append(float(loss.detach()))
    first, last = sum(losses[:10]) / 10, sum(losses[-10:]) / 10
    assert last < 0.35 * first, f"loss went from {first:.4f} to {last:.4f}"
    # a state-dict round trip gives the same outputs
    enc2 = HashEncoding(2**12, 8, 3, 2, 8, 128).to(DEV)
    mlp2 = FullyFusedMLP(16, 64, 4, 2).to(DEV)
    enc2.load_state_dict(enc.state_dict())
    mlp2.load_state_dict(mlp.state_dict())
    x = torch.rand(1000, 3, device=DEV)
    with torch.no_grad(), torch.autocast("cuda", dtype=amp_dtype):
        a = mlp(enc(x).view(1, -1, 16))
        b = mlp2(enc2(x).view(1, -1, 16))
    assert torch.equal(a, b)
