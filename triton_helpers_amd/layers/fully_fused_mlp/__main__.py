"""``python -m triton_helpers.layers.fully_fused_mlp benchmark|profile ...`` (reference fully_fused_mlp/__main__.py:12-92).

Dimensions as in the reference: ``x (32, L, D)``, every layer ``D`` wide, ``H`` hidden-to-hidden layers.  Providers: a
chain of ``F.linear`` + ReLU calls (``baseline``) and the fused kernels (``fully-fused``).
"""
import torch
import torch.nn.functional as F

from ...benchmark import Workload, run_cli
from .kernel import fully_fused_mlp


def _inputs(L, D, H, device="cuda", dtype=torch.float32, requires_grad=False):
    def leaf(*shape, scale=1.0):
        return (torch.randn(shape, device=device) * scale).to(dtype).requires_grad_(requires_grad)

    s = D**-0.5
    return {
        "x": leaf(32, L, D), "w_in": leaf(D, D, scale=s), "b_in": leaf(D, scale=s), "w_out": leaf(D, D, scale=s), "b_out": leaf(D, scale=s),
        "w_hid": leaf(D * H, D, scale=s) if H >= 1 else None, "b_hid": leaf(H, D, scale=s) if H >= 1 else None,
    }


def _linear_chain(x, w_in, b_in, w_out, b_out, w_hid, b_hid):
    D = w_in.shape[0]
    h = F.relu(F.linear(x, w_in, b_in))
    for k in range(0 if w_hid is None else w_hid.shape[0] // D):
        h = F.relu(F.linear(h, w_hid[D * k : D * (k + 1)], b_hid[k]))
    return F.linear(h, w_out, b_out)


def _fused(x, w_in, b_in, w_out, b_out, w_hid, b_hid):
    return fully_fused_mlp(x, w_in, b_in, w_out, b_out, w_hid, b_hid)


def main(argv=None):
    return run_cli(
        "MLP",
        [Workload("baseline", _inputs, _linear_chain), Workload("fully-fused", _inputs, _fused)],
        dims={
            "L": ((512, 2048, 8192, 16384, 32768, 65536), "values"),
            "D": (64, "values"),
            "H": (8, "values"),
        },
        argv=argv,
    )


if __name__ == "__main__":
    main()
