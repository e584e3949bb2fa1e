"""``python -m triton_helpers.layers.fully_fused_mlp benchmark|profile ...`` (reference fully_fused_mlp/__main__.py:12-92).

Dimensions as in the reference: ``x (32, L, D)``, every layer ``D`` wide, ``H`` hidden-to-hidden layers.  Providers: a
chain of ``F.linear`` + ReLU calls (``baseline``) and the fused kernels (``fully-fused``).
"""
from dataclasses import dataclass
from typing import Dict, Optional

import torch
import torch.nn.functional as F
from torch import Tensor

from ...benchmark import CLI, KernelExecutor
from .kernel import fully_fused_mlp


@dataclass
class Baseline(KernelExecutor):
    def prepare_inputs(self, L: int, D: int, H: int, **kwargs) -> Dict[str, Optional[Tensor]]:
        device, dtype, grad = kwargs.get("device", "cuda"), kwargs.get("dtype", torch.float32), kwargs.get("requires_grad", False)
        mk = lambda *shape: (self.randn(shape, device=device) / D**0.5).to(dtype).requires_grad_(grad)  # noqa: E731
        x = self.randn((32, L, D), device=device).to(dtype).requires_grad_(grad)
        return {
            "x": x, "w_in": mk(D, D), "b_in": mk(D), "w_out": mk(D, D), "b_out": mk(D),
            "w_hid": mk(D * H, D) if H >= 1 else None, "b_hid": mk(H, D) if H >= 1 else None, "H": H,
        }

    def forward(self, x, w_in, b_in, w_out, b_out, w_hid, b_hid, H) -> Tensor:
        x = F.relu(F.linear(x, w_in, b_in))
        D = w_in.shape[0]
        for i in range(H):
            x = F.relu(F.linear(x, w_hid[D * i : D * (i + 1)], b_hid[i]))
        return F.linear(x, w_out, b_out)


@dataclass
class Native(Baseline):
    def forward(self, x, w_in, b_in, w_out, b_out, w_hid, b_hid, H) -> Tensor:
        return fully_fused_mlp(x, w_in, b_in, w_out, b_out, w_hid, b_hid)


def main(argv=None):
    return CLI.entrypoint(
        "MLP",
        [Baseline("baseline"), Native("fully-fused")],
        dims={
            "L": ((512, 2048, 8192, 16384, 32768, 65536), "values"),
            "D": (64, "values"),
            "H": (8, "values"),
        },
        argv=argv,
    )


if __name__ == "__main__":
    main()
