"""``python -m triton_helpers.layers.hash_encoding benchmark|profile ...`` (reference hash_encoding/__main__.py:20-90).

Dimensions as in the reference: a batch of ``(32, L, D)`` points, ``F`` features per row, ``T`` rows per level, ``N``
levels with resolutions ``X .. Y``.  The provider is this package's kernel; the reference's comparison provider
(tiny-cuda-nn) does not exist for this GPU.
"""
from dataclasses import dataclass
from typing import Any, Dict

import torch
from torch import Tensor

from ...benchmark import CLI, KernelExecutor
from .kernel import hash_encoding
from .module import HashEncoding


@dataclass
class Native(KernelExecutor):
    @torch.no_grad()
    def prepare_inputs(self, L: int, D: int, F: int, T: int, N: int, X: int, Y: int, **kwargs) -> Dict[str, Any]:
        device = kwargs.get("device", "cuda")
        torch.random.manual_seed(0)
        x = self.rand((32, L, D), device=device)
        layer = HashEncoding(T, N, D, F, X, Y).to(device)
        e = layer.embeddings.detach().to(kwargs.get("dtype", torch.float32))
        e.requires_grad = kwargs.get("requires_grad", False)
        return {"x": x, "e": e, "pi": layer.pi.detach(), "geometry": (T, X, Y, N)}

    def forward(self, x: Tensor, e: Tensor, pi: Tensor, geometry) -> Tensor:
        T, X, Y, N = geometry
        return hash_encoding(x, e, None, pi, T, X, Y, N)


def main(argv=None):
    return CLI.entrypoint(
        "InstantNGP Hash Encoding",
        [Native("hip-hash")],
        dims={
            "L": ((512, 2048, 8192, 16384, 32768, 65536, 65536 * 2), "values"),
            "D": (3, "values"),
            "F": (2, "values"),
            "T": (2**14, "values"),
            "N": (16, "values"),
            "X": (16, "values"),
            "Y": (512, "values"),
        },
        argv=argv,
    )


if __name__ == "__main__":
    main()
