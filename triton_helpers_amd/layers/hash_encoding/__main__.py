"""``python -m triton_helpers.layers.hash_encoding benchmark|profile ...`` (reference hash_encoding/__main__.py:20-90).

Dimensions as in the reference: a batch of ``(32, L, D)`` points, ``F`` features per row, ``T`` rows per level, ``N``
levels with resolutions ``X .. Y``.  The provider is this package's kernel; the reference's comparison provider
(tiny-cuda-nn) does not exist for this GPU.
"""
import torch

from ...benchmark import Workload, run_cli
from .kernel import hash_encoding
from .module import HashEncoding


@torch.no_grad()
def _inputs(L, D, F, T, N, X, Y, device="cuda", dtype=torch.float32, requires_grad=False):
    torch.random.manual_seed(0)
    layer = HashEncoding(T, N, D, F, X, Y).to(device)
    table = layer.embeddings.detach().to(dtype)
    table.requires_grad = requires_grad
    return {"x": torch.rand((32, L, D), device=device), "table": table, "pi": layer.pi.detach(), "geometry": (T, X, Y, N)}


def _encode(x, table, pi, geometry):
    T, X, Y, N = geometry
    return hash_encoding(x, table, None, pi, T, X, Y, N)


def main(argv=None):
    return run_cli(
        "InstantNGP Hash Encoding",
        [Workload("hip-hash", _inputs, _encode)],
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
