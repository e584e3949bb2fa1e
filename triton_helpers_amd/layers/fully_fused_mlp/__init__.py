from .kernel import feedforward, feedforward_bwd_dw, feedforward_bwd_dx, feedforward_bwd_dz, fully_fused_mlp
from .module import FullyFusedMLP

__all__ = [
    "fully_fused_mlp",
    "feedforward",
    "feedforward_bwd_dw",
    "feedforward_bwd_dx",
    "feedforward_bwd_dz",
    "FullyFusedMLP",
]
