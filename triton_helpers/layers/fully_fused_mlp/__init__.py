from triton_helpers_amd.layers.fully_fused_mlp import (  # noqa: F401
    FullyFusedMLP,
    feedforward,
    feedforward_bwd_dw,
    feedforward_bwd_dx,
    feedforward_bwd_dz,
    fully_fused_mlp,
)

__all__ = ["fully_fused_mlp", "feedforward", "feedforward_bwd_dw", "feedforward_bwd_dx", "feedforward_bwd_dz", "FullyFusedMLP"]
