"""Alias of ``triton_helpers_amd.layers.fully_fused_mlp.kernel`` with the names code written against the reference imports."""
from triton_helpers_amd.layers.fully_fused_mlp.kernel import (  # noqa: F401
    FULLY_FUSED_MAX_DIM, _fully_fused_mlp, feedforward, feedforward_bwd_dw, feedforward_bwd_dx, feedforward_bwd_dz,
    fully_fused_mlp, get_float32_operands, set_float32_operands,
)
