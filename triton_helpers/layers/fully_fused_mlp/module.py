"""Alias of ``triton_helpers_amd.layers.fully_fused_mlp.module``."""
from triton_helpers_amd.layers.fully_fused_mlp.module import FullyFusedMLP  # noqa: F401
