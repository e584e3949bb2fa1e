from triton_helpers_amd.layers.reversible_mlp import ReversibleMLP, reversible_mlp, reversible_mlp_inverse  # noqa: F401

__all__ = ["reversible_mlp", "reversible_mlp_inverse", "ReversibleMLP"]
