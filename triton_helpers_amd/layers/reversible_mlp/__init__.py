from .kernel import reversible_mlp, reversible_mlp_inverse
from .module import ReversibleMLP

__all__ = ["reversible_mlp", "reversible_mlp_inverse", "ReversibleMLP"]
