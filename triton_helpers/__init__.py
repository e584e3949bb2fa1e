"""Drop-in alias: ``triton_helpers.layers.*`` resolves to the MI355X implementation in ``triton_helpers_amd``.

Code written against the reference (``from triton_helpers.layers.hash_encoding import hash_encoding`` ...)
imports unchanged.  Only the three neural-field layers exist here.
"""
from triton_helpers_amd import TENSOR_CORE_K, __version__

__all__ = ["TENSOR_CORE_K", "__version__"]
