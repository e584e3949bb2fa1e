"""MI355X-native implementation of the ``triton_helpers.layers`` neural-field hot paths.

``triton_helpers_amd.layers`` mirrors ``triton_helpers.layers`` of the reference:
``hash_encoding``, ``fully_fused_mlp`` and (new) ``reversible_mlp``.  All compute
runs in hand-written gfx950 kernels inside ``libnf_cdna4.so``.
"""
TENSOR_CORE_K = 16  # kept for API presence (triton_helpers/__init__.py of the reference)
__version__ = "0.1.0"
