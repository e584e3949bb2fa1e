"""Alias of ``triton_helpers_amd.layers.hash_encoding.module``."""
from triton_helpers_amd.layers.hash_encoding.module import HashEncoding  # noqa: F401
