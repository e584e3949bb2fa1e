from triton_helpers_amd.layers.hash_encoding import HashEncoding, hash_encoding  # noqa: F401

__all__ = ["hash_encoding", "HashEncoding"]
