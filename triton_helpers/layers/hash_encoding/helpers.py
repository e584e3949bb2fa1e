"""Alias of ``triton_helpers_amd.layers.hash_encoding.helpers`` (level geometry under the reference's names)."""
from triton_helpers_amd.layers.hash_encoding.helpers import (  # noqa: F401
    compute_b, compute_embedding_counts, compute_level_embedding_offset, compute_resolutions, get_first_hash_level,
    level_geometry, seek_to_level_embeddings, total_rows,
)
