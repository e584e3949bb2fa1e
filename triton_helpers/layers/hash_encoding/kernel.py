"""Alias of ``triton_helpers_amd.layers.hash_encoding.kernel`` with the names code written against the reference imports."""
from triton_helpers_amd.layers.hash_encoding.kernel import (  # noqa: F401
    BWD_DIVIDER_CONFIGS, DIVIDER_CONFIGS, PI_1, PI_2, PI_3, HashEncoding, hash_encoding, hash_encoding_indices,
    hash_encoding_table_grad,
)
from triton_helpers_amd.layers.hash_encoding.helpers import (  # noqa: F401
    compute_b, compute_embedding_counts, compute_level_embedding_offset, compute_resolutions, get_first_hash_level,
    seek_to_level_embeddings,
)
