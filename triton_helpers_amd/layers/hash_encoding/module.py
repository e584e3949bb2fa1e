"""``nn.Module`` wrapper of the hash encoding (reference hash_encoding/module.py:8-39).

State-dict keys (``embeddings``, ``pi``), constructor arguments and the N(0,1)
initialisation (one ``torch.randn`` draw per level, in level order, reference module.py:21)
are those of the reference, so checkpoints interchange and a seed gives the same table.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
from torch import Tensor

from .helpers import compute_embedding_counts
from .kernel import PI_1, PI_2, PI_3, hash_encoding


class HashEncoding(nn.Module):
    def __init__(
        self,
        max_entries_per_level: int = 2**14,
        num_levels: int = 16,
        d_in: int = 3,
        d_embed: int = 2,
        min_res: int = 16,
        max_res: int = 512,
    ):
        super().__init__()
        counts = compute_embedding_counts(num_levels, max_entries_per_level, d_in, min_res, max_res)
        # one draw per level: the generator's block-wise normal sampling makes this differ from a single draw over
        # the stacked table, and the seeded table has to be the reference's
        self.embeddings = nn.Parameter(torch.cat([torch.randn(t, d_embed) for t in counts], dim=0))
        self.register_buffer("pi", torch.tensor([PI_1, PI_2, PI_3], dtype=torch.int64))
        self.max_entries_per_level = max_entries_per_level
        self.num_levels = num_levels
        self.min_res = min_res
        self.max_res = max_res

    def forward(self, coords: Tensor, features: Optional[Tensor] = None, scale: float = 1.0) -> Tensor:
        return hash_encoding(
            coords,
            self.embeddings,
            features,
            self.pi,
            max_entries_per_level=self.max_entries_per_level,
            min_res=self.min_res,
            max_res=self.max_res,
            levels=self.num_levels,
            scale=scale,
        )

    def extra_repr(self) -> str:
        return (
            f"T={self.max_entries_per_level}, levels={self.num_levels}, d_embed={self.embeddings.shape[-1]}, "
            f"res={self.min_res}..{self.max_res}"
        )
