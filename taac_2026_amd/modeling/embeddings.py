"""Embedding primitives in front of the token backbone (src/taac2026/infrastructure/modeling/embeddings.py:65-80).

``sparse_embedding_bag_mean`` follows the reference helper of the same name in the forward. The reference wraps it in an
autograd function that hands the optimiser an uncoalesced sparse COO gradient (embeddings.py:17-63); here a table that
requires a gradient takes the dense gradient of the accelerator's autograd route (the embedding-bag backward kernel).
``hash_compress_ids`` is the small integer helper that folds raw ids into a table's bucket range before the lookup.
"""

from __future__ import annotations

import torch

from taac_2026_amd.accelerators.embedding import embedding_bag_mean


def sparse_embedding_bag_mean(weight: torch.Tensor, values: torch.Tensor) -> torch.Tensor:
    """Mean of ``weight`` rows over each bag's non-zero ids (embeddings.py:65-71)."""
    return embedding_bag_mean(weight, values)


def hash_compress_ids(values: torch.Tensor, num_buckets: int) -> torch.Tensor:
    """Positive ids -> ``(id - 1) mod num_buckets + 1``; ids <= 0 (padding) -> 0; no buckets -> all zeros
    (embeddings.py:74-80)."""
    if num_buckets <= 0:
        return values.new_zeros(values.shape)
    compressed = torch.remainder(values.clamp_min(1) - 1, int(num_buckets)) + 1
    return torch.where(values > 0, compressed, values.new_zeros(values.shape))


__all__ = ["hash_compress_ids", "sparse_embedding_bag_mean"]
