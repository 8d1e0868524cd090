"""Model-level attention masks of the reference's experiment packages in the factored form the HIP attention kernel
consumes: a structural (query, key) matrix shared by the batch and the heads, the per-sample key validity and the
per-sample query rows that fall back to themselves.

``bfts_attention_mask`` follows ``PCVRTokenFormer._bfts_attention_mask`` (experiments/tokenformer/model.py:474-503),
``MetadataAttentionMask`` follows the module of the same name (experiments/symbiosis/attention.py:17-60). Both return a
:class:`StructuredAttentionMask`; its ``dense()`` is the (B, 1, T, T) bool mask the reference builds. The structural
part is a few (T, T) elementwise torch expressions on the inputs' device; the B * T * T mask is never materialised.
"""

from __future__ import annotations

import math

import torch
import torch.nn as nn

from taac_2026_amd.accelerators.attention import StructuredAttentionMask, build_structured_mask
from taac_2026_amd.modeling.sequence import safe_key_padding_mask

# Token roles of the TokenFormer package (experiments/tokenformer/model.py:32-37).
BFTS_ROLE_USER, BFTS_ROLE_SEQUENCE, BFTS_ROLE_ITEM, BFTS_ROLE_TARGET, BFTS_ROLE_SEPARATOR, BFTS_ROLE_DENSE = range(6)
# Token roles of the Symbiosis package (experiments/symbiosis/tokenization.py:22-30).
(ROLE_CLS, ROLE_CANDIDATE, ROLE_USER, ROLE_ITEM, ROLE_DENSE, ROLE_MISSING, ROLE_SEQUENCE, ROLE_STATS) = range(8)


def bfts_structural_mask(role_ids: torch.Tensor, layer_index: int, num_layers: int, *, seq_causal: bool,
                         seq_keep_per_domain: int) -> torch.Tensor:
    """The (T, T) part of the bottom-full / top-sliding mask: the lower ``max(1, num_layers // 2)`` layers see everything
    (or the causal triangle), layer ``s`` above them a window of ``max(4, ceil(seq_keep_per_domain / 2**s))`` positions;
    every query sees itself, a target query sees everything, separator keys are seen by everyone."""
    token_count = role_ids.shape[0]
    positions = torch.arange(token_count, device=role_ids.device)
    key_positions, query_positions = positions[None, :], positions[:, None]
    bottom_full_layers = max(1, int(num_layers) // 2)
    if layer_index < bottom_full_layers:
        if seq_causal:
            structural = key_positions <= query_positions
        else:
            structural = torch.ones(token_count, token_count, dtype=torch.bool, device=role_ids.device)
    else:
        window = max(4, math.ceil(int(seq_keep_per_domain) / (2 ** (layer_index - bottom_full_layers))))
        distance = query_positions - key_positions
        structural = ((distance >= 0) & (distance <= window)) if seq_causal else (distance.abs() <= window)
    structural = structural | torch.eye(token_count, dtype=torch.bool, device=role_ids.device)
    structural = torch.where((role_ids == BFTS_ROLE_TARGET)[:, None], torch.ones_like(structural), structural)
    return structural | (role_ids == BFTS_ROLE_SEPARATOR)[None, :]


def bfts_attention_mask(padding_mask: torch.Tensor, role_ids: torch.Tensor, layer_index: int, num_layers: int, *,
                        seq_causal: bool, seq_keep_per_domain: int) -> StructuredAttentionMask:
    """``structural & key_valid`` with padded query rows attending to themselves only (model.py:499-503)."""
    structural = bfts_structural_mask(role_ids, layer_index, num_layers, seq_causal=seq_causal,
                                      seq_keep_per_domain=seq_keep_per_domain)
    # window layers: a 32-query tile sees its band (two or three key tiles) and the separator columns
    bottom_full_layers = max(1, int(num_layers) // 2)
    window = None if layer_index < bottom_full_layers else max(
        4, math.ceil(int(seq_keep_per_domain) / (2 ** (layer_index - bottom_full_layers))))
    sparse = window is not None and role_ids.shape[0] <= 2048 and 4 * (window + 64) <= role_ids.shape[0]
    return build_structured_mask(structural, ~safe_key_padding_mask(padding_mask), padding_mask, sparse=sparse)


def metadata_structural_mask(role_ids: torch.Tensor) -> torch.Tensor:
    """Which key roles a query role may read (attention.py:26-58): readout (CLS, candidate) and statistics queries read
    everything; field queries (user, item, dense, missing) read readout, field and statistics keys; sequence queries
    read readout, item, sequence, missing and statistics keys; every query reads itself."""
    token_count = role_ids.shape[0]
    key_roles, query_roles = role_ids[None, :], role_ids[:, None]

    def any_of(roles: torch.Tensor, *values: int) -> torch.Tensor:
        result = torch.zeros_like(roles, dtype=torch.bool)
        for value in values:
            result = result | (roles == value)
        return result

    readout_query = any_of(query_roles, ROLE_CLS, ROLE_CANDIDATE)
    field_query = any_of(query_roles, ROLE_USER, ROLE_ITEM, ROLE_DENSE, ROLE_MISSING)
    sequence_query = query_roles == ROLE_SEQUENCE
    stats_query = query_roles == ROLE_STATS
    all_keys = torch.ones_like(key_roles, dtype=torch.bool)
    field_keys = any_of(key_roles, ROLE_CLS, ROLE_CANDIDATE, ROLE_USER, ROLE_ITEM, ROLE_DENSE, ROLE_MISSING, ROLE_STATS)
    sequence_keys = any_of(key_roles, ROLE_CLS, ROLE_CANDIDATE, ROLE_ITEM, ROLE_SEQUENCE, ROLE_MISSING, ROLE_STATS)
    structural = torch.zeros(token_count, token_count, dtype=torch.bool, device=role_ids.device)
    structural = torch.where(readout_query, all_keys.expand_as(structural), structural)
    structural = torch.where(field_query, field_keys.expand_as(structural), structural)
    structural = torch.where(sequence_query, sequence_keys.expand_as(structural), structural)
    structural = torch.where(stats_query, all_keys.expand_as(structural), structural)
    return structural | torch.eye(token_count, dtype=torch.bool, device=role_ids.device)


class MetadataAttentionMask(nn.Module):
    """``forward(padding_mask (B, T), role_ids (T,)) -> StructuredAttentionMask``; disabled: every valid key is visible.
    (The reference module takes its token batch object and reads these two fields from it.)"""

    def __init__(self, *, enabled: bool = True) -> None:
        super().__init__()
        self.enabled = bool(enabled)

    def forward(self, padding_mask: torch.Tensor, role_ids: torch.Tensor) -> StructuredAttentionMask:
        token_count = padding_mask.shape[1]
        if self.enabled:
            structural = metadata_structural_mask(role_ids)
        else:
            structural = torch.ones(token_count, token_count, dtype=torch.bool, device=padding_mask.device)
        return build_structured_mask(structural, ~safe_key_padding_mask(padding_mask), None, padding_source=padding_mask)


__all__ = [
    "MetadataAttentionMask",
    "bfts_attention_mask",
    "bfts_structural_mask",
    "metadata_structural_mask",
]
