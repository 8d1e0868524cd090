"""Model-level primitives built on the HIP operators."""

from taac_2026_amd.modeling.backbone import (
    BFTSAttention,
    FeedForward,
    MixedFeedForward,
    PCVRBackbone,
    SwiGLUFeedForward,
    TokenFormerBlock,
    UnifiedInteractionBlock,
    run_interaction_blocks,
    UnifiedSelfAttention,
)
from taac_2026_amd.modeling.embeddings import hash_compress_ids, sparse_embedding_bag_mean
from taac_2026_amd.modeling.masks import (
    MetadataAttentionMask,
    bfts_attention_mask,
    bfts_structural_mask,
    metadata_structural_mask,
)
from taac_2026_amd.modeling.normalization import (
    LayerNorm,
    RMSNorm,
    configure_rms_norm_runtime,
    rms_norm_runtime_state,
)
from taac_2026_amd.modeling.readout import CandidateClsPooler, CandidateReadoutHead
from taac_2026_amd.modeling.sequence import (
    causal_valid_attention_mask,
    configure_flash_attention_runtime,
    flash_attention_runtime_state,
    make_padding_mask,
    masked_mean,
    safe_key_padding_mask,
    scaled_dot_product_attention,
)

__all__ = [
    "BFTSAttention",
    "FeedForward",
    "MixedFeedForward",
    "CandidateClsPooler",
    "CandidateReadoutHead",
    "LayerNorm",
    "MetadataAttentionMask",
    "PCVRBackbone",
    "RMSNorm",
    "SwiGLUFeedForward",
    "TokenFormerBlock",
    "UnifiedInteractionBlock",
    "run_interaction_blocks",
    "UnifiedSelfAttention",
    "bfts_attention_mask",
    "bfts_structural_mask",
    "causal_valid_attention_mask",
    "configure_flash_attention_runtime",
    "configure_rms_norm_runtime",
    "flash_attention_runtime_state",
    "hash_compress_ids",
    "make_padding_mask",
    "masked_mean",
    "metadata_structural_mask",
    "rms_norm_runtime_state",
    "safe_key_padding_mask",
    "scaled_dot_product_attention",
    "sparse_embedding_bag_mean",
]
