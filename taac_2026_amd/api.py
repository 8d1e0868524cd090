"""Stable facade: the names experiment packages import from the reference's ``taac2026.api`` for this path
(src/taac2026/api.py:31-52), served by the HIP kernels, plus the block modules and dense-layer operators."""

from taac_2026_amd.accelerators import (
    amax,
    flash_attention,
    layer_norm,
    linear,
    linear_fp8,
    quantize_fp8,
    rms_norm,
    swiglu_ffn,
    swiglu_linear,
)
from taac_2026_amd.modeling import (
    LayerNorm,
    PCVRBackbone,
    RMSNorm,
    SwiGLUFeedForward,
    UnifiedInteractionBlock,
    UnifiedSelfAttention,
    causal_valid_attention_mask,
    configure_flash_attention_runtime,
    configure_rms_norm_runtime,
    make_padding_mask,
    masked_mean,
    safe_key_padding_mask,
    scaled_dot_product_attention,
)

__all__ = [
    "LayerNorm",
    "PCVRBackbone",
    "RMSNorm",
    "SwiGLUFeedForward",
    "UnifiedInteractionBlock",
    "UnifiedSelfAttention",
    "amax",
    "causal_valid_attention_mask",
    "configure_flash_attention_runtime",
    "configure_rms_norm_runtime",
    "flash_attention",
    "layer_norm",
    "linear",
    "linear_fp8",
    "make_padding_mask",
    "masked_mean",
    "quantize_fp8",
    "rms_norm",
    "safe_key_padding_mask",
    "scaled_dot_product_attention",
    "swiglu_ffn",
    "swiglu_linear",
]
