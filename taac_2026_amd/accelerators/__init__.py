"""Operator boundary of the HIP kernel path: flat re-exports in the style of the reference's
``taac2026.infrastructure.accelerators`` package (accelerators/__init__.py:83-138)."""

from taac_2026_amd.accelerators.attention import (
    FlashAttentionMaskPlan,
    StructuredAttentionMask,
    _plan_tilelang_flash_attention_mask,
    build_structured_mask,
    flash_attention,
    hip_flash_attention_kernel,
    plan_flash_attention_mask,
    plan_structured_attention_mask,
    qk_norm_rope,
    resolved_flash_attention_backend,
    rope_table,
)
from taac_2026_amd.accelerators.embedding import (
    embedding_bag_mean,
    hip_embedding_bag_mean_kernel,
    resolved_embedding_bag_mean_backend,
)
from taac_2026_amd.accelerators.linear import (
    amax,
    attention_out_ffn,
    linear,
    linear_fp8,
    norm_linear,
    qkv_projection,
    quantize_fp8,
    swiglu_ffn,
    swiglu_linear,
    valid_rows,
)
from taac_2026_amd.accelerators.readout import candidate_readout
from taac_2026_amd.accelerators.normalization import (
    hip_layer_norm_kernel,
    hip_rms_norm_kernel,
    layer_norm,
    resolved_layer_norm_backend,
    resolved_rms_norm_backend,
    rms_norm,
)
from taac_2026_amd.accelerators.tensor_validation import (
    concrete_tensors,
    require_cuda_tensors,
    require_same_device,
    require_same_dtype,
)

__all__ = [
    "candidate_readout",
    "attention_out_ffn",
    "FlashAttentionMaskPlan",
    "StructuredAttentionMask",
    "_plan_tilelang_flash_attention_mask",
    "amax",
    "build_structured_mask",
    "concrete_tensors",
    "embedding_bag_mean",
    "flash_attention",
    "hip_embedding_bag_mean_kernel",
    "hip_flash_attention_kernel",
    "hip_layer_norm_kernel",
    "hip_rms_norm_kernel",
    "layer_norm",
    "linear",
    "linear_fp8",
    "norm_linear",
    "plan_flash_attention_mask",
    "plan_structured_attention_mask",
    "qk_norm_rope",
    "qkv_projection",
    "quantize_fp8",
    "require_cuda_tensors",
    "require_same_device",
    "require_same_dtype",
    "resolved_embedding_bag_mean_backend",
    "resolved_flash_attention_backend",
    "resolved_layer_norm_backend",
    "resolved_rms_norm_backend",
    "rms_norm",
    "rope_table",
    "swiglu_ffn",
    "swiglu_linear",
    "valid_rows",
]
