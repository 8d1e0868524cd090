"""Sequence helpers around the HIP attention kernel.

Follows src/taac2026/infrastructure/modeling/sequence.py:22-60,81-127. ``scaled_dot_product_attention`` hands the
kernel (B, T, H, dh)-strided views of the (B, T, D) projections and gets the result back in the same memory layout,
so none of the reference's four layout copies is made. The mask / pooling helpers are small integer or elementwise
host-side torch expressions that run on whatever device their inputs live on.
"""

from __future__ import annotations

from contextvars import ContextVar

import torch

from taac_2026_amd.accelerators.attention import FLASH_ATTENTION_BACKENDS, StructuredAttentionMask, flash_attention

_FLASH_ATTENTION_BACKEND: ContextVar[str] = ContextVar("taac_2026_amd_flash_attention_backend", default="hip")


def configure_flash_attention_runtime(*, backend: str) -> None:
    if backend not in FLASH_ATTENTION_BACKENDS:
        raise ValueError(f"unsupported flash attention backend: {backend}")
    _FLASH_ATTENTION_BACKEND.set(backend)


def flash_attention_runtime_state() -> str:
    return _FLASH_ATTENTION_BACKEND.get()


def make_padding_mask(lengths: torch.Tensor, max_len: int) -> torch.Tensor:
    """(B,) lengths -> (B, max_len) bool, True = padding (position >= length)."""
    return torch.arange(max_len, device=lengths.device)[None, :] >= lengths[:, None]


def safe_key_padding_mask(mask: torch.Tensor) -> torch.Tensor:
    """Un-mask position 0 of rows that are padded everywhere, so that no softmax row is empty."""
    if mask.numel() == 0 or mask.shape[1] == 0:
        return mask
    fully_padded = mask.all(dim=1)
    result = mask.clone()
    result[fully_padded, 0] = False
    return result


def masked_mean(tokens: torch.Tensor, padding_mask: torch.Tensor | None = None) -> torch.Tensor:
    """Mean over the sequence axis of the non-padded tokens; the divisor is clamped to >= 1."""
    if tokens.shape[1] == 0:
        return tokens.new_zeros(tokens.shape[0], tokens.shape[-1])
    if padding_mask is None:
        return tokens.mean(dim=1)
    keep = (~padding_mask).to(tokens.dtype).unsqueeze(-1)
    return (tokens * keep).sum(dim=1) / keep.sum(dim=1).clamp_min(1.0)


def causal_valid_attention_mask(padding_mask: torch.Tensor, num_heads: int) -> torch.Tensor:
    """(B, T) padding mask -> (B, H, T, T) bool: causal over valid keys; padded queries see only themselves."""
    batch, tokens = padding_mask.shape
    positions = torch.arange(tokens, device=padding_mask.device)
    lower = positions[:, None] >= positions[None, :]
    visible = lower[None] & ~padding_mask[:, None, :]
    diagonal = torch.eye(tokens, dtype=torch.bool, device=padding_mask.device)[None]
    mask = torch.where(padding_mask[:, :, None], diagonal, visible)
    return mask[:, None].expand(batch, num_heads, tokens, tokens)


def scaled_dot_product_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    *,
    num_heads: int,
    attn_mask: torch.Tensor | None,
    dropout_p: float,
    training: bool,
    backend: str | None = None,
    is_causal: bool = False,
    block_m: int = 64,
    block_n: int = 64,
    num_stages: int = 1,
    threads: int = 128,
    key_lengths: torch.Tensor | None = None,
    zero_padded_queries: bool = False,
    q_row_scale: torch.Tensor | None = None,
    k_row_scale: torch.Tensor | None = None,
    q_col_scale: torch.Tensor | None = None,
    structured_mask: StructuredAttentionMask | None = None,
    dropout_mask: torch.Tensor | None = None,
) -> torch.Tensor:
    """Multi-head attention over (B, T, D) projections; returns (B, Tq, D). ``dropout_mask``: the uint8 keep mask
    (B, H, Tq, Tk) of a training forward with ``dropout_p > 0`` (drawn when not given). ``q_row_scale`` / ``k_row_scale``
    (float32 (B, T)) and ``q_col_scale`` (float32 (D,)): optional factors of the query / key rows and of the query
    features applied inside the kernel. ``structured_mask``: a :class:`StructuredAttentionMask` in place of ``attn_mask``."""
    batch, query_len, d_model = q.shape
    head_dim = d_model // num_heads
    q4 = q.view(batch, query_len, num_heads, head_dim).transpose(1, 2)
    k4 = k.view(batch, k.shape[1], num_heads, head_dim).transpose(1, 2)
    v4 = v.view(batch, v.shape[1], num_heads, head_dim).transpose(1, 2)
    output = flash_attention(
        q4,
        k4,
        v4,
        backend=flash_attention_runtime_state() if backend is None else backend,
        attn_mask=attn_mask,
        dropout_p=dropout_p,
        training=training,
        is_causal=is_causal,
        block_m=block_m,
        block_n=block_n,
        num_stages=num_stages,
        threads=threads,
        key_lengths=key_lengths,
        zero_padded_queries=zero_padded_queries,
        q_row_scale=q_row_scale,
        k_row_scale=k_row_scale,
        q_col_scale=q_col_scale,
        structured_mask=structured_mask,
        dropout_mask=dropout_mask,
    )
    return output.transpose(1, 2).contiguous().view(batch, query_len, d_model)


__all__ = [
    "causal_valid_attention_mask",
    "configure_flash_attention_runtime",
    "flash_attention_runtime_state",
    "make_padding_mask",
    "masked_mean",
    "safe_key_padding_mask",
    "scaled_dot_product_attention",
]
