"""Flash-attention operator boundary backed by the gfx950 key-length kernel.

Mirrors ``flash_attention`` and its mask planner
(src/taac2026/infrastructure/accelerators/attention/flash_attention.py:107-209, 871-919). The kernel understands one
mask family: a per-sample valid key prefix (``key_lengths``), optionally combined with a causal triangle. A 4-D bool
``attn_mask`` is reduced to that form by :func:`plan_flash_attention_mask`, which accepts the same structured masks
as the reference planner and rejects the rest with the reference's messages; callers that already know the lengths
pass ``key_lengths=`` and skip the planning (and its device-to-host synchronisation) entirely.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import ctypes

import torch

from taac_2026_amd import _native
from taac_2026_amd.accelerators.tensor_validation import (
    require_cuda_tensors,
    require_inference,
    require_same_dtype,
)

FLASH_ATTENTION_BACKENDS = ("hip", "torch", "tilelang")


@dataclass(frozen=True)
class FlashAttentionMaskPlan:
    """What the kernel needs to know about a mask (flash_attention.py:60-64)."""

    key_lengths: torch.Tensor | None
    query_self_mask: torch.Tensor | None
    is_causal: bool


@dataclass(frozen=True)
class StructuredAttentionMask:
    """Bit form of a mask ``visible[b, i, j] = structural[i, j] & key_valid[b, j]`` (shared by the heads), optionally with
    query rows that attend to themselves only (``query_self``: their output is their value row). This is the shape of the
    reference's model-level masks (experiments/tokenformer/model.py:474-503, experiments/symbiosis/attention.py:21-60).
    Built by :func:`build_structured_mask`; ``dense()`` gives the (B, 1, Tq, Tk) bool mask the reference would pass."""

    struct_bits: torch.Tensor          # int32 (Tq, ceil(Tk / 32)); front layout: (B * Tq, ceil(Tk / 32))
    block_any: torch.Tensor | None     # uint8 (ceil(Tq / 128), ceil(Tk / 64)); front layout: None
    valid_bits: torch.Tensor | None    # int32 (B, ceil(Tk / 32))
    self_bits: torch.Tensor | None     # int32 (B, ceil(Tq / 32))
    structural: torch.Tensor           # bool (Tq, Tk)
    key_valid: torch.Tensor | None     # bool (B, Tk)
    query_self: torch.Tensor | None    # bool (B, Tq)
    sample_stride: int = 0             # words between the bit matrices of consecutive samples (front layout), else 0
    padding_source: torch.Tensor | None = None  # the (B, Tk) padding mask that key_valid is the complement of, if any
    # few visible 32 x 32 tiles per query tile (sliding windows, a few global rows / columns): the kernel that gives every
    # 32-query tile its own wavefront and visits only that tile's visible key tiles pays; dense masks keep the chunked one
    sparse: bool = False
    # what callers derive from this mask once per forward pass (row indices, its front-layout form): the blocks of a
    # stack receive the same mask object and share it
    cache: dict = field(default_factory=dict, compare=False, repr=False)

    def dense(self) -> torch.Tensor:
        if self.sample_stride:
            raise RuntimeError("a mask in the front layout has no dense form; use the mask it was made from")
        query_len, kv_len = self.structural.shape
        mask = self.structural[None]
        if self.key_valid is not None:
            mask = mask & self.key_valid[:, None, :]
        if self.query_self is not None:
            eye = torch.eye(query_len, kv_len, dtype=torch.bool, device=self.structural.device)
            mask = torch.where(self.query_self[:, :, None], eye[None], mask)
        return mask[:, None]


def front_structured_mask(mask: StructuredAttentionMask, token_rows: tuple[torch.Tensor, torch.Tensor],
                          batch: int) -> StructuredAttentionMask:
    """``mask`` for samples whose valid tokens were moved to the front of their rows (``token_rows`` = the index of
    ``valid_rows(..., padding_mask=)`` over the same validity as ``mask.key_valid``): one structural bit matrix per
    sample, ``bits[b, r, j] = structural[position(b, r), position(b, j)]``, every listed key valid. Use it together
    with ``key_lengths`` = the samples' numbers of valid tokens."""
    name = "hip front_structured_mask"
    query_len, kv_len = mask.structural.shape
    if query_len != kv_len or mask.query_self is not None or mask.sample_stride:
        raise ValueError(f"{name}: needs a square mask without self rows that is not in the front layout already")
    rows, _ = token_rows
    require_cuda_tensors(name, rows, mask.struct_bits)
    words = (kv_len + 31) // 32
    if rows.dtype != torch.int32 or rows.numel() < batch * query_len + batch + 1 or not rows.is_contiguous():
        raise ValueError(f"{name}: token_rows must be the index returned by valid_rows for (batch, tokens)")
    bits = torch.empty(batch * query_len, words, dtype=torch.int32, device=rows.device)
    library = _native.load_library()
    status = library.taac_mask_front_bits(mask.struct_bits.data_ptr(), query_len, rows.data_ptr(), int(batch),
                                          bits.data_ptr(), _native.current_stream(rows.device))
    _native.check(status, "mask_front_bits")
    return StructuredAttentionMask(bits, None, None, None, mask.structural, None, None, query_len * words)


def _pack_bits(mask: torch.Tensor) -> torch.Tensor:
    rows, cols = mask.shape
    bits = torch.empty(rows, (cols + 31) // 32, dtype=torch.int32, device=mask.device)
    library = _native.load_library()
    status = library.taac_mask_pack_bits(mask.data_ptr(), rows, cols, bits.data_ptr(), _native.current_stream(mask.device))
    _native.check(status, "mask_pack_bits")
    return bits


def build_structured_mask(
    structural: torch.Tensor, key_valid: torch.Tensor | None = None, query_self: torch.Tensor | None = None,
    *, padding_source: torch.Tensor | None = None, sparse: bool = False,
) -> StructuredAttentionMask:
    """``structural`` (Tq, Tk) bool, True = attend; ``key_valid`` (B, Tk) bool or None; ``query_self`` (B, Tq) bool or
    None (needs Tq == Tk). Everything stays on the device (no host synchronisation). ``padding_source``: the padding
    mask whose non-padded positions are exactly the valid keys of every sample that has one (a caller that skips the
    padded rows with the same mask can then run the attention over the valid tokens only). ``sparse``: the caller knows
    that a query tile sees few key tiles (a sliding window plus a few global rows and columns) and prefers the kernel
    built for that; the result does not depend on it."""
    name = "hip build_structured_mask"
    require_cuda_tensors(name, structural, key_valid, query_self)
    for tensor, label in ((structural, "structural"), (key_valid, "key_valid"), (query_self, "query_self")):
        if tensor is not None and (tensor.dtype is not torch.bool or tensor.ndim != 2):
            raise ValueError(f"{name}: {label} must be a 2-D bool tensor")
    query_len, kv_len = structural.shape
    if key_valid is not None and key_valid.shape[1] != kv_len:
        raise ValueError(f"{name}: key_valid must have shape (batch, kv_len)")
    if query_self is not None and (query_len != kv_len or query_self.shape[1] != query_len):
        raise ValueError(f"{name}: query_self must have shape (batch, query_len) and needs query_len == kv_len")
    structural = structural.contiguous()
    struct_bits = _pack_bits(structural)
    block_any = torch.empty((query_len + 127) // 128, (kv_len + 63) // 64, dtype=torch.uint8, device=structural.device)
    library = _native.load_library()
    status = library.taac_mask_block_any(struct_bits.data_ptr(), query_len, kv_len, block_any.data_ptr(),
                                         _native.current_stream(structural.device))
    _native.check(status, "mask_block_any")
    key_valid = None if key_valid is None else key_valid.contiguous()
    query_self = None if query_self is None else query_self.contiguous()
    return StructuredAttentionMask(
        struct_bits, block_any, None if key_valid is None else _pack_bits(key_valid),
        None if query_self is None else _pack_bits(query_self), structural, key_valid, query_self, 0, padding_source,
        sparse=bool(sparse),
    )


def plan_structured_attention_mask(q: torch.Tensor, k: torch.Tensor, attn_mask: torch.Tensor) -> StructuredAttentionMask:
    """Factor a (B, H | 1, Tq, Tk) bool mask into ``structural[i, j] & key_valid[b, j]`` with optional self-only query
    rows, verifying the factorisation exactly; ``RuntimeError`` when the mask has no such form. This reads the full mask
    several times and synchronises with the host (as the reference's planner does, flash_attention.py:149-198): callers
    that know the factors pass ``structured_mask=build_structured_mask(...)`` instead."""
    batch, heads, query_len, kv_len = q.shape[0], q.shape[1], q.shape[2], k.shape[2]
    if attn_mask.dtype is not torch.bool:
        raise RuntimeError("hip flash_attention only supports structured bool attention masks")
    if attn_mask.ndim != 4 or attn_mask.shape[0] != batch or attn_mask.shape[1] not in (1, heads) or \
            attn_mask.shape[2:] != (query_len, kv_len):
        raise RuntimeError("hip flash_attention only supports 4D bool masks matching (batch, heads, query_len, kv_len)")
    if attn_mask.shape[1] != 1 and not torch.equal(attn_mask, attn_mask[:, :1].expand_as(attn_mask)):
        raise RuntimeError("hip flash_attention requires the bool attention mask to be shared across heads")
    mask = attn_mask[:, 0]
    query_self = None
    live = mask
    if query_len == kv_len:
        eye = torch.eye(query_len, dtype=torch.bool, device=mask.device)
        query_self = (mask == eye[None]).all(dim=-1)
        live = mask & ~query_self[:, :, None]
    key_valid = live.any(dim=1)
    structural = live.any(dim=0)
    expected = structural[None] & key_valid[:, None, :]
    if query_self is not None:
        expected = torch.where(query_self[:, :, None], eye[None], expected)
    if not torch.equal(expected, mask):
        raise RuntimeError(
            "hip flash_attention only supports bool masks of the form structural[query, key] & key_valid[batch, key] "
            "(shared by the heads), optionally with padded query rows that attend to themselves only"
        )
    if query_self is not None and not bool(query_self.any()):
        query_self = None
    return build_structured_mask(structural, key_valid, query_self, sparse=_few_visible_tiles(structural))


def _few_visible_tiles(structural: torch.Tensor) -> bool:
    """True when at most a third of the 32 x 32 tiles of the (Tq, Tk) structure hold a visible pair (one host sync)."""
    query_len, kv_len = structural.shape
    if kv_len > 2048:
        return False
    padded = torch.zeros((query_len + 31) // 32 * 32, (kv_len + 31) // 32 * 32, dtype=torch.bool, device=structural.device)
    padded[:query_len, :kv_len] = structural
    tiles = padded.view(padded.shape[0] // 32, 32, padded.shape[1] // 32, 32).any(dim=3).any(dim=1)
    return bool(tiles.float().mean().item() <= 1.0 / 3.0)


def _compact_tables(mask: StructuredAttentionMask, batch: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """The mask's structure in the per-tile kernel's compact form (made once per mask object): per 32-query tile the
    visible key columns, per compact tile of 32 such keys the key words it draws from, per query row its words."""
    tables = mask.cache.get("compact_tables")
    if tables is None:
        query_len, kv_len = mask.structural.shape
        samples = batch if mask.sample_stride else 1
        words = (kv_len + 31) // 32
        tiles = (query_len + 31) // 32
        device = mask.struct_bits.device
        bits = torch.empty(samples, query_len, words, dtype=torch.int32, device=device)
        keys = torch.empty(samples, tiles, 32 * words, dtype=torch.int32, device=device)
        tile_words = torch.empty(samples, tiles, 64, dtype=torch.int64, device=device)
        library = _native.load_library()
        status = library.taac_mask_compact(mask.struct_bits.data_ptr(), samples, query_len, kv_len, int(mask.sample_stride),
                                           bits.data_ptr(), keys.data_ptr(), tile_words.data_ptr(),
                                           _native.current_stream(device))
        _native.check(status, "mask_compact")
        tables = (bits, keys, tile_words)
        mask.cache["compact_tables"] = tables
    return tables


def _normalize_flash_attention_inputs(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Shape / dtype checks of flash_attention.py:107-123; layout is left alone (the kernel reads strides)."""
    if q.ndim != 4 or k.ndim != 4 or v.ndim != 4:
        raise ValueError("flash_attention expects q, k, and v with shape (batch, heads, seq_len, head_dim)")
    if q.shape[0] != k.shape[0] or q.shape[0] != v.shape[0]:
        raise ValueError("flash_attention requires matching batch dimensions")
    if q.shape[1] != k.shape[1] or q.shape[1] != v.shape[1]:
        raise ValueError("flash_attention requires matching head counts")
    if k.shape[2] != v.shape[2]:
        raise ValueError("flash_attention requires matching key and value sequence lengths")
    if q.shape[3] != k.shape[3] or q.shape[3] != v.shape[3]:
        raise ValueError("flash_attention requires matching head dimensions")
    require_same_dtype("flash_attention", q, k, v)
    return q, k, v


def _full_key_lengths(q: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
    return torch.full((q.shape[0],), k.shape[2], dtype=torch.int32, device=q.device)


def _is_prefix_valid_mask(valid: torch.Tensor) -> bool:
    """True iff every row of the (B, Tk) bool matrix is ``True`` on a prefix and ``False`` after it."""
    lengths = valid.sum(dim=1, dtype=torch.int32).unsqueeze(1)
    expected = torch.arange(valid.shape[1], device=valid.device).unsqueeze(0) < lengths
    return bool(torch.equal(valid, expected))


def _causal_valid_mask_from_lengths(lengths: torch.Tensor, token_count: int, num_heads: int) -> torch.Tensor:
    """The mask ``causal_valid_attention_mask`` builds for prefix lengths (modeling/sequence.py:119-127)."""
    positions = torch.arange(token_count, device=lengths.device)
    padded = positions.unsqueeze(0) >= lengths.unsqueeze(1)  # (B, T)
    lower = positions.unsqueeze(1) >= positions.unsqueeze(0)  # (T, T), query >= key
    visible = lower.unsqueeze(0) & ~padded.unsqueeze(1)
    diagonal = torch.eye(token_count, dtype=torch.bool, device=lengths.device).unsqueeze(0)
    mask = torch.where(padded.unsqueeze(-1), diagonal, visible)
    return mask.unsqueeze(1).expand(lengths.shape[0], num_heads, token_count, token_count)


def plan_flash_attention_mask(
    q: torch.Tensor,
    k: torch.Tensor,
    attn_mask: torch.Tensor | None,
    *,
    is_causal: bool,
) -> FlashAttentionMaskPlan:
    """Reduce a bool mask to ``key_lengths`` (+ optional padded-query fallback), like flash_attention.py:149-198.

    Accepted: ``None``; a (B, H, Tq, Tk) bool mask that is head-shared, query-broadcast and prefix-valid on keys;
    a ``causal_valid_attention_mask``-style (B, H, T, T) mask. In addition to the reference, the broadcastable
    key-padding forms (B, Tk) and (B, 1, 1, Tk) (True = attend) are accepted without expanding them.
    """
    if attn_mask is None:
        return FlashAttentionMaskPlan(_full_key_lengths(q, k), None, is_causal)
    if attn_mask.dtype is not torch.bool:
        raise RuntimeError("hip flash_attention only supports structured bool attention masks")

    batch, heads, query_len, kv_len = q.shape[0], q.shape[1], q.shape[2], k.shape[2]
    key_valid: torch.Tensor | None = None
    if attn_mask.ndim == 2 and attn_mask.shape == (batch, kv_len):
        key_valid = attn_mask
    elif attn_mask.ndim == 4 and attn_mask.shape == (batch, 1, 1, kv_len):
        key_valid = attn_mask[:, 0, 0, :]
    if key_valid is not None:
        if not _is_prefix_valid_mask(key_valid):
            raise RuntimeError("hip flash_attention requires bool key masks to be prefix-valid")
        return FlashAttentionMaskPlan(key_valid.sum(dim=1, dtype=torch.int32), None, is_causal)

    if attn_mask.ndim != 4 or attn_mask.shape != (batch, heads, query_len, kv_len):
        raise RuntimeError(
            "hip flash_attention only supports 4D bool masks matching (batch, heads, query_len, kv_len)"
        )
    first_head = attn_mask[:, :1]
    if not torch.equal(attn_mask, first_head.expand_as(attn_mask)):
        raise RuntimeError("hip flash_attention requires the bool attention mask to be shared across heads")

    per_query = first_head[:, 0]  # (B, Tq, Tk)
    if torch.equal(per_query, per_query[:, :1, :].expand_as(per_query)):
        key_valid = per_query[:, 0, :]
        if not _is_prefix_valid_mask(key_valid):
            raise RuntimeError("hip flash_attention requires bool key masks to be prefix-valid")
        return FlashAttentionMaskPlan(key_valid.sum(dim=1, dtype=torch.int32), None, is_causal)

    if query_len != kv_len:
        raise RuntimeError(
            "hip flash_attention only supports non-broadcast bool masks when query and key lengths match"
        )
    query_lengths = per_query[:, :, 0].sum(dim=1, dtype=torch.int32)
    if not torch.equal(attn_mask, _causal_valid_mask_from_lengths(query_lengths, query_len, heads)):
        raise RuntimeError(
            "hip flash_attention only supports prefix key masks or causal_valid_attention_mask-style bool masks"
        )
    positions = torch.arange(query_len, device=q.device).unsqueeze(0)
    return FlashAttentionMaskPlan(query_lengths, positions >= query_lengths.unsqueeze(1), True)


# Name under which the reference exports its planner (accelerators/__init__.py:83-138).
_plan_tilelang_flash_attention_mask = plan_flash_attention_mask


def _apply_query_self_mask_fallback(
    output: torch.Tensor, value: torch.Tensor, query_self_mask: torch.Tensor | None
) -> torch.Tensor:
    """Padded query rows of a causal-valid mask attend only to themselves: their output is their value row."""
    if query_self_mask is None:
        return output
    return torch.where(query_self_mask[:, None, :, None], value, output)


def _resolve_flash_attention_backend(q: torch.Tensor, backend: str, *, dropout_p: float, training: bool) -> str:
    if backend not in FLASH_ATTENTION_BACKENDS:
        raise ValueError(f"unsupported flash attention backend: {backend}")
    if dropout_p < 0.0 or dropout_p >= 1.0:
        raise RuntimeError("hip flash_attention requires dropout_p to be in [0, 1)")
    if dropout_p != 0.0 and not training:
        raise RuntimeError("hip flash_attention only supports dropout during training")
    require_cuda_tensors("hip flash_attention", q)
    return "hip"


def resolved_flash_attention_backend(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    backend: str = "hip",
    *,
    attn_mask: torch.Tensor | None = None,
    dropout_p: float = 0.0,
    training: bool = False,
    is_causal: bool = False,
) -> str:
    _normalize_flash_attention_inputs(q, k, v)
    plan_flash_attention_mask(q, k, attn_mask, is_causal=is_causal)
    return _resolve_flash_attention_backend(q, backend, dropout_p=dropout_p, training=training)


def _kernel_view(t: torch.Tensor) -> torch.Tensor:
    """Return ``t`` if the kernel can read it in place (unit last stride, other strides multiples of 8 elements,
    16-byte aligned base), else a contiguous copy."""
    strides = t.stride()
    if strides[-1] == 1 and all(s % 8 == 0 and s >= 0 for s in strides[:-1]) and t.data_ptr() % 16 == 0:
        return t
    return t.contiguous()


def hip_flash_attention_kernel(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    key_lengths: torch.Tensor | None,
    *,
    is_causal: bool = False,
    zero_padded_queries: bool | int = False,
    q_row_scale: torch.Tensor | None = None,
    k_row_scale: torch.Tensor | None = None,
    q_col_scale: torch.Tensor | None = None,
    structured_mask: StructuredAttentionMask | None = None,
    kv_staging: str = "direct",
    amax_out: torch.Tensor | None = None,
) -> torch.Tensor:
    """``(q, k, v: (B, H, T, d) bf16/fp16, key_lengths: int32[B]) -> (B, H, Tq, d)``.

    Same contract as a kernel handed to the reference's ``register_flash_attention_kernel``
    (flash_attention.py:26,102-104, called at :351-352), extended by the keyword arguments. The output keeps
    q's memory layout, so (B, T, H, d)-strided views stay copy-free in both directions. ``q_row_scale`` (B, Tq) /
    ``k_row_scale`` (B, Tk): optional positive fp32 factors of the query / key rows, shared by the heads (a
    normalisation statistic applied inside the kernel instead of in a pass of its own); ``q_col_scale`` (H * d,):
    optional fp32 factors of the query features (the product of a query and a key norm weight). ``structured_mask``:
    a :class:`StructuredAttentionMask` (excludes ``is_causal``; combines with ``key_lengths``). ``kv_staging``:
    ``"direct"`` (K / V chunks go from global memory straight into LDS) or ``"registers"`` (the general kernel; same
    results, kept as a comparison route). ``amax_out``: a float32 scalar tensor that receives ``max |output|`` over the rows
    the kernel writes (the FP8 scale of the layer that consumes the output; not with a structured mask).
    """
    library = _native.load_library()
    require_cuda_tensors("hip flash_attention", q, k, v, key_lengths)
    if q.dtype not in (torch.bfloat16, torch.float16):
        raise RuntimeError(f"hip flash_attention kernel does not support dtype {q.dtype}")
    q, k, v = _kernel_view(q), _kernel_view(k), _kernel_view(v)
    out = torch.empty_like(q)  # keeps q's dimension order in memory, without q's gaps
    if out.stride(-1) != 1 or any(s % 8 for s in out.stride()[:-1]):
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    if key_lengths is not None:
        if key_lengths.ndim != 1 or key_lengths.shape[0] != q.shape[0]:
            raise ValueError("flash_attention key_lengths must have shape (batch,)")
        if key_lengths.dtype != torch.int32 or not key_lengths.is_contiguous():
            key_lengths = key_lengths.to(torch.int32).contiguous()
    batch, heads, query_len, head_dim = q.shape
    for scale, rows, label in ((q_row_scale, query_len, "q_row_scale"), (k_row_scale, k.shape[2], "k_row_scale")):
        if scale is None:
            continue
        require_cuda_tensors("hip flash_attention", scale)
        if scale.dtype != torch.float32 or scale.shape != (batch, rows) or not scale.is_contiguous():
            raise ValueError(f"flash_attention {label} must be a contiguous float32 tensor of shape (batch, rows)")
    if q_col_scale is not None:
        require_cuda_tensors("hip flash_attention", q_col_scale)
        if q_col_scale.dtype != torch.float32 or q_col_scale.numel() != heads * head_dim or not q_col_scale.is_contiguous():
            raise ValueError("flash_attention q_col_scale must be a contiguous float32 tensor of heads * head_dim values")
    if structured_mask is not None:
        if amax_out is not None:
            raise ValueError("flash_attention: amax_out is not available under a structured mask")
        if is_causal:
            raise ValueError("flash_attention: a structured mask carries its own causal triangle (is_causal must be False)")
        sm = structured_mask
        if sm.structural.shape != (query_len, k.shape[2]) or (sm.key_valid is not None and sm.key_valid.shape[0] != batch) \
                or (sm.query_self is not None and sm.query_self.shape[0] != batch) \
                or (sm.sample_stride and sm.struct_bits.shape[0] != batch * query_len):
            raise ValueError("flash_attention: the structured mask does not match (batch, query_len, kv_len)")
        require_cuda_tensors("hip flash_attention", sm.struct_bits)
        per_tile = sm.sparse and head_dim in (32, 64) and k.shape[2] <= 2048 and k.stride(2) < (1 << 20) and v.stride(2) < (1 << 20)
        tail = (
            _native.ptr(sm.valid_bits), _native.ptr(sm.self_bits), _native.ptr(q_row_scale),
            _native.ptr(k_row_scale), _native.ptr(q_col_scale), out.data_ptr(),
            batch, heads, query_len, k.shape[2], head_dim,
            _native.Int64x4(*q.stride()), _native.Int64x4(*k.stride()), _native.Int64x4(*v.stride()),
            _native.Int64x4(*out.stride()), int(zero_padded_queries), _native.dtype_code(q.dtype),
            _native.current_stream(q.device),
        )
        if per_tile:
            bits, keys, tile_words = _compact_tables(sm, batch)
            status = library.taac_flash_attn_sparse_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), _native.ptr(key_lengths), bits.data_ptr(),
                query_len * bits.shape[2] if sm.sample_stride else 0, keys.data_ptr(), tile_words.data_ptr(), *tail)
        else:
            status = library.taac_flash_attn_masked_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), _native.ptr(key_lengths), sm.struct_bits.data_ptr(),
                int(sm.sample_stride), _native.ptr(sm.block_any), *tail)
        _native.check(status, "flash_attention")
        return out
    if amax_out is not None:
        require_cuda_tensors("hip flash_attention", amax_out)
        if amax_out.dtype != torch.float32 or amax_out.numel() != 1:
            raise ValueError("flash_attention amax_out must be a float32 scalar tensor")
        status = library.taac_flash_attn_amax_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), _native.ptr(key_lengths), _native.ptr(q_row_scale),
            _native.ptr(k_row_scale), _native.ptr(q_col_scale), out.data_ptr(), amax_out.data_ptr(),
            batch, heads, query_len, k.shape[2], head_dim,
            _native.Int64x4(*q.stride()), _native.Int64x4(*k.stride()), _native.Int64x4(*v.stride()),
            _native.Int64x4(*out.stride()),
            _mask_flags(is_causal, kv_staging), int(zero_padded_queries), _native.dtype_code(q.dtype),
            _native.current_stream(q.device),
        )
        _native.check(status, "flash_attention")
        return out
    status = library.taac_flash_attn_scaled_fwd(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), _native.ptr(key_lengths), _native.ptr(q_row_scale),
        _native.ptr(k_row_scale), _native.ptr(q_col_scale), out.data_ptr(),
        batch, heads, query_len, k.shape[2], head_dim,
        _native.Int64x4(*q.stride()), _native.Int64x4(*k.stride()), _native.Int64x4(*v.stride()),
        _native.Int64x4(*out.stride()),
        _mask_flags(is_causal, kv_staging), int(zero_padded_queries), _native.dtype_code(q.dtype),
        _native.current_stream(q.device),
    )
    _native.check(status, "flash_attention")
    return out


def _mask_flags(is_causal: bool, kv_staging: str) -> int:
    if kv_staging not in ("direct", "registers"):
        raise ValueError(f"flash_attention kv_staging must be 'direct' or 'registers', got {kv_staging!r}")
    return (_native.ATTN_CAUSAL if is_causal else 0) | (_native.ATTN_REGISTER_STAGING if kv_staging == "registers" else 0)


def _dense_like(t: torch.Tensor) -> torch.Tensor:
    out = torch.empty_like(t)
    if out.stride(-1) != 1 or any(s % 8 for s in out.stride()[:-1]):
        out = torch.empty(t.shape, dtype=t.dtype, device=t.device)
    return out


def build_dropout_mask(q: torch.Tensor, k: torch.Tensor, dropout_p: float) -> torch.Tensor:
    """uint8 keep mask (B, H, Tq, Tk) drawn as the reference's ``_build_tilelang_dropout_mask`` does
    (attention/flash_attention.py:316-325): ``rand >= p``."""
    if not 0.0 < dropout_p < 1.0:
        raise RuntimeError("hip flash_attention requires dropout_p to be in [0, 1)")
    return (torch.rand((q.shape[0], q.shape[1], q.shape[2], k.shape[2]), device=q.device) >= dropout_p).to(torch.uint8).contiguous()


class _HipFlashAttentionFunction(torch.autograd.Function):
    """Training path (key-length mask, optional causal triangle, optional dropout with a caller-supplied keep mask): the
    forward also saves the log-sum-exp of every query row, the backward runs the two HIP backward kernels (the role of
    the reference's TileLang training functions, flash_attention.py:397-525, 575-650)."""

    @staticmethod
    def forward(ctx, q, k, v, key_lengths, is_causal: bool, zero_padded_queries: bool, kv_staging: str = "direct",
                dropout_mask: torch.Tensor | None = None, dropout_p: float = 0.0):
        library = _native.load_library()
        q, k, v = _kernel_view(q), _kernel_view(k), _kernel_view(v)
        out = _dense_like(q)
        batch, heads, query_len, head_dim = q.shape
        lse = torch.empty(batch, heads, query_len, dtype=torch.float32, device=q.device)
        shape = (batch, heads, query_len, k.shape[2], head_dim)
        strides = (_native.Int64x4(*q.stride()), _native.Int64x4(*k.stride()), _native.Int64x4(*v.stride()),
                   _native.Int64x4(*out.stride()))
        tail = (_mask_flags(is_causal, kv_staging), int(bool(zero_padded_queries)), _native.dtype_code(q.dtype),
                _native.current_stream(q.device))
        scale = 1.0
        if dropout_mask is not None:
            if dropout_mask.dtype != torch.uint8 or tuple(dropout_mask.shape) != (batch, heads, query_len, k.shape[2]):
                raise ValueError("flash_attention dropout_mask must be uint8 of shape (B, H, Tq, Tk)")
            require_cuda_tensors("hip flash_attention", dropout_mask)
            dropout_mask = dropout_mask.contiguous()
            scale = 1.0 / (1.0 - dropout_p)
            status = library.taac_flash_attn_train_dropout_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), _native.ptr(key_lengths), dropout_mask.data_ptr(),
                ctypes.c_float(scale), out.data_ptr(), lse.data_ptr(), *shape, *strides, *tail)
        else:
            status = library.taac_flash_attn_train_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), _native.ptr(key_lengths), out.data_ptr(), lse.data_ptr(),
                *shape, *strides, *tail)
        _native.check(status, "flash_attention")
        saved = [q, k, v, out, lse]
        ctx.has_lengths = key_lengths is not None
        ctx.has_dropout = dropout_mask is not None
        if ctx.has_lengths:
            saved.append(key_lengths)
        if ctx.has_dropout:
            saved.append(dropout_mask)
        ctx.save_for_backward(*saved)
        ctx.dropout_scale = scale
        ctx.flags = (_mask_flags(is_causal, kv_staging), bool(zero_padded_queries))
        return out

    @staticmethod
    def backward(ctx, grad_out):
        library = _native.load_library()
        saved = list(ctx.saved_tensors)
        q, k, v, out, lse = saved[:5]
        rest = saved[5:]
        key_lengths = rest.pop(0) if ctx.has_lengths else None
        dropout_mask = rest.pop(0) if ctx.has_dropout else None
        grad_out = _kernel_view(grad_out)
        dq, dk, dv = _dense_like(q), _dense_like(k), _dense_like(v)
        delta = torch.empty_like(lse)
        batch, heads, query_len, head_dim = q.shape
        strides = [_native.Int64x4(*t.stride()) for t in (q, k, v, out, grad_out, dq, dk, dv)]
        head = (q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), grad_out.data_ptr(), lse.data_ptr(),
                _native.ptr(key_lengths))
        tail = (dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), delta.data_ptr(), batch, heads, query_len, k.shape[2],
                head_dim, *strides, int(ctx.flags[0]), int(ctx.flags[1]), _native.dtype_code(q.dtype),
                _native.current_stream(q.device))
        if dropout_mask is not None:
            status = library.taac_flash_attn_dropout_bwd(*head, dropout_mask.data_ptr(), ctypes.c_float(ctx.dropout_scale),
                                                         *tail)
        else:
            status = library.taac_flash_attn_bwd(*head, *tail)
        _native.check(status, "flash_attention backward")
        return dq, dk, dv, None, None, None, None, None, None


def masked_attention_backward(q, k, v, out, grad_out, lse, key_lengths, mask: StructuredAttentionMask, dq, dk, dv, *,
                              zero_padded_queries: bool = False, dropout_mask: torch.Tensor | None = None,
                              dropout_scale: float = 1.0, self_factor: torch.Tensor | None = None) -> None:
    """``taac_flash_attn_bits_bwd`` for (B, H, T, d) views under a structured mask (either layout: one structure for the
    batch, or one per sample with the valid tokens in front), writing into ``dq`` / ``dk`` / ``dv`` (any element strides
    with a unit last one). A self-only query returned its own value row: its row is taken out of the kernels
    (log-sum-exp +inf: zero probabilities) and ``grad_out`` of that row is added to ``dv``."""
    library = _native.load_library()
    batch, heads, query_len, head_dim = q.shape
    if mask.query_self is not None:
        lse = torch.where(mask.query_self[:, None, :], torch.full_like(lse, float("inf")), lse)
    delta = torch.empty_like(lse)
    strides = [_native.Int64x4(*t.stride()) for t in (q, k, v, out, grad_out, dq, dk, dv)]
    status = library.taac_flash_attn_bits_bwd(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), grad_out.data_ptr(), lse.data_ptr(),
        _native.ptr(key_lengths), mask.struct_bits.data_ptr(), int(mask.sample_stride), _native.ptr(mask.valid_bits),
        _native.ptr(dropout_mask), ctypes.c_float(dropout_scale), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
        delta.data_ptr(), batch, heads, query_len, k.shape[2], head_dim,
        *strides, int(bool(zero_padded_queries)), _native.dtype_code(q.dtype), _native.current_stream(q.device))
    _native.check(status, "flash_attention backward")
    if mask.query_self is not None:  # ``self_factor`` (B, H, T): keep / (1 - p) of the row's own key under dropout
        factor = mask.query_self[:, None, :, None].to(grad_out.dtype) if self_factor is None else self_factor[..., None]
        dv.add_(grad_out * factor)


class _HipMaskedAttentionFunction(torch.autograd.Function):
    """Training path under a :class:`StructuredAttentionMask` (either layout), optionally with dropout under a keep mask:
    the structured forward kernel also saves the log-sum-exp; the backward kernels read the mask in the same bit form.
    What torch autograd derives for SDPA under the reference models' bool masks, which the reference's accelerated path
    rejects (flash_attention.py:183-209)."""

    @staticmethod
    def forward(ctx, q, k, v, key_lengths, mask: StructuredAttentionMask, zero_padded_queries: bool,
                dropout_mask: torch.Tensor | None = None, dropout_p: float = 0.0):
        library = _native.load_library()
        q, k, v = _kernel_view(q), _kernel_view(k), _kernel_view(v)
        out = _dense_like(q)
        batch, heads, query_len, head_dim = q.shape
        if mask.structural.shape != (query_len, k.shape[2]) \
                or (mask.key_valid is not None and mask.key_valid.shape[0] != batch) \
                or (mask.query_self is not None and mask.query_self.shape[0] != batch) \
                or (mask.sample_stride and mask.struct_bits.shape[0] != batch * query_len):
            raise ValueError("flash_attention: the structured mask does not match (batch, query_len, kv_len)")
        require_cuda_tensors("hip flash_attention", q, k, v, mask.struct_bits)
        scale = 1.0
        self_bits, self_factor = mask.self_bits, None
        if dropout_mask is not None:
            if dropout_mask.dtype != torch.uint8 or tuple(dropout_mask.shape) != (batch, heads, query_len, k.shape[2]):
                raise ValueError("flash_attention dropout_mask must be uint8 of shape (B, H, Tq, Tk)")
            require_cuda_tensors("hip flash_attention", dropout_mask)
            dropout_mask = dropout_mask.contiguous()
            scale = 1.0 / (1.0 - dropout_p)
            if mask.query_self is not None:
                # A self-only query has probability 1 on its own key, which dropout keeps or drops like any other: its
                # output is keep[i, i] / (1 - p) * v[i]. The kernels run without the self rows (whatever they compute
                # for them is replaced here, and the backward takes the rows out through their log-sum-exp).
                self_bits = None
                diagonal = torch.diagonal(dropout_mask, dim1=-2, dim2=-1).to(v.dtype) * scale        # (B, H, T)
                self_factor = diagonal * mask.query_self[:, None, :].to(v.dtype)
        lse = torch.empty(batch, heads, query_len, dtype=torch.float32, device=q.device)
        status = library.taac_flash_attn_masked_train_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), _native.ptr(key_lengths), mask.struct_bits.data_ptr(),
            int(mask.sample_stride), _native.ptr(mask.block_any), _native.ptr(mask.valid_bits), _native.ptr(self_bits),
            _native.ptr(dropout_mask), ctypes.c_float(scale), out.data_ptr(),
            lse.data_ptr(), batch, heads, query_len, k.shape[2], head_dim, _native.Int64x4(*q.stride()),
            _native.Int64x4(*k.stride()), _native.Int64x4(*v.stride()), _native.Int64x4(*out.stride()),
            int(bool(zero_padded_queries)), _native.dtype_code(q.dtype), _native.current_stream(q.device))
        _native.check(status, "flash_attention")
        if self_factor is not None:
            out = torch.where(mask.query_self[:, None, :, None], v * self_factor[..., None], out)
        # optional tensors travel through save_for_backward as well (in-place version checks, saved-tensor hooks, and the
        # (B, H, Tq, Tk) keep mask is released with the graph); `present` records which of them follow the fixed five
        optional = (key_lengths, dropout_mask, self_factor)
        ctx.save_for_backward(q, k, v, out, lse, *(t for t in optional if t is not None))
        ctx.present = tuple(t is not None for t in optional)
        ctx.mask, ctx.zero_padded_queries, ctx.dropout_scale = mask, bool(zero_padded_queries), scale
        return out

    @staticmethod
    def backward(ctx, grad_out):
        q, k, v, out, lse, *rest = ctx.saved_tensors
        rest = iter(rest)
        key_lengths, dropout_mask, self_factor = (next(rest) if here else None for here in ctx.present)
        grad_out = _kernel_view(grad_out)
        dq, dk, dv = _dense_like(q), _dense_like(k), _dense_like(v)
        masked_attention_backward(q, k, v, out, grad_out, lse, key_lengths, ctx.mask, dq, dk, dv,
                                  zero_padded_queries=ctx.zero_padded_queries, dropout_mask=dropout_mask,
                                  dropout_scale=ctx.dropout_scale, self_factor=self_factor)
        return dq, dk, dv, None, None, None, None, None


def flash_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    *,
    backend: str = "hip",
    attn_mask: torch.Tensor | None = None,
    dropout_p: float = 0.0,
    training: bool = False,
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
    kv_staging: str = "direct",
    dropout_mask: torch.Tensor | None = None,
) -> torch.Tensor:
    """``softmax(q k^T / sqrt(d) + mask) v`` for (B, H, T, d) tensors.

    ``dropout_p`` with ``training=True`` drops attention probabilities as the reference's training kernels do: a uint8
    keep mask (B, H, Tq, Tk) - ``dropout_mask`` if given, else drawn by :func:`build_dropout_mask` - multiplies the
    probabilities by ``keep / (1 - p)`` behind the softmax normaliser (flash_attention.py:316-325, 575-650).

    ``attn_mask`` is a bool mask with True = attend (structured as described in :func:`plan_flash_attention_mask`);
    ``key_lengths`` (int32 [B]) states the valid key prefix directly and excludes ``attn_mask``.
    fp32 inputs are computed in bf16 and returned as fp32, as the reference's accelerated path does
    (flash_attention.py:249-252, 300-309). ``block_m`` .. ``threads`` are TileLang launch hints, accepted and ignored.
    With ``zero_padded_queries`` the query rows at or beyond ``key_lengths[b]`` are returned as zeros; otherwise they
    attend to the valid keys like every other row (the behaviour of the reference's torch and TileLang paths).
    ``q_row_scale`` / ``k_row_scale`` / ``q_col_scale``: optional float32 factors of the query / key rows and of the
    query features, see :func:`hip_flash_attention_kernel`. ``structured_mask``: a :class:`StructuredAttentionMask`
    instead of ``attn_mask``; an ``attn_mask`` that is neither a key-prefix nor a causal-valid mask is factored into one
    by :func:`plan_structured_attention_mask` (the reference's accelerated path rejects such masks). ``kv_staging``:
    see :func:`hip_flash_attention_kernel`.
    """
    del block_m, block_n, num_stages, threads
    q, k, v = _normalize_flash_attention_inputs(q, k, v)
    _resolve_flash_attention_backend(q, backend, dropout_p=dropout_p, training=training)
    needs_grad = torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v))
    use_dropout = training and dropout_p > 0.0
    if use_dropout and (q_row_scale is not None or k_row_scale is not None or q_col_scale is not None):
        raise RuntimeError("hip flash_attention dropout does not come with row factors")
    if needs_grad and (q_row_scale is not None or k_row_scale is not None or q_col_scale is not None
                       or q.dtype == torch.float32):
        raise RuntimeError("hip flash_attention backward covers bf16 / fp16 inputs without row factors; call it under "
                           "torch.no_grad() for row factors or fp32 inputs")
    if structured_mask is not None and attn_mask is not None:
        raise ValueError("flash_attention takes either attn_mask or structured_mask, not both")
    if key_lengths is not None:
        if attn_mask is not None:
            raise ValueError("flash_attention takes either attn_mask or key_lengths, not both")
        plan = FlashAttentionMaskPlan(key_lengths, None, is_causal)
    elif structured_mask is not None:
        plan = FlashAttentionMaskPlan(None, None, is_causal)
    else:
        try:
            plan = plan_flash_attention_mask(q, k, attn_mask, is_causal=is_causal)
        except RuntimeError:
            if attn_mask is None or attn_mask.dtype is not torch.bool or attn_mask.ndim != 4 or is_causal:
                raise
            structured_mask = plan_structured_attention_mask(q, k, attn_mask)
            plan = FlashAttentionMaskPlan(None, None, False)
    output_dtype = v.dtype
    if q.dtype == torch.float32:
        q, k, v = q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)
    lengths = plan.key_lengths if (plan.key_lengths is not None and (attn_mask is not None or key_lengths is not None)) else None
    if needs_grad or use_dropout:
        if lengths is not None:
            lengths = lengths.to(torch.int32).contiguous()
        mask = None
        if use_dropout:
            mask = dropout_mask if dropout_mask is not None else build_dropout_mask(q, k, dropout_p)
        if structured_mask is not None:
            output = _HipMaskedAttentionFunction.apply(q, k, v, lengths, structured_mask, zero_padded_queries, mask,
                                                       float(dropout_p) if use_dropout else 0.0)
            return output if output.dtype == output_dtype else output.to(output_dtype)
        output = _HipFlashAttentionFunction.apply(q, k, v, lengths, plan.is_causal, zero_padded_queries, kv_staging, mask,
                                                  float(dropout_p) if use_dropout else 0.0)
        if plan.query_self_mask is not None:
            output = torch.where(plan.query_self_mask[:, None, :, None], v, output)
        return output if output.dtype == output_dtype else output.to(output_dtype)
    output = hip_flash_attention_kernel(
        q, k, v, lengths, is_causal=plan.is_causal, zero_padded_queries=zero_padded_queries,
        q_row_scale=q_row_scale, k_row_scale=k_row_scale, q_col_scale=q_col_scale, structured_mask=structured_mask,
        kv_staging=kv_staging,
    )
    output = _apply_query_self_mask_fallback(output, v, plan.query_self_mask)
    return output if output.dtype == output_dtype else output.to(output_dtype)


# ---- query / key preparation: RMSNorm over the model width + rotary embedding ----------------------------------------

_ROPE_TABLES: dict[tuple, torch.Tensor] = {}


def rope_table(token_count: int, head_dim: int, rope_base: float, dtype: torch.dtype, device: torch.device, *,
               inverse: bool = False) -> torch.Tensor:
    """``[tokens, head_dim / 2, 2]`` table of (cos, sin) of ``position * rope_base ** (-2i / head_dim)``, computed in
    float32 and rounded to the activation dtype as ``BFTSAttention._apply_rope`` does
    (experiments/tokenformer/model.py:174-179); cached per shape, base, dtype and device. ``inverse``: (cos, -sin), the
    rotation by the opposite angles - the transpose of the rotation, which is what its backward applies."""
    if head_dim % 2 != 0:
        raise ValueError("hip qk_norm_rope rotates whole heads: head_dim must be even")
    key = (int(token_count), int(head_dim), float(rope_base), dtype, str(device), bool(inverse))
    table = _ROPE_TABLES.get(key)
    if table is None:
        positions = torch.arange(token_count, dtype=torch.float32)
        frequencies = torch.arange(0, head_dim, 2, dtype=torch.float32)
        inv_freq = torch.pow(torch.tensor(float(rope_base)), -frequencies / max(1, head_dim))
        angles = positions[:, None] * inv_freq[None, :]
        sin = angles.sin().to(dtype)
        table = torch.stack((angles.cos().to(dtype), -sin if inverse else sin), dim=-1).contiguous().to(device)
        _ROPE_TABLES[key] = table
    return table


def _row_stride(name: str, t: torch.Tensor) -> int | None:
    """Row stride (elements) when the (..., D) tensor is a uniform stack of contiguous rows, else None."""
    if t.stride(-1) != 1:
        return None
    for dim in range(t.ndim - 2):
        if t.shape[dim] != 1 and t.stride(dim) != t.stride(dim + 1) * t.shape[dim + 1]:
            return None
    return int(t.stride(-2))


def qk_norm_rope(
    query: torch.Tensor,
    key: torch.Tensor,
    query_weight: torch.Tensor | None,
    key_weight: torch.Tensor | None,
    *,
    num_heads: int,
    eps: float = 1e-6,
    rope_base: float | None = None,
    token_rows: tuple[torch.Tensor, torch.Tensor] | None = None,
    inplace: bool = False,
    inverse_rotation: bool = False,
) -> tuple[torch.Tensor, torch.Tensor]:
    """What the reference's attention layers do to the query and key projections before attention, in one pass:
    ``RMSNorm(d_model)`` of each (experiments/symbiosis/backbone.py:33-36) and, with ``rope_base``, the rotary embedding
    over the token positions (experiments/tokenformer/model.py:165-192). ``query`` / ``key``: (batch, tokens, d_model),
    possibly the ``chunk(3, -1)`` views of a packed projection (rows are read with their stride). ``inplace`` writes the
    result over the inputs. ``token_rows`` (:func:`valid_rows`) restricts the pass to the valid tokens; the other rows
    of the result are then zero (new tensors) or untouched (in place). Tensors that require a gradient take the
    differentiable route :func:`qk_norm_rope_autograd`. ``inverse_rotation`` rotates by the opposite angles."""
    name = "hip qk_norm_rope"
    if query.ndim != 3 or key.shape != query.shape:
        raise ValueError("qk_norm_rope expects query and key of the same shape (batch, tokens, d_model)")
    require_same_dtype("qk_norm_rope", query, key)
    require_cuda_tensors(name, query, key)
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (query, key, query_weight, key_weight)):
        if token_rows is not None or inplace or inverse_rotation:
            raise RuntimeError(f"{name}: token_rows / inplace belong to the inference route; call it under "
                               "torch.no_grad() or pass plain tensors when a gradient is needed")
        return qk_norm_rope_autograd(query, key, query_weight, key_weight, num_heads=num_heads, eps=eps, rope_base=rope_base)
    batch, tokens, d_model = query.shape
    if d_model % int(num_heads) != 0:
        raise ValueError("d_model must be divisible by num_heads")
    if (query_weight is None) != (key_weight is None):
        raise ValueError("qk_norm_rope takes both norm weights or neither")
    if query_weight is None and rope_base is None:
        raise ValueError("qk_norm_rope needs norm weights, a rope_base, or both")
    weights = []
    for weight in (query_weight, key_weight):
        if weight is None:
            weights.append(None)
            continue
        if weight.ndim != 1 or weight.shape[0] != d_model:
            raise ValueError("rms_norm weight must be 1D and match the normalized dimension")
        require_cuda_tensors(name, weight)
        weights.append(weight.detach().to(dtype=query.dtype).contiguous())
    table = None
    if rope_base is not None:
        table = rope_table(tokens, d_model // int(num_heads), rope_base, query.dtype, query.device, inverse=inverse_rotation)
    strides = (_row_stride(name, query), _row_stride(name, key))
    if strides[0] is None or strides[0] != strides[1]:
        if inplace:
            raise ValueError(f"{name}: in-place operation needs query and key with one common uniform row stride")
        query, key = query.contiguous(), key.contiguous()
        strides = (d_model, d_model)
    index, count = (None, None)
    if token_rows is not None:
        index, count = token_rows
        require_cuda_tensors(name, index, count)
        if index.dtype != torch.int32 or count.dtype != torch.int32 or count.numel() != 1 or index.numel() < batch * tokens:
            raise ValueError(f"{name}: token_rows must be (int32 row index, int32 scalar count) as returned by valid_rows")
    if inplace:
        query_out, key_out, ld_out = query, key, strides[0]
    else:
        make = torch.zeros if token_rows is not None else torch.empty
        query_out = make((batch, tokens, d_model), dtype=query.dtype, device=query.device)
        key_out = make((batch, tokens, d_model), dtype=query.dtype, device=query.device)
        ld_out = d_model
    library = _native.load_library()
    status = library.taac_qk_norm_rope_fwd(
        query.data_ptr(), key.data_ptr(), strides[0], query_out.data_ptr(), key_out.data_ptr(), ld_out, batch * tokens,
        tokens, d_model, int(num_heads), _native.ptr(weights[0]), _native.ptr(weights[1]), float(eps), _native.ptr(table),
        _native.ptr(index), _native.ptr(count), _native.dtype_code(query.dtype), _native.current_stream(query.device),
    )
    _native.check(status, "qk_norm_rope")
    return query_out, key_out


class _RotaryFunction(torch.autograd.Function):
    """The rotary embedding of query and key as one pass of the preparation kernel; the backward is the same pass with
    the opposite angles (a rotation's transpose), applied to the incoming gradients."""

    @staticmethod
    def forward(ctx, query, key, num_heads: int, rope_base: float):
        ctx.config = (int(num_heads), float(rope_base), query.shape, key.shape, query.dtype, query.device)
        with torch.no_grad():
            return qk_norm_rope(query.detach(), key.detach(), None, None, num_heads=num_heads, rope_base=rope_base)

    @staticmethod
    def backward(ctx, grad_query, grad_key):
        num_heads, rope_base, query_shape, key_shape, dtype, device = ctx.config
        if grad_query is None and grad_key is None:
            return None, None, None, None
        # only one of the two outputs fed the loss: the pass rotates both, so the other one's gradient enters as zeros
        has_query, has_key = grad_query is not None, grad_key is not None
        if not has_query:
            grad_query = torch.zeros(query_shape, dtype=dtype, device=device)
        if not has_key:
            grad_key = torch.zeros(key_shape, dtype=dtype, device=device)
        with torch.no_grad():
            grad_query, grad_key = qk_norm_rope(grad_query.contiguous(), grad_key.contiguous(), None, None, num_heads=num_heads,
                                                rope_base=rope_base, inverse_rotation=True)
        return (grad_query if has_query else None), (grad_key if has_key else None), None, None


def qk_norm_rope_autograd(query: torch.Tensor, key: torch.Tensor, query_weight: torch.Tensor | None,
                          key_weight: torch.Tensor | None, *, num_heads: int, eps: float = 1e-6,
                          rope_base: float | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """:func:`qk_norm_rope` for tensors that take a gradient, as two differentiable steps the way the reference's layers
    run them (experiments/symbiosis/backbone.py:33-36, experiments/tokenformer/model.py:149-154): ``RMSNorm(d_model)`` of
    the query and of the key through the norm kernels and their backward, then the rotation (its backward is the
    rotation by the opposite angles)."""
    from taac_2026_amd.accelerators.normalization import rms_norm

    if (query_weight is None) != (key_weight is None):
        raise ValueError("qk_norm_rope takes both norm weights or neither")
    if query_weight is not None:
        query = rms_norm(query.contiguous(), query_weight, eps)
        key = rms_norm(key.contiguous(), key_weight, eps)
    if rope_base is not None:
        query, key = _RotaryFunction.apply(query, key, int(num_heads), float(rope_base))
    return query, key


__all__ = [
    "FLASH_ATTENTION_BACKENDS",
    "FlashAttentionMaskPlan",
    "StructuredAttentionMask",
    "_plan_tilelang_flash_attention_mask",
    "build_structured_mask",
    "flash_attention",
    "hip_flash_attention_kernel",
    "plan_flash_attention_mask",
    "plan_structured_attention_mask",
    "qk_norm_rope",
    "qk_norm_rope_autograd",
    "resolved_flash_attention_backend",
    "rope_table",
]
