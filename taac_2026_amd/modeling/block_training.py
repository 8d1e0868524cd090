"""Training route of ``UnifiedInteractionBlock`` (experiments/symbiosis/backbone.py:51-68) under prefix padding (key
lengths) or under a structured mask built from the padding mask (scattered padding, e.g. the role mask of
experiments/symbiosis/attention.py:21-60): one autograd function for the whole block whose forward and backward run over
the VALID tokens only.

The reference multiplies both residual updates by ``~padding_mask``, so a padded position passes its input through and
contributes nothing to any weight gradient. The function therefore gathers the valid rows of the token stream once
into a compact ``[valid, D]`` tensor and runs every dense layer, norm and weight gradient on compact tensors; only the
attention kernels see the padded ``[B, T, .]`` layout, which the projections on either side of them write and read
through the row index of :func:`valid_rows` (no copy). At the benchmark's lengths (54 % of the positions valid) the dense
forward and backward kernels do 54 % of the work of the layer-by-layer route, the packed q | k | v gradient is written
in place (no concatenation) and the mask multiplications and residual adds of autograd disappear.

The number of valid rows sizes the compact tensors, so it is read back from the device once per ``key_lengths`` tensor
or mask object (one host synchronisation, shared by the blocks of a stack).
"""

from __future__ import annotations

import ctypes
import importlib
import weakref

import torch

from taac_2026_amd import _native

# the package re-exports a function of the same name, which shadows the module as an attribute
_linear = importlib.import_module("taac_2026_amd.accelerators.linear")
from taac_2026_amd.accelerators.normalization import hip_rms_norm_backward_kernel, hip_rms_norm_kernel


class _RowIndex:
    """Valid-row index of a ``key_lengths`` tensor: ``rows`` (int32, :func:`valid_rows`) and ``count`` (device scalar) at
    once; ``compact()`` adds what the backward needs and what costs the host synchronisation: ``valid`` (the count on the
    host) and ``identity`` (int32 ``0..valid-1``: the row numbers of a compact tensor). The index of the last tensor seen
    is kept, so the blocks of a stack share it."""

    _last: tuple | None = None

    def __init__(self, key_lengths: torch.Tensor, tokens: int) -> None:
        self.rows, self.count = _linear.valid_rows(key_lengths, tokens)
        self.valid: int | None = None
        self.identity = None

    def compact(self) -> "_RowIndex":
        if self.valid is None:
            self.valid = int(self.count.item())
            self.identity = torch.arange(max(self.valid, 1), dtype=torch.int32, device=self.rows.device)
        return self

    @classmethod
    def for_mask(cls, mask, padding_mask: torch.Tensor, tokens: int) -> "_RowIndex":
        """Index of the positions ``~padding_mask`` (any pattern), kept on the mask object the blocks of a stack share;
        ``bits``: the same validity as packed words, for ``taac_rows_merge_bits``."""
        entry = mask.cache.get("training_rows")
        if entry is None or entry[0] != padding_mask._version:
            from taac_2026_amd.accelerators.attention import _pack_bits

            from taac_2026_amd.accelerators.attention import front_structured_mask

            index = cls.__new__(cls)
            index.rows, index.count = _linear.valid_rows(None, tokens, padding_mask=padding_mask)
            index.bits = _pack_bits((~padding_mask).contiguous())
            # valid tokens in the 32-token words before each word: the rank of a position without a walk over the words
            words = index.bits.shape[1]
            per_word = torch.nn.functional.pad(~padding_mask, (0, words * 32 - tokens)).view(-1, words, 32).sum(-1)
            index.word_prefix = (per_word.cumsum(1) - per_word).to(torch.int32).contiguous()
            index.valid = None
            index.identity = None
            # Without self-only queries the attention side runs in the layout that has every sample's valid tokens at the
            # front of its rows (prefix padding: its cost follows the valid tokens), under the structure gathered per sample.
            index.front = index.lengths = index.front_mask = None
            if mask.query_self is None:
                batch = padding_mask.shape[0]
                index.front, index.lengths = _linear.front_rows((index.rows, index.count), batch, tokens)
                index.front_mask = front_structured_mask(mask, (index.rows, index.count), batch)
            entry = mask.cache["training_rows"] = (padding_mask._version, index)
        return entry[1]

    @classmethod
    def get(cls, key_lengths: torch.Tensor, tokens: int) -> "_RowIndex":
        stamp = cls._last
        if stamp is not None:
            ref, version, pointer, width, entry = stamp
            if ref() is key_lengths and version == key_lengths._version and pointer == key_lengths.data_ptr() and width == tokens:
                return entry
        entry = cls(key_lengths, tokens)
        cls._last = (weakref.ref(key_lengths), key_lengths._version, key_lengths.data_ptr(), tokens, entry)
        return entry


def _indexed_linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor, *, tokens: int,
                    out_rows: torch.Tensor, count: torch.Tensor, x_rows: torch.Tensor | None, norm_weight: torch.Tensor | None = None,
                    eps: float = 1e-6, residual: torch.Tensor | None = None, cache_weight: bool = True) -> None:
    """``out[out_rows[i]] = residual[out_rows[i]] + linear(rmsnorm(x[x_rows[i]]))`` for ``i < min(tokens, count)``
    (``taac_norm_linear_fwd`` with its row indices; ``x_rows`` None: the rows of ``x`` are ``out_rows`` too): a projection
    over the valid rows of the padded layout, or one that crosses between the compact and the padded layout."""
    out_features, in_features = weight.shape
    packed = _linear._packed_linear(weight, norm_weight) if cache_weight else _linear.pack_linear_weight(weight, norm_weight)
    library = _native.load_library()
    status = library.taac_norm_linear_fwd(
        x.data_ptr(), x.stride(0), _native.ptr(norm_weight), float(eps), None, _native.ptr(bias), packed.data_ptr(),
        _native.ptr(residual), residual.stride(0) if residual is not None else out_features, out.data_ptr(), out.stride(0),
        tokens, out_features, in_features, out_rows.data_ptr(), count.data_ptr(), _native.ptr(x_rows),
        int(norm_weight is not None), _native.current_stream(x.device))
    _native.check(status, "interaction block (training): projection")


def _gather_rows(src: torch.Tensor, index: "_RowIndex", rows: torch.Tensor | None = None) -> torch.Tensor:
    """The valid rows of a padded ``[B * T, W]`` tensor as a compact ``[valid, W]`` one (``taac_rows_gather``); ``rows``:
    where the valid tokens lie when that is not their position (the front layout of the attention side)."""
    out = torch.empty(index.valid, src.shape[1], dtype=src.dtype, device=src.device)
    rows = index.rows if rows is None else rows
    status = _native.load_library().taac_rows_gather(src.data_ptr(), src.stride(0), rows.data_ptr(), index.valid,
                                                     out.data_ptr(), src.shape[1], _native.current_stream(src.device))
    _native.check(status, "interaction block (training): gather")
    return out


def _attention_strides(width: int, heads: int, row_stride: int, tokens: int):
    """Element strides of a logical (B, H, T, d) view of ``[B * T, row_stride]`` rows whose heads lie side by side."""
    return _native.Int64x4(tokens * row_stride, width // heads, row_stride, 1)


class InteractionBlockFunction(torch.autograd.Function):
    """``UnifiedInteractionBlock.forward`` (with or without the query / key norms) without rotary embedding or dropout,
    under key lengths (``mask`` None) or under a structured mask whose key validity comes from ``padding_mask`` (``key_lengths``
    None). Inputs: tokens ``[B, T, D]`` bf16, ``key_lengths`` int32 ``[B]`` or None, the mask and its padding mask or None,
    then the block's parameters. Returns ``(output, attn_tokens)`` like the module (``attn_tokens`` is None unless asked for)."""

    @staticmethod
    def forward(ctx, tokens, key_lengths, mask, padding_mask, want_attn_tokens, num_heads, attn_eps, ffn_eps, gate_first,
                qk_eps, attn_norm_w, w_qkv, b_qkv, w_out, b_out, ffn_norm_w, w_up, b_up, w_down, b_down, query_norm_w,
                key_norm_w):
        batch, token_count, width = tokens.shape
        total = batch * token_count
        index = _RowIndex.get(key_lengths, token_count) if mask is None else _RowIndex.for_mask(mask, padding_mask, token_count)
        rows, count = index.rows, index.count
        flat = tokens.detach().reshape(total, width)
        if not flat.is_contiguous():
            flat = flat.contiguous()
        library = _native.load_library()
        # Layout of the attention side (q | k | v, the attention output and their gradients): the positions (key lengths,
        # or a mask with self-only queries), or the samples' valid tokens in front (any other mask), where the mask's
        # structure is the one gathered per sample and the samples' numbers of valid tokens are the key lengths.
        front = getattr(index, "front", None) if mask is not None else None
        arows = rows if front is None else front
        if front is not None:
            mask, key_lengths = index.front_mask, index.lengths
        # q | k | v of the valid rows. Under key lengths the attention kernels never read a row beyond a sample's length;
        # under a mask over the positions they do (an invisible pair is a zero factor, not a skipped one), so the padded
        # rows hold zeros there.
        in_positions = mask is not None and front is None
        qkv = (torch.zeros if in_positions else torch.empty)(total, 3 * width, dtype=flat.dtype, device=flat.device)
        _indexed_linear(flat, w_qkv, b_qkv, qkv, tokens=total, out_rows=arows, count=count,
                        x_rows=None if front is None else rows, norm_weight=attn_norm_w, eps=attn_eps)
        element = qkv.element_size()
        if query_norm_w is not None:
            # RMSNorm(d_model) of the query and of the key, in place on the valid rows of the packed projection; the
            # backward recomputes the projection for the norms' own backward
            status = library.taac_qk_norm_rope_fwd(
                qkv.data_ptr(), qkv.data_ptr() + width * element, 3 * width, qkv.data_ptr(), qkv.data_ptr() + width * element,
                3 * width, total, token_count, width, int(num_heads), query_norm_w.data_ptr(), key_norm_w.data_ptr(),
                float(qk_eps), None, arows.data_ptr(), count.data_ptr(), _native.dtype_code(flat.dtype),
                _native.current_stream(tokens.device))
            _native.check(status, "interaction block (training): query / key norm")
        attended = torch.empty(total, width, dtype=flat.dtype, device=flat.device)
        lse = torch.empty(batch, num_heads, token_count, dtype=torch.float32, device=flat.device)
        qkv_strides = _attention_strides(width, num_heads, 3 * width, token_count)
        out_strides = _attention_strides(width, num_heads, width, token_count)
        if mask is None:
            status = library.taac_flash_attn_train_fwd(
                qkv.data_ptr(), qkv.data_ptr() + width * element, qkv.data_ptr() + 2 * width * element, key_lengths.data_ptr(),
                attended.data_ptr(), lse.data_ptr(), batch, num_heads, token_count, token_count, width // num_heads,
                qkv_strides, qkv_strides, qkv_strides, out_strides, 0, 1, _native.dtype_code(flat.dtype),
                _native.current_stream(tokens.device))
        else:
            status = library.taac_flash_attn_masked_train_fwd(
                qkv.data_ptr(), qkv.data_ptr() + width * element, qkv.data_ptr() + 2 * width * element,
                _native.ptr(key_lengths), mask.struct_bits.data_ptr(), int(mask.sample_stride), _native.ptr(mask.block_any),
                _native.ptr(mask.valid_bits), _native.ptr(mask.self_bits), None, ctypes.c_float(1.0), attended.data_ptr(),
                lse.data_ptr(), batch, num_heads, token_count, token_count, width // num_heads, qkv_strides, qkv_strides,
                qkv_strides, out_strides, 0 if front is None else 1, _native.dtype_code(flat.dtype),
                _native.current_stream(tokens.device))
        _native.check(status, "interaction block (training): attention")
        # Second half on the valid rows of copies of the stream (padded rows pass through): one kernel when the caller
        # does not want the tokens between the halves, two otherwise.
        attn_tokens = None
        if want_attn_tokens or not gate_first:
            attn_tokens = flat.clone()
            _indexed_linear(attended, w_out, b_out, attn_tokens, tokens=total, out_rows=rows, count=count, x_rows=front,
                            residual=flat)
            output = attn_tokens.clone()
            _linear.swiglu_ffn(attn_tokens, w_up, b_up, w_down, b_down, residual=attn_tokens, gate_first=gate_first,
                               norm_weight=ffn_norm_w, eps=ffn_eps, token_rows=(rows, count), out=output)
        else:
            output = flat.clone()
            _linear.attention_out_ffn(attended, w_out, b_out, flat, w_up, b_up, w_down, b_down, norm_weight=ffn_norm_w,
                                      eps=ffn_eps, token_rows=(rows, count), input_rows=front, out=output)
        ctx.mask, ctx.front = mask, front
        # (a mask over the positions has no key lengths: the slot keeps a tensor it never reads)
        ctx.save_for_backward(flat, qkv, attended, lse, key_lengths if key_lengths is not None else lse, attn_norm_w, w_qkv,
                              w_out, ffn_norm_w, w_up, w_down,
                              *(t for t in (b_out, b_up, attn_tokens, b_qkv if query_norm_w is not None else None,
                                            query_norm_w, key_norm_w) if t is not None))
        ctx.index = index
        ctx.config = (batch, token_count, width, int(num_heads), float(attn_eps), float(ffn_eps), bool(gate_first),
                      b_qkv is not None, b_out is not None, b_up is not None, b_down is not None, attn_tokens is not None,
                      query_norm_w is not None, float(qk_eps))
        ctx.set_materialize_grads(False)
        if attn_tokens is not None:
            attn_tokens = attn_tokens.view(batch, token_count, width) if want_attn_tokens else None
        return output.view(batch, token_count, width), attn_tokens

    @staticmethod
    def backward(ctx, grad_output, grad_attn_tokens):
        (flat, qkv, attended, lse, key_lengths, attn_norm_w, w_qkv, w_out, ffn_norm_w, w_up, w_down, *rest) = ctx.saved_tensors
        (batch, token_count, width, num_heads, attn_eps, ffn_eps, gate_first, has_b_qkv, has_b_out, has_b_up, has_b_down,
         has_attn_tokens, has_qk_norm, qk_eps) = ctx.config
        rest = list(rest)
        b_out = rest.pop(0) if has_b_out else None
        b_up = rest.pop(0) if has_b_up else None
        attn_tokens_saved = rest.pop(0) if has_attn_tokens else None
        b_qkv = rest.pop(0) if (has_qk_norm and has_b_qkv) else None
        query_norm_w, key_norm_w = (rest.pop(0), rest.pop(0)) if has_qk_norm else (None, None)
        index = ctx.index.compact()
        rows, count, valid, identity = index.rows, index.count, index.valid, index.identity
        mask, front = ctx.mask, ctx.front
        arows = rows if front is None else front       # where the attention side keeps the valid tokens
        total = batch * token_count
        dtype, device = flat.dtype, flat.device
        if valid == 0:                              # no valid token: the block is the identity
            grads = [g for g in (grad_output, grad_attn_tokens) if g is not None]
            return (sum(grads[1:], grads[0]) if grads else None,) + (None,) * 21
        # the compact rows of the stream and of the tokens between the halves (gathered, or recomputed from the attention
        # output when the forward ran the one-kernel second half)
        xc = _gather_rows(flat, index)
        if has_attn_tokens:
            x1c = _gather_rows(attn_tokens_saved, index)
        else:
            x1c = torch.empty(valid, width, dtype=dtype, device=device)
            _indexed_linear(attended, w_out, b_out, x1c, tokens=valid, out_rows=identity, count=count, x_rows=arows, residual=xc)

        def flat_grad(g):
            g = g.reshape(total, width)
            return g if g.dtype == dtype and g.is_contiguous() else g.to(dtype).contiguous()

        # gradient arriving at the padded rows (they pass through the block) and, gathered, at the valid ones
        grad_padded = None
        grad_x1c = None
        if grad_attn_tokens is not None:       # the caller used attn_tokens: identity on padded rows, x1 on valid ones
            grad_padded = flat_grad(grad_attn_tokens)
            grad_x1c = _gather_rows(grad_padded, index)
        weight_grads = dict.fromkeys(("up", "b_up", "down", "b_down", "ffn_norm"))
        if grad_output is not None:
            g_out = flat_grad(grad_output)
            grad_padded = g_out if grad_padded is None else grad_padded + g_out
            gc = _gather_rows(g_out, index)                                           # [valid, D]
            # ---- feed-forward half ---------------------------------------------------------------------------------------
            h2 = hip_rms_norm_kernel(x1c, ffn_norm_w, ffn_eps)
            hidden, grad_pre = _linear.swiglu_ffn_backward_hidden(h2, gc, w_up, b_up, w_down, gate_first=gate_first)
            weight_grads["down"], weight_grads["b_down"] = _linear.linear_wgrad(gc, hidden, with_bias=has_b_down)
            weight_grads["up"], weight_grads["b_up"] = _linear.linear_wgrad(grad_pre, h2, with_bias=has_b_up)
            grad_h2 = _linear._input_grad(grad_pre, w_up)
            del hidden, grad_pre
            grad_x1_norm, weight_grads["ffn_norm"] = hip_rms_norm_backward_kernel(x1c, ffn_norm_w, grad_h2, ffn_eps)
            grad_x1c = gc.add_(grad_x1_norm) if grad_x1c is None else grad_x1c.add_(gc).add_(grad_x1_norm)
        if grad_x1c is None:
            return (None,) * 22
        # ---- out projection: weight gradient on compact rows, input gradient written into the padded layout ------------
        attended_c = _gather_rows(attended, index, arows)
        grad_w_out, grad_b_out = _linear.linear_wgrad(grad_x1c, attended_c, with_bias=has_b_out)
        del attended_c
        grad_attended = torch.zeros(total, width, dtype=dtype, device=device)
        _indexed_linear(grad_x1c, w_out.t().contiguous(), None, grad_attended, tokens=valid, out_rows=arows, count=count,
                        x_rows=identity, cache_weight=False)
        # ---- attention: the gradient of the packed q | k | v projection in place ---------------------------------------------
        grad_qkv = torch.empty(total, 3 * width, dtype=dtype, device=device)
        delta = torch.empty_like(lse)
        library = _native.load_library()
        qkv_strides = _attention_strides(width, num_heads, 3 * width, token_count)
        out_strides = _attention_strides(width, num_heads, width, token_count)
        element = qkv.element_size()
        q_ptr, g_ptr = qkv.data_ptr(), grad_qkv.data_ptr()
        if mask is None:
            status = library.taac_flash_attn_bwd(
                q_ptr, q_ptr + width * element, q_ptr + 2 * width * element, attended.data_ptr(), grad_attended.data_ptr(),
                lse.data_ptr(), key_lengths.data_ptr(), g_ptr, g_ptr + width * element, g_ptr + 2 * width * element,
                delta.data_ptr(), batch, num_heads, token_count, token_count, width // num_heads, qkv_strides, qkv_strides,
                qkv_strides, out_strides, out_strides, qkv_strides, qkv_strides, qkv_strides, 0, 1, _native.dtype_code(dtype),
                _native.current_stream(device))
            _native.check(status, "interaction block (training): attention backward")
        else:
            from taac_2026_amd.accelerators.attention import masked_attention_backward

            head_dim = width // num_heads
            heads_of = lambda t, parts: t.view(batch, token_count, parts, num_heads, head_dim).permute(2, 0, 3, 1, 4)  # noqa: E731
            q4, k4, v4 = heads_of(qkv, 3)
            dq4, dk4, dv4 = heads_of(grad_qkv, 3)
            (o4,), (do4,) = heads_of(attended, 1), heads_of(grad_attended, 1)
            # positions: the padded rows of q | k | v are zeros and receive finite values that nobody reads; front layout:
            # the rows beyond a sample's number of valid tokens are never touched
            masked_attention_backward(q4, k4, v4, o4, do4, lse, None if front is None else key_lengths, mask, dq4, dk4, dv4,
                                      zero_padded_queries=front is not None)
        grad_qkv_c = _gather_rows(grad_qkv, index, arows)                             # [valid, 3D]
        del grad_qkv, grad_attended
        grad_query_norm = grad_key_norm = None
        if has_qk_norm:
            # the attention backward produced the gradients of the NORMALISED query and key: the projection's q | k columns
            # are recomputed on the compact rows and each norm's backward runs on contiguous copies of its columns
            qk_pre = torch.empty(valid, 2 * width, dtype=dtype, device=device)
            _indexed_linear(xc, w_qkv[: 2 * width], None if b_qkv is None else b_qkv[: 2 * width], qk_pre, tokens=valid,
                            out_rows=identity, count=count, x_rows=None, norm_weight=attn_norm_w, eps=attn_eps,
                            cache_weight=False)
            norm_grads = []
            for part, norm_w in enumerate((query_norm_w, key_norm_w)):
                columns = slice(part * width, (part + 1) * width)
                grad_part, grad_w = hip_rms_norm_backward_kernel(qk_pre[:, columns].contiguous(), norm_w,
                                                                 grad_qkv_c[:, columns].contiguous(), qk_eps)
                grad_qkv_c[:, columns].copy_(grad_part)
                norm_grads.append(grad_w)
            grad_query_norm, grad_key_norm = norm_grads
            del qk_pre
        # ---- q | k | v projection and its norm ------------------------------------------------------------------------------
        h1 = hip_rms_norm_kernel(xc, attn_norm_w, attn_eps)
        grad_w_qkv, grad_b_qkv = _linear.linear_wgrad(grad_qkv_c, h1, with_bias=has_b_qkv)
        grad_h1 = _linear._input_grad(grad_qkv_c, w_qkv)
        grad_xc_norm, grad_attn_norm = hip_rms_norm_backward_kernel(xc, attn_norm_w, grad_h1, attn_eps)
        # valid rows: the gradient of the tokens between the halves + that of the norm's input; padded rows: what arrived
        grad_tokens = torch.empty(total, width, dtype=dtype, device=device)
        if not hasattr(index, "bits"):
            status = library.taac_rows_merge(grad_padded.data_ptr(), grad_x1c.data_ptr(), grad_xc_norm.data_ptr(),
                                             key_lengths.data_ptr(), rows.data_ptr() + 4 * total, grad_tokens.data_ptr(),
                                             batch, token_count, width, _native.current_stream(device))
        else:
            status = library.taac_rows_merge_bits(grad_padded.data_ptr(), grad_x1c.data_ptr(), grad_xc_norm.data_ptr(),
                                                  ctx.index.bits.data_ptr(), ctx.index.word_prefix.data_ptr(),
                                                  rows.data_ptr() + 4 * total,
                                                  grad_tokens.data_ptr(), batch, token_count, width,
                                                  _native.current_stream(device))
        _native.check(status, "interaction block (training): gradient merge")
        return (grad_tokens.view(batch, token_count, width), None, None, None, None, None, None, None, None, None,
                grad_attn_norm,
                grad_w_qkv, grad_b_qkv, grad_w_out, grad_b_out, weight_grads["ffn_norm"], weight_grads["up"],
                weight_grads["b_up"], weight_grads["down"], weight_grads["b_down"], grad_query_norm, grad_key_norm)


def training_route_applies(block, tokens: torch.Tensor, attention_mask, key_lengths, padding_mask=None) -> bool:
    """Whether :class:`InteractionBlockFunction` covers this call of ``block`` (a ``UnifiedInteractionBlock``): key lengths
    and no mask, or a structured mask (same for every sample apart from key validity) that was built from
    ``padding_mask``, so that no query can see a padded key."""
    from taac_2026_amd.accelerators.attention import StructuredAttentionMask

    if isinstance(attention_mask, StructuredAttentionMask):
        if key_lengths is not None or padding_mask is None or attention_mask.padding_source is not padding_mask:
            return False
        if attention_mask.sample_stride or attention_mask.key_valid is None or tokens.ndim != 3:
            return False
        if attention_mask.structural.shape != (tokens.shape[1], tokens.shape[1]):
            return False
        if padding_mask.dtype is not torch.bool or not padding_mask.is_cuda or padding_mask.shape != tokens.shape[:2]:
            return False
    elif attention_mask is not None or key_lengths is None:
        return False
    if not (tokens.is_cuda and tokens.dtype == torch.bfloat16 and tokens.ndim == 3 and tokens.shape[-1] in (128, 256)):
        return False
    attention, ffn = block.attention, block.ffn
    width = tokens.shape[-1]
    head_dim = width // attention.num_heads
    if attention.rope_base is not None or head_dim not in (32, 64) or width % attention.num_heads:
        return False
    if (attention.query_norm is None) != (attention.key_norm is None):
        return False
    if ffn.down.weight.shape[1] % 32 != 0 or not _linear.swiglu_ffn_backward_supported(width, ffn.down.weight.shape[1]):
        return False  # (the forward kernels take any such F; the backward's hidden-state kernel bounds it)
    if block.training and (attention.dropout > 0.0 or ffn.dropout.p > 0.0):
        return False
    if key_lengths is not None and (key_lengths.dtype != torch.int32 or not key_lengths.is_cuda
                                    or not key_lengths.is_contiguous()):
        return False
    # float32 parameters (master weights of mixed-precision training) are cast to bf16 on the way in, as every route of the
    # module does; autograd carries the gradient back through the cast
    return all(p.dtype in (torch.bfloat16, torch.float32) and p.is_cuda for p in block.parameters())


def run_training_block(block, tokens: torch.Tensor, key_lengths: torch.Tensor | None, return_attention_tokens: bool,
                       mask=None, padding_mask: torch.Tensor | None = None):
    """The block through :class:`InteractionBlockFunction`."""
    attention, ffn = block.attention, block.ffn
    qk_norm = attention.query_norm is not None

    def bf16(parameter):
        return parameter if parameter is None or parameter.dtype == torch.bfloat16 else parameter.to(torch.bfloat16)

    return InteractionBlockFunction.apply(
        tokens, key_lengths, mask, padding_mask, bool(return_attention_tokens), attention.num_heads, block.attn_norm.eps,
        block.ffn_norm.eps, ffn.gate_first, attention.query_norm.eps if qk_norm else 1e-6, bf16(block.attn_norm.weight),
        bf16(attention.qkv.weight), bf16(attention.qkv.bias), bf16(attention.out.weight), bf16(attention.out.bias),
        bf16(block.ffn_norm.weight), bf16(ffn.up.weight), bf16(ffn.up.bias), bf16(ffn.down.weight), bf16(ffn.down.bias),
        bf16(attention.query_norm.weight) if qk_norm else None, bf16(attention.key_norm.weight) if qk_norm else None)
