"""Unified token backbone blocks on the HIP kernels.

``SwiGLUFeedForward`` / ``UnifiedSelfAttention`` / ``BFTSAttention`` / ``UnifiedInteractionBlock`` keep the constructor signatures,
parameter names (``up``, ``down``, ``qkv``, ``out``, ``attn_norm`` ...) and forward semantics of
experiments/symbiosis/backbone.py:11-68 (TokenFormer's feed-forward, experiments/tokenformer/model.py:118-128, is the
same module), with every dense layer, norm and attention call routed to libtaac_hip.so. Dropout probabilities are stored
but only the eval-mode behaviour (identity) exists for the feed-forward dropout; tensors that require grad take the
autograd routes of the operators, and ``UnifiedInteractionBlock`` under prefix padding the one-function training route of
``block_training``.

``PCVRBackbone`` is the canonical pre-norm stack + pCVR readout (mean-pool over valid tokens -> Linear(D, 1) ->
sigmoid) executed by a single ``taac_backbone_fwd`` call.
"""

from __future__ import annotations

import ctypes

import torch
import torch.nn as nn

from taac_2026_amd import _native
from taac_2026_amd.accelerators.attention import StructuredAttentionMask, front_structured_mask, qk_norm_rope, rope_table
from taac_2026_amd.accelerators.linear import (attention_out_ffn, front_rows, norm_linear, qkv_projection, silu_mlp,
                                               swiglu_ffn, swiglu_ffn_backward_supported, swiglu_ffn_dropout, valid_rows)
from taac_2026_amd.accelerators.tensor_validation import require_cuda_tensors, require_inference
from taac_2026_amd.modeling.block_training import run_training_block, training_route_applies
from taac_2026_amd.modeling.normalization import RMSNorm
from taac_2026_amd.modeling.sequence import scaled_dot_product_attention


def _bf16(parameter: torch.Tensor | None) -> torch.Tensor | None:
    if parameter is None:
        return None
    return parameter if parameter.dtype == torch.bfloat16 else parameter.to(torch.bfloat16)


def _compute_dtype(tokens: torch.Tensor) -> torch.dtype:
    """The 16-bit type a layer computes in: float16 tokens stay float16 (tiled kernels, forward only), everything else
    runs in bfloat16."""
    return torch.float16 if tokens.dtype == torch.float16 else torch.bfloat16


def _as(parameter: torch.Tensor | None, dtype: torch.dtype) -> torch.Tensor | None:
    if parameter is None:
        return None
    return parameter if parameter.dtype == dtype else parameter.to(dtype)


def _dense(layer: nn.Linear, x: torch.Tensor, *, residual: torch.Tensor | None = None) -> torch.Tensor:
    return norm_linear(x, _as(layer.weight, x.dtype), _as(layer.bias, x.dtype), residual=residual)


class SwiGLUFeedForward(nn.Module):
    """``down(silu(gate) * value)``, ``gate, value = up(x).chunk(2, -1)``: one fused kernel for model widths 128 / 256
    (the projection and the gated hidden state stay in registers), up(+SiLU-gate) and down kernels otherwise."""

    def __init__(self, d_model: int, hidden_mult: int, dropout: float = 0.0, *, gate_first: bool = True) -> None:
        super().__init__()
        hidden_dim = int(d_model) * int(hidden_mult)
        self.up = nn.Linear(d_model, hidden_dim * 2)
        self.dropout = nn.Dropout(dropout)
        self.down = nn.Linear(hidden_dim, d_model)
        self.gate_first = bool(gate_first)

    def forward(self, tokens: torch.Tensor, *, residual: torch.Tensor | None = None) -> torch.Tensor:
        output_dtype = tokens.dtype
        dtype = _compute_dtype(tokens)
        x = _as(tokens, dtype)
        if self.training and self.dropout.p > 0.0:
            # dropout of the hidden state (experiments/symbiosis/backbone.py:19-21): the hidden state reaches memory
            out = swiglu_ffn_dropout(x, _as(self.up.weight, dtype), _as(self.up.bias, dtype), _as(self.down.weight, dtype),
                                     _as(self.down.bias, dtype), dropout_p=self.dropout.p, residual=_as(residual, dtype),
                                     gate_first=self.gate_first)
            return out if out.dtype == output_dtype else out.to(output_dtype)
        out = swiglu_ffn(x, _as(self.up.weight, dtype), _as(self.up.bias, dtype), _as(self.down.weight, dtype),
                         _as(self.down.bias, dtype), residual=_as(residual, dtype), gate_first=self.gate_first)
        return out if out.dtype == output_dtype else out.to(output_dtype)


class FeedForward(nn.Module):
    """OneTrans' feed-forward (experiments/onetrans/model.py:33-44): ``net = Sequential(Linear(d_model, d_model *
    hidden_mult), SiLU, Dropout, Linear(d_model * hidden_mult, d_model))``, same constructor and parameter names
    (``net.0``, ``net.3``). Under ``torch.no_grad()`` bf16 tokens of width 128 / 256 run as one kernel with the hidden
    state in registers; ``norm_weight`` / ``residual`` additionally fuse the RMSNorm in front and the residual add
    behind (``tokens + ffn(ffn_norm(tokens))`` of ``OneTransBlock.forward``, :107). Training-mode dropout of the hidden
    state runs the two layers as kernels of their own with torch's dropout between them."""

    def __init__(self, d_model: int, hidden_mult: int, dropout: float = 0.0) -> None:
        super().__init__()
        self.net = nn.Sequential(
            nn.Linear(d_model, d_model * hidden_mult),
            nn.SiLU(),
            nn.Dropout(dropout),
            nn.Linear(d_model * hidden_mult, d_model),
        )

    def forward(self, x: torch.Tensor, *, residual: torch.Tensor | None = None, norm_weight: torch.Tensor | None = None,
                eps: float = 1e-6) -> torch.Tensor:
        output_dtype = x.dtype
        dtype = _compute_dtype(x)
        tokens = _as(x, dtype)
        fc1, fc2 = self.net[0], self.net[3]
        if self.training and self.net[2].p > 0.0:
            from taac_2026_amd.accelerators.linear import linear
            from taac_2026_amd.accelerators.normalization import rms_norm

            h = tokens if norm_weight is None else rms_norm(tokens, _as(norm_weight, dtype), eps)
            hidden = self.net[2](torch.nn.functional.silu(linear(h, _as(fc1.weight, dtype), _as(fc1.bias, dtype))))
            out = linear(hidden, _as(fc2.weight, dtype), _as(fc2.bias, dtype), residual=_as(residual, dtype))
        else:
            out = silu_mlp(tokens, _as(fc1.weight, dtype), _as(fc1.bias, dtype), _as(fc2.weight, dtype), _as(fc2.bias, dtype),
                           residual=_as(residual, dtype), norm_weight=_as(norm_weight, dtype), eps=eps)
        return out if out.dtype == output_dtype else out.to(output_dtype)


class MixedFeedForward(nn.Module):
    """OneTrans' mixed feed-forward (experiments/onetrans/model.py:80-94): a shared ``FeedForward`` over every token, and
    for the i-th non-sequence token (position ``seq_token_count + i``) a feed-forward of its own whose output replaces
    the shared one. The token-specific layers read their token as a strided ``[B, D]`` view of the stream."""

    def __init__(self, d_model: int, hidden_mult: int, num_ns_tokens: int, dropout: float = 0.0) -> None:
        super().__init__()
        self.shared = FeedForward(d_model, hidden_mult, dropout)
        self.ns_specific = nn.ModuleList(FeedForward(d_model, hidden_mult, dropout) for _ in range(num_ns_tokens))

    def forward(self, tokens: torch.Tensor, seq_token_count: int) -> torch.Tensor:
        output = self.shared(tokens)
        if not output.requires_grad:
            for ns_index, ffn in enumerate(self.ns_specific):
                position = seq_token_count + ns_index
                if position >= tokens.shape[1]:
                    continue
                output[:, position, :] = ffn(tokens[:, position, :])
            return output
        pieces = []  # under autograd: no in-place writes into a tensor the graph holds
        for ns_index, ffn in enumerate(self.ns_specific):
            position = seq_token_count + ns_index
            if position < tokens.shape[1]:
                pieces.append((position, ffn(tokens[:, position, :])))
        if not pieces:
            return output
        replaced = output.clone()
        for position, value in pieces:
            replaced[:, position, :] = value
        return replaced


class UnifiedSelfAttention(nn.Module):
    """qkv projection -> RMSNorm(d_model) of the query and of the key -> attention -> out projection
    (experiments/symbiosis/backbone.py:24-48). The two norms (and the rotary embedding of the subclass) run as one
    in-place pass over the packed projection."""

    rope_base: float | None = None

    def __init__(self, d_model: int, num_heads: int, dropout: float = 0.0, *, qk_norm: bool = True) -> None:
        super().__init__()
        self.num_heads = int(num_heads)
        self.dropout = float(dropout)
        self.qkv = nn.Linear(d_model, d_model * 3)
        self.query_norm = RMSNorm(d_model) if qk_norm else None
        self.key_norm = RMSNorm(d_model) if qk_norm else None
        self.out = nn.Linear(d_model, d_model)

    def forward(
        self,
        tokens: torch.Tensor,
        attention_mask: torch.Tensor | StructuredAttentionMask | None = None,
        *,
        key_lengths: torch.Tensor | None = None,
        zero_padded_queries: bool = False,
        residual: torch.Tensor | None = None,
    ) -> torch.Tensor:
        output_dtype = tokens.dtype
        dtype = _compute_dtype(tokens)
        x = _as(tokens, dtype)
        prepare = self.query_norm is not None or self.rope_base is not None
        query_weight = None if self.query_norm is None else _as(self.query_norm.weight, dtype)
        key_weight = None if self.key_norm is None else _as(self.key_norm.weight, dtype)
        qk_eps = 1e-6 if self.query_norm is None else self.query_norm.eps
        q_row_scale = k_row_scale = q_col_scale = None
        needs_grad = torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters()))
        if prepare and needs_grad:
            # training: projection, query / key norm and rotation as differentiable steps
            query, key, value = _dense(self.qkv, x).chunk(3, dim=-1)
            query, key = qk_norm_rope(query, key, query_weight, key_weight, num_heads=self.num_heads, eps=qk_eps,
                                      rope_base=self.rope_base)
        elif (prepare and dtype == torch.bfloat16 and x.ndim == 3 and x.shape[-1] in (128, 256)
              and not (self.training and self.dropout > 0.0)):
            # the norm statistic (and, with a rotation, weight and rotation) come out of the projection's epilogue; the
            # per-token factor of the norm and the weights of the unrotated case are applied inside the attention
            # kernel: no pass over q and k at all (the attention call with dropout takes no row factors: a train-mode
            # block with dropout goes through the explicit pass below, also when nothing requires a gradient)
            qkv, q_row_scale, k_row_scale, q_col_scale = qkv_projection(
                x, _bf16(self.qkv.weight), _bf16(self.qkv.bias), num_heads=self.num_heads, query_weight=query_weight,
                key_weight=key_weight, qk_eps=qk_eps, rope_base=self.rope_base,
            )
            query, key, value = qkv.chunk(3, dim=-1)
        else:
            query, key, value = _dense(self.qkv, x).chunk(3, dim=-1)
            if prepare:  # one pass over the q and k columns of the packed projection, in place
                qk_norm_rope(query, key, query_weight, key_weight, num_heads=self.num_heads, eps=qk_eps,
                             rope_base=self.rope_base, inplace=True)
        structured = attention_mask if isinstance(attention_mask, StructuredAttentionMask) else None
        attended = scaled_dot_product_attention(
            query,
            key,
            value,
            num_heads=self.num_heads,
            attn_mask=None if structured is not None else attention_mask,
            structured_mask=structured,
            dropout_p=self.dropout,
            training=self.training,
            key_lengths=key_lengths,
            zero_padded_queries=zero_padded_queries,
            q_row_scale=q_row_scale,
            k_row_scale=k_row_scale,
            q_col_scale=q_col_scale,
        )
        out = _dense(self.out, attended, residual=_as(residual, dtype))
        return out if out.dtype == output_dtype else out.to(output_dtype)


class BFTSAttention(UnifiedSelfAttention):
    """TokenFormer's attention layer (experiments/tokenformer/model.py:139-163): the same layer with an optional
    rotary embedding of the normalised query and key over the token positions (``_apply_rope``, :165-192)."""

    def __init__(self, d_model: int, num_heads: int, dropout: float = 0.0, *, use_rope: bool, rope_base: float) -> None:
        super().__init__(d_model, num_heads, dropout, qk_norm=True)
        if (int(d_model) // int(num_heads)) % 2 != 0 and use_rope:
            raise ValueError("hip BFTSAttention rotates whole heads: head_dim must be even")
        self.use_rope = bool(use_rope)
        self.rope_base = float(rope_base) if use_rope else None


# Debugging aid: verify on every block call that padding_mask is the prefix mask of key_lengths (see the block's docstring).
CHECK_PADDING_CONTRACT = False


def check_padding_contract(padding_mask: torch.Tensor, key_lengths: torch.Tensor) -> None:
    """Raise ValueError unless ``padding_mask[b, t] == (t >= key_lengths[b])`` everywhere (synchronises the device)."""
    positions = torch.arange(padding_mask.shape[1], device=padding_mask.device)
    expected = positions[None, :] >= key_lengths.to(padding_mask.device)[:, None]
    if padding_mask.shape != expected.shape or not bool((padding_mask.bool() == expected).all()):
        raise ValueError("padding_mask is not the prefix mask of key_lengths: the routes that walk the valid rows of "
                         "key_lengths and the layer-by-layer route would disagree")


class UnifiedInteractionBlock(nn.Module):
    """Pre-RMSNorm self-attention and SwiGLU feed-forward with residuals masked at padded positions
    (experiments/symbiosis/backbone.py:51-68).

    For bf16 GPU tokens of width 128 / 256 under ``torch.no_grad()`` the block runs on the fused kernels: the dense
    layers walk the valid rows only (``update * ~padding_mask`` becomes "the padded rows are never touched": they keep
    their input values, as ``x + 0`` does), ``attn_norm`` and the query / key norm statistic are part of the projection
    kernel, and with ``return_attention_tokens=False`` the out projection, both residual adds, ``ffn_norm`` and the
    feed-forward are one kernel. ``attention_mask`` may be a dense bool mask, a :class:`StructuredAttentionMask`
    (what ``MetadataAttentionMask`` returns) or None; ``key_lengths`` states prefix padding without a mask.
    Contract of ``key_lengths``: when it is given, ``padding_mask`` must be exactly its prefix mask
    (``padding_mask[b, t] == (t >= key_lengths[b])``) - the fused route and the training route take the valid rows from
    ``key_lengths`` alone and never read ``padding_mask``, while the layer-by-layer route multiplies the updates by
    ``~padding_mask``. ``taac_2026_amd.modeling.backbone.CHECK_PADDING_CONTRACT = True`` makes ``forward`` verify this
    (one device synchronisation per call: a debugging aid, off by default) and raise ``ValueError`` on a mismatch.
    ``inplace=True`` lets the fused route update ``tokens`` itself instead of a copy. ``token_layout``: ``"front"``
    (default) lets the fused route move every sample's valid tokens to the front of its rows for the attention call
    when the mask allows it, ``"positions"`` keeps them where they are (comparison route; same results)."""

    def __init__(self, d_model: int, num_heads: int, hidden_mult: int, dropout: float = 0.0, *, qk_norm: bool = True,
                 token_layout: str = "front") -> None:
        super().__init__()
        if token_layout not in ("front", "positions"):
            raise ValueError("token_layout must be 'front' or 'positions'")
        self.token_layout = token_layout
        self.attn_norm = RMSNorm(d_model)
        self.attention = UnifiedSelfAttention(d_model, num_heads, dropout, qk_norm=qk_norm)
        self.ffn_norm = RMSNorm(d_model)
        self.ffn = SwiGLUFeedForward(d_model, hidden_mult, dropout)

    def _fused_route(self, tokens: torch.Tensor) -> bool:
        if not (tokens.is_cuda and tokens.dtype == torch.bfloat16 and tokens.ndim == 3 and tokens.shape[-1] in (128, 256)):
            return False
        if self.ffn.down.weight.shape[1] % 32 != 0:
            return False
        if self.training and (self.attention.dropout > 0.0 or self.ffn.dropout.p > 0.0):
            return False
        return not (torch.is_grad_enabled() and (tokens.requires_grad or any(p.requires_grad for p in self.parameters())))

    def _forward_fused(self, tokens, padding_mask, attention_mask, key_lengths, return_attention_tokens, inplace):
        batch, token_count, d_model = tokens.shape
        x = tokens.contiguous()
        attention = self.attention
        structured = attention_mask if isinstance(attention_mask, StructuredAttentionMask) else None
        dense_mask = None if structured is not None else attention_mask
        # Padding scattered inside the samples, under a structured mask whose valid keys are exactly the non-padded
        # positions: the projection writes every sample's valid tokens at the front of its rows, so that the attention
        # call sees prefix padding (its cost follows the valid tokens, not the positions) with the mask's structure
        # gathered per sample, and the out projection reads that layout back. token_layout="positions" keeps the
        # tokens where they are (comparison route).
        # The indices and the gathered mask depend on the mask object only: the blocks of a stack, which all receive it,
        # share them through its cache.
        front = lengths = None
        if (structured is not None and key_lengths is None and structured.padding_source is padding_mask
                and structured.query_self is None and not structured.sample_stride
                and structured.structural.shape == (token_count, token_count)
                and self.token_layout != "positions"):
            entry = structured.cache.get("front")
            if entry is None or entry[0] != padding_mask._version:  # rebuilt when the padding mask was written to
                index = valid_rows(None, token_count, padding_mask=padding_mask)
                entry = (padding_mask._version, index, *front_rows(index, batch, token_count),
                         front_structured_mask(structured, index, batch))
                structured.cache["front"] = entry
            _, index, front, lengths, structured = entry
        elif key_lengths is not None:
            index = valid_rows(key_lengths, token_count)
        elif structured is not None and structured.padding_source is padding_mask:
            entry = structured.cache.get("rows")
            if entry is None or entry[0] != padding_mask._version:
                entry = structured.cache["rows"] = (padding_mask._version,
                                                    valid_rows(None, token_count, padding_mask=padding_mask))
            index = entry[1]
        else:
            index = valid_rows(None, token_count, padding_mask=padding_mask)
        # The projection may skip the padded tokens only when the mask proves that no query can see a padded key: a key
        # length handed to the attention call, or a structured mask whose key validity was derived from this padding
        # mask. Otherwise (no mask, a dense mask, a structured mask of unknown origin) the padded tokens are projected
        # like every other token, as the reference block does (experiments/symbiosis/backbone.py:58-63), and only the
        # residual updates skip them.
        padded_keys_hidden = (front is not None or (key_lengths is not None and attention_mask is None)
                              or (structured is not None and structured.padding_source is padding_mask))
        if front is not None:
            qkv_rows = dict(token_rows=(front, index[1]), input_rows=index[0])
        else:
            qkv_rows = dict(token_rows=index) if padded_keys_hidden else {}
        qkv = torch.empty(batch * token_count, 3 * d_model, dtype=x.dtype, device=x.device)
        q_row_scale = k_row_scale = q_col_scale = None
        if attention.query_norm is not None or attention.rope_base is not None:
            _, q_row_scale, k_row_scale, q_col_scale = qkv_projection(
                x, _bf16(attention.qkv.weight), _bf16(attention.qkv.bias), num_heads=attention.num_heads,
                norm_weight=_bf16(self.attn_norm.weight), eps=self.attn_norm.eps,
                query_weight=None if attention.query_norm is None else _bf16(attention.query_norm.weight),
                key_weight=None if attention.key_norm is None else _bf16(attention.key_norm.weight),
                qk_eps=1e-6 if attention.query_norm is None else attention.query_norm.eps, rope_base=attention.rope_base,
                out=qkv, **qkv_rows)
        else:
            norm_linear(x, _bf16(attention.qkv.weight), _bf16(attention.qkv.bias), norm_weight=_bf16(self.attn_norm.weight),
                        eps=self.attn_norm.eps, out=qkv, **qkv_rows)
        query, key, value = qkv.view(batch, token_count, 3 * d_model).chunk(3, dim=-1)
        attended = scaled_dot_product_attention(
            query, key, value, num_heads=attention.num_heads, attn_mask=dense_mask, structured_mask=structured,
            dropout_p=0.0, training=False, key_lengths=lengths if front is not None else (key_lengths if attention_mask is None else None),
            zero_padded_queries=2 if front is not None else False,
            q_row_scale=q_row_scale, k_row_scale=k_row_scale, q_col_scale=q_col_scale)
        ffn = self.ffn
        dense = dict(norm_weight=_bf16(self.ffn_norm.weight), eps=self.ffn_norm.eps, token_rows=index)
        if front is not None:
            dense["input_rows"] = front
        gate_layer = getattr(self, "nlir_gate", None)
        if gate_layer is not None:
            # the gate layer reads the normalised block input, like the projection in front of attention; its output (before
            # the sigmoid) is written at the valid rows and consumed by the kernel that applies the update
            gate = torch.empty(batch * token_count, d_model, dtype=x.dtype, device=x.device)
            norm_linear(x, _bf16(gate_layer.weight), _bf16(gate_layer.bias), norm_weight=_bf16(self.attn_norm.weight),
                        eps=self.attn_norm.eps, token_rows=index, out=gate)
            output = x if inplace else x.clone()
            attention_out_ffn(attended, _bf16(attention.out.weight), _bf16(attention.out.bias), x, _bf16(ffn.up.weight),
                              _bf16(ffn.up.bias), _bf16(ffn.down.weight), _bf16(ffn.down.bias), out=output,
                              update_gate=gate.view(batch, token_count, d_model), **dense)
            return output, None
        if not return_attention_tokens and ffn.gate_first:
            output = x if inplace else x.clone()
            attention_out_ffn(attended, _bf16(attention.out.weight), _bf16(attention.out.bias), x, _bf16(ffn.up.weight),
                              _bf16(ffn.up.bias), _bf16(ffn.down.weight), _bf16(ffn.down.bias), out=output, **dense)
            return output, None
        attn_tokens = x.clone()  # padded rows pass through
        norm_linear(attended, _bf16(attention.out.weight), _bf16(attention.out.bias), residual=x, token_rows=index,
                    input_rows=front, out=attn_tokens)
        output = attn_tokens.clone()
        dense.pop("input_rows", None)
        swiglu_ffn(attn_tokens, _bf16(ffn.up.weight), _bf16(ffn.up.bias), _bf16(ffn.down.weight), _bf16(ffn.down.bias),
                   residual=attn_tokens, gate_first=ffn.gate_first, out=output, **dense)
        return output, attn_tokens

    def forward(
        self,
        tokens: torch.Tensor,
        padding_mask: torch.Tensor,
        attention_mask: torch.Tensor | StructuredAttentionMask | None,
        *,
        key_lengths: torch.Tensor | None = None,
        return_attention_tokens: bool = True,
        inplace: bool = False,
    ) -> tuple[torch.Tensor, torch.Tensor | None]:
        if CHECK_PADDING_CONTRACT and key_lengths is not None:
            check_padding_contract(padding_mask, key_lengths)
        if self._fused_route(tokens):
            return self._forward_fused(tokens, padding_mask, attention_mask, key_lengths, return_attention_tokens, inplace)
        if torch.is_grad_enabled() and training_route_applies(self, tokens, attention_mask, key_lengths, padding_mask):
            # key lengths or a structured mask built from the padding mask, no rotary embedding, no dropout: the whole block
            # as one autograd function over the valid rows
            structured = attention_mask if isinstance(attention_mask, StructuredAttentionMask) else None
            result = run_training_block(self, tokens, key_lengths, return_attention_tokens, structured,
                                        padding_mask if structured is not None else None)
            if result is not None:
                return result
        keep = (~padding_mask).unsqueeze(-1)
        attn_update = self.attention(self.attn_norm(tokens), attention_mask, key_lengths=key_lengths)
        attn_tokens = tokens + attn_update * keep.to(attn_update.dtype)
        ffn_update = self.ffn(self.ffn_norm(attn_tokens))
        output = attn_tokens + ffn_update * keep.to(ffn_update.dtype)
        return output, attn_tokens


class TokenFormerBlock(UnifiedInteractionBlock):
    """TokenFormer's block (experiments/tokenformer/model.py:195-215): the interaction block with ``BFTSAttention`` as its
    attention layer and the NLIR gate on the attention update,
    ``tokens + sigmoid(nlir_gate(attn_norm(tokens))) * attention(attn_norm(tokens)) * valid``, followed by the same
    feed-forward half. Same constructor signature, parameter names and ``forward(tokens, padding_mask, attention_mask)``
    -> tokens. For bf16 GPU tokens of width 128 / 256 under ``torch.no_grad()`` the block runs on the fused kernels: the
    gate layer's output comes from the projection kernel over the valid rows, and its sigmoid, the gated update, both
    residual adds, ``ffn_norm`` and the feed-forward are one kernel (``taac_attn_out_gate_ffn_fwd``); padded rows are
    never touched. Other inputs (and tensors that take a gradient) run layer by layer."""

    def __init__(self, d_model: int, num_heads: int, hidden_mult: int, dropout: float = 0.0, *, use_rope: bool,
                 rope_base: float, token_layout: str = "front") -> None:
        super().__init__(d_model, num_heads, hidden_mult, dropout, qk_norm=True, token_layout=token_layout)
        self.attention = BFTSAttention(d_model, num_heads, dropout, use_rope=use_rope, rope_base=rope_base)
        self.nlir_gate = nn.Linear(d_model, d_model)

    def forward(self, tokens: torch.Tensor, padding_mask: torch.Tensor,
                attention_mask: torch.Tensor | StructuredAttentionMask | None, *, key_lengths: torch.Tensor | None = None,
                inplace: bool = False) -> torch.Tensor:
        if CHECK_PADDING_CONTRACT and key_lengths is not None:
            check_padding_contract(padding_mask, key_lengths)
        if self._fused_route(tokens) and self.ffn.gate_first:
            return self._forward_fused(tokens, padding_mask, attention_mask, key_lengths, False, inplace)[0]
        keep = (~padding_mask).unsqueeze(-1)
        attention_input = self.attn_norm(tokens)
        attention_update = self.attention(attention_input, attention_mask, key_lengths=key_lengths)
        gate_input = attention_input if attention_input.dtype == torch.bfloat16 else attention_input.to(torch.bfloat16)
        gate = torch.sigmoid(_dense(self.nlir_gate, gate_input)).to(attention_update.dtype)
        tokens = tokens + gate * attention_update * keep.to(attention_update.dtype)
        ffn_update = self.ffn(self.ffn_norm(tokens))
        return tokens + ffn_update * keep.to(ffn_update.dtype)


def run_interaction_blocks(blocks, tokens: torch.Tensor, padding_mask: torch.Tensor,
                           attention_mask: torch.Tensor | StructuredAttentionMask | None) -> torch.Tensor:
    """The block loop of the reference model's ``_run_backbone`` (experiments/symbiosis/model.py:283-292, without its
    ``final_norm``, which the readout head applies): every block receives the same padding mask and attention mask and
    only its output stream is kept. The stream is copied once and the blocks then update it in place; with a mask from
    ``MetadataAttentionMask`` the row indices and the mask gathered per sample are built by the first block and shared
    by the others. The padding mask must not be modified while the loop runs."""
    stream = tokens
    for position, block in enumerate(blocks):
        stream, _ = block(stream, padding_mask, attention_mask, return_attention_tokens=False, inplace=position > 0)
    return stream


class _PlainBlock(nn.Module):
    """Parameter container of one canonical block: RMSNorm -> MHA -> +res -> RMSNorm -> SwiGLU -> +res."""

    def __init__(self, d_model: int, num_heads: int, d_ff: int, qk_norm: bool = False) -> None:
        super().__init__()
        self.attn_norm = RMSNorm(d_model)
        self.qkv = nn.Linear(d_model, 3 * d_model)
        self.query_norm = RMSNorm(d_model) if qk_norm else None
        self.key_norm = RMSNorm(d_model) if qk_norm else None
        self.out = nn.Linear(d_model, d_model)
        self.ffn_norm = RMSNorm(d_model)
        self.up = nn.Linear(d_model, 2 * d_ff)
        self.down = nn.Linear(d_ff, d_model)
        self.num_heads = num_heads


class PCVRBackbone(nn.Module):
    """n_blocks pre-norm blocks + masked mean-pool -> Linear(D, 1) -> sigmoid, run by one ``taac_backbone_fwd`` call.

    Initialisation: Xavier-uniform weights, zero biases, unit norm weights.
    ``forward(emb[B, T, D] bf16, key_lengths[B] int32) -> p[B] float32``; ``return_hidden=True`` also returns the
    final hidden state (rows at or beyond ``key_lengths[b]`` are zeros). ``dense_tokens=True`` runs the dense layers over
    the padded positions too (what the reference's dense ``[B, T, D]`` formulation does; same valid rows, bit for bit),
    ``split_out_ffn=True`` runs the out projection and the feed-forward half as two kernels, ``row_major_qkv=True`` keeps
    q | k | v and the attention output of the workspace as rows instead of per-head planes (comparison routes;
    ``row_major_qkv`` gives bit-identical results).
    ``fp8=True`` runs the four dense layers of every block with e4m3 operands and per-tensor scales (d_model 256, plain
    attention layer).
    ``qk_norm=True`` adds the reference layer's ``RMSNorm(d_model)`` of the query and the key
    (experiments/symbiosis/backbone.py:30-36), ``rope_base`` TokenFormer's rotary embedding of both over the token
    positions (experiments/tokenformer/model.py:165-192); the benchmark recipe has neither.
    """

    def __init__(self, d_model: int = 256, num_heads: int = 8, d_ff: int = 1024, n_blocks: int = 4, eps: float = 1e-6,
                 *, qk_norm: bool = False, rope_base: float | None = None) -> None:
        super().__init__()
        if d_model % num_heads != 0:
            raise ValueError("d_model must be divisible by num_heads")
        self.d_model, self.num_heads, self.d_ff, self.eps = int(d_model), int(num_heads), int(d_ff), float(eps)
        self.rope_base = None if rope_base is None else float(rope_base)
        self.blocks = nn.ModuleList(_PlainBlock(d_model, num_heads, d_ff, qk_norm) for _ in range(n_blocks))
        self.head = nn.Linear(d_model, 1)
        self.reset_parameters()
        self._workspace: torch.Tensor | None = None

    def reset_parameters(self) -> None:
        for module in self.modules():
            if isinstance(module, nn.Linear):
                nn.init.xavier_uniform_(module.weight)
                nn.init.zeros_(module.bias)

    def _get_workspace(self, nbytes: int, device: torch.device) -> torch.Tensor:
        ws = self._workspace
        if ws is None or ws.numel() < nbytes or ws.device != device:
            ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
            self._workspace = ws
        return ws

    def forward(self, emb: torch.Tensor, key_lengths: torch.Tensor, *, return_hidden: bool = False,
                dense_tokens: bool = False, split_out_ffn: bool = False, fp8: bool = False, row_major_qkv: bool = False):
        name = "hip PCVRBackbone"
        require_cuda_tensors(name, emb, key_lengths)
        if torch.is_grad_enabled() and (emb.requires_grad or any(p.requires_grad for p in self.parameters())):
            if dense_tokens or split_out_ffn or fp8 or row_major_qkv:
                raise RuntimeError(f"{name}: dense_tokens, split_out_ffn, fp8 and row_major_qkv are inference routes: call "
                                   "them under torch.no_grad()")
            return self._forward_training(emb, key_lengths, return_hidden)
        if emb.ndim != 3 or emb.shape[-1] != self.d_model:
            raise ValueError(f"PCVRBackbone expects embeddings of shape (batch, tokens, {self.d_model})")
        if emb.dtype != torch.bfloat16:
            raise RuntimeError(f"{name} expects bfloat16 embeddings, got {emb.dtype}")
        if key_lengths.shape != (emb.shape[0],):
            raise ValueError("key_lengths must have shape (batch,)")
        emb = emb.contiguous()
        key_lengths = key_lengths.to(torch.int32).contiguous()
        batch, tokens, _ = emb.shape
        library = _native.load_library()

        keep_alive: list[torch.Tensor] = []

        def dev(parameter: torch.Tensor | None) -> int | None:
            tensor = _bf16(parameter)
            if tensor is None:
                return None
            tensor = tensor.detach().contiguous()
            keep_alive.append(tensor)
            return tensor.data_ptr()

        packed = (_native.BlockWeights * len(self.blocks))()
        for slot, block in zip(packed, self.blocks):
            slot.attn_norm_weight = dev(block.attn_norm.weight)
            slot.qkv_weight, slot.qkv_bias = dev(block.qkv.weight), dev(block.qkv.bias)
            slot.out_weight, slot.out_bias = dev(block.out.weight), dev(block.out.bias)
            slot.ffn_norm_weight = dev(block.ffn_norm.weight)
            slot.up_weight, slot.up_bias = dev(block.up.weight), dev(block.up.bias)
            slot.down_weight, slot.down_bias = dev(block.down.weight), dev(block.down.bias)
            if block.query_norm is not None:
                slot.query_norm_weight = dev(block.query_norm.weight)
                slot.key_norm_weight = dev(block.key_norm.weight)
        table = None
        if self.rope_base is not None:
            table = rope_table(tokens, self.d_model // self.num_heads, self.rope_base, torch.bfloat16, emb.device)

        nbytes = library.taac_backbone_workspace_bytes(batch, tokens, self.d_model, self.d_ff, len(self.blocks))
        workspace = self._get_workspace(int(nbytes), emb.device)
        hidden = torch.empty_like(emb) if return_hidden else None
        flags = ((_native.BACKBONE_DENSE_TOKENS if dense_tokens else 0) | (_native.BACKBONE_SPLIT_OUT_FFN if split_out_ffn else 0)
                 | (_native.BACKBONE_FP8 if fp8 else 0) | (_native.BACKBONE_ROW_MAJOR_QKV if row_major_qkv else 0))
        probabilities = torch.empty(batch, dtype=torch.float32, device=emb.device)
        status = library.taac_backbone_fwd(
            emb.data_ptr(), key_lengths.data_ptr(), packed, len(self.blocks), dev(self.head.weight.reshape(-1)),
            dev(self.head.bias), batch, tokens, self.d_model, self.num_heads, self.d_ff, ctypes.c_float(self.eps),
            _native.ptr(table), flags, workspace.data_ptr(), workspace.numel(), _native.ptr(hidden),
            probabilities.data_ptr(),
            _native.current_stream(emb.device),
        )
        _native.check(status, "backbone_fwd")
        self._fp8_maxima = None
        if fp8:
            offset = library.taac_backbone_fp8_scales_offset(batch, tokens, self.d_model, self.d_ff, len(self.blocks))
            count = (len(self.blocks) + 1) * 8
            self._fp8_maxima = workspace[offset:offset + 4 * count].view(torch.float32).view(-1, 8)
        if return_hidden:
            return probabilities, hidden
        return probabilities

    def _forward_training(self, emb: torch.Tensor, key_lengths: torch.Tensor, return_hidden: bool):
        """The same network under autograd: every block as one function over the valid rows
        (:class:`InteractionBlockFunction`), then the masked mean over the valid tokens, the head and the sigmoid as
        differentiable tensor operations (``masked_mean``, modeling/sequence.py:54-60). One host synchronisation per
        ``key_lengths`` tensor (the number of valid rows sizes the backward's tensors)."""
        from taac_2026_amd.modeling.block_training import InteractionBlockFunction

        name = "hip PCVRBackbone"
        if emb.ndim != 3 or emb.shape[-1] != self.d_model or emb.dtype != torch.bfloat16:
            raise ValueError(f"{name} expects bfloat16 embeddings of shape (batch, tokens, {self.d_model})")
        if key_lengths.shape != (emb.shape[0],):
            raise ValueError("key_lengths must have shape (batch,)")
        head_dim = self.d_model // self.num_heads
        if self.rope_base is not None or self.d_model not in (128, 256) or head_dim not in (32, 64) or self.d_ff % 32 != 0 \
                or any(p.dtype not in (torch.bfloat16, torch.float32) for p in self.parameters()) \
                or not swiglu_ffn_backward_supported(self.d_model, self.d_ff):
            raise RuntimeError(f"{name}: the training route covers bf16 (or float32 master) parameters, d_model 128 / 256, "
                               "head dims 32 / 64, d_ff a multiple of 32 within the backward kernel's bound "
                               "(taac_swiglu_ffn_bwd_packed_bytes) and no rotary embedding")
        if key_lengths.dtype != torch.int32 or not key_lengths.is_contiguous():
            key_lengths = key_lengths.to(torch.int32).contiguous()
        stream = emb
        for block in self.blocks:
            qk = block.query_norm is not None
            stream, _ = InteractionBlockFunction.apply(
                stream, key_lengths, None, None, False, self.num_heads, self.eps, self.eps, True, self.eps,
                _bf16(block.attn_norm.weight), _bf16(block.qkv.weight), _bf16(block.qkv.bias), _bf16(block.out.weight),
                _bf16(block.out.bias), _bf16(block.ffn_norm.weight), _bf16(block.up.weight), _bf16(block.up.bias),
                _bf16(block.down.weight), _bf16(block.down.bias), _bf16(block.query_norm.weight) if qk else None,
                _bf16(block.key_norm.weight) if qk else None)
        tokens = emb.shape[1]
        valid = (torch.arange(tokens, device=emb.device)[None, :] < key_lengths[:, None]).to(stream.dtype).unsqueeze(-1)
        pooled = (stream * valid).sum(dim=1) / valid.sum(dim=1).clamp_min(1.0)
        logits = torch.nn.functional.linear(pooled, _bf16(self.head.weight), _bf16(self.head.bias)).squeeze(-1)
        probabilities = torch.sigmoid(logits.float())
        if return_hidden:
            return probabilities, stream * valid      # rows at or beyond key_lengths[b] are zeros, as in the forward-only route
        return probabilities

    FP8_MAXIMA = ("qkv.weight", "out.weight", "up.weight", "down.weight", "attn_norm", "attention", "ffn_norm", "hidden")

    def fp8_maxima(self) -> list[dict[str, torch.Tensor]]:
        """Per block, the per-tensor maxima (scale = maximum / 448) the last ``fp8=True`` forward quantised with: the four
        weights, the two normalised streams, the attention output and the gated hidden state (host tensors; waits for
        the forward)."""
        if getattr(self, "_fp8_maxima", None) is None:
            raise RuntimeError("hip PCVRBackbone: no fp8 forward has run on this module")
        table = self._fp8_maxima[:len(self.blocks)].cpu()
        return [dict(zip(self.FP8_MAXIMA, row)) for row in table]


__all__ = [
    "BFTSAttention",
    "PCVRBackbone",
    "SwiGLUFeedForward",
    "UnifiedInteractionBlock",
    "UnifiedSelfAttention",
]
