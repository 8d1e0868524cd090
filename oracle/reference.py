"""CPU oracle: a restatement of the reference's torch implementation of the backbone kernel path.

TEST INFRASTRUCTURE ONLY. Nothing under ``taac_2026_amd/`` imports this module; it is used by ``tests/``, by
``__graft_entry__.smoke()`` as the checker, and by ``bench.py``'s ``cpu_baseline`` leg as the thing timed on the host.
Everything here runs on CPU tensors with plain torch / numpy; it never touches the HIP library.

Each function cites the reference source it restates (paths relative to the reference tree,
Puiching-Memory/TAAC_2026). How each function is pinned, independently of its own formula (tests/test_oracle.py):

  rms_norm            closed form restated by the reference's own test (tests/unit/infrastructure/accelerators/
                      test_tilelang_ops.py:533-540); float64 loop brute force, scale equivariance, row independence,
                      the identity sum((y/w)^2)/D = 1 - eps*s^2.
  layer_norm          torch.nn.functional.layer_norm (library routine, test_tilelang_ops.py:543-551); float64 brute
                      force; zero mean / unit variance of the normalised rows; shift invariance.
  attention           F.scaled_dot_product_attention with a bool mask (test_tilelang_ops.py:305-313); float64 loop
                      brute force; len == T reduces to unmasked SDPA; len == 1 returns v[0]; identical keys return the
                      mean of the valid values; committed golden vector tests/golden/attention_small.json.
  make_padding_mask / safe_key_padding_mask / plan of structured masks
                      literal known answers held by the reference's tests (tests/unit/infrastructure/modeling/
                      test_primitives.py:36-39, tests/contract/experiments/test_packages.py:597-617,
                      test_tilelang_ops.py:361-428), committed as tests/golden/mask_vectors.json.
  masked_mean         float64 brute force; all-padded rows give zeros (divisor clamp).
  embedding_bag_mean  the library routine F.embedding_bag and the closed form held by the reference's own test
                      (test_tilelang_ops.py:123-140) on that test's literal id matrix; float64 loop brute force.
  bfts_attention_mask / metadata_attention_mask
                      the reference holds no known answer for them (its contract test checks the shape and that the
                      readout rows see a key, tests/contract/experiments/test_packages.py:430-440); restated here as
                      per-element rules, pinned by hand-derived small cases and invariants (every valid query sees
                      itself, padded keys are never seen, target rows and separator columns are full, window counts).
  rotate_half_pairs / rope_tables / apply_rope / qk_norm_rope
                      the reference holds no numeric test for them; pinned by what a rotation fixes: multiplication of
                      even + i*odd by exp(i*angle) (numpy complex128), position 0 is the identity, pair norms are
                      kept, the score of a rotated query and key depends only on the position difference, angles
                      against a float64 loop; the norm part reduces to rms_norm over the model width.
  swiglu_ffn / linear / block / backbone
                      compositions of library routines F.linear, F.silu, the functions above; float64 loop brute
                      force on tiny shapes for swiglu_ffn; the reference holds no numeric test for these
                      (tests/contract/experiments/test_packages.py:170-192 checks shapes and finiteness only).
  candidate_readout / interaction_block
                      compositions of the functions above as the reference's modules write them (experiments/symbiosis/
                      pooling.py:24-32, model.py:217-222, backbone.py:58-68); candidate_readout is pinned by a float64
                      loop and special cases (no candidate -> zero third, all-padded sample -> zero mean, no norms ->
                      picked rows and plain masked mean); qk_norm_rope and embedding_bag_mean additionally by the
                      pure-Python float64 vectors of tests/golden/qk_rope_embedding_small.json.
  tokenformer_block / silu_mlp / mixed_feed_forward
                      the reference holds no numeric test for them (shape / finiteness contract tests only); compositions
                      of the functions above as the modules write them (experiments/tokenformer/model.py:203-215,
                      experiments/onetrans/model.py:33-44, 80-94), pinned by float64 per-element loops on tiny shapes
                      (gate = 1 / (1 + exp(-z)) applied to the update before the residual add; padded rows pass
                      through; a zero gate layer halves the update), the gated block reducing to interaction_block's
                      arithmetic when the gate is forced to one, and token replacement checked slot by slot.
  fp8 emulation       PARITY UNPINNED by the reference (it has no FP8 code). Defined by the configuration text:
                      s = amax/448, q = (t/s).to(float8_e4m3fn), y = (qa.float() @ qw.float().T) * s_a * s_w.
                      The e4m3 rounding itself is pinned against an exhaustive decode table of all 256 codes and
                      nearest-even brute force (tests/test_oracle.py).
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F

FP8_MAX = 448.0


# ---- normalisation ---------------------------------------------------------------------------------------------------


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """``_torch_rms_norm`` (src/taac2026/infrastructure/accelerators/normalization/rms_norm.py:71-73), computed in
    x's dtype exactly as the reference's torch backend does (bf16 inputs round x^2 to bf16 before the mean)."""
    weight = weight.to(dtype=x.dtype)  # rms_norm.py:85
    scale = torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)
    return x * scale * weight


def rms_norm_fp32(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """Same closed form with fp32 statistics and a single rounding to x's dtype - what the reference's Triton and
    TileLang kernels compute (normalization/kernels/triton.py:30-50). This is the parity target for 16-bit inputs."""
    xf = x.float()
    wf = weight.to(dtype=x.dtype).float()
    scale = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    return (xf * scale * wf).to(x.dtype)


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """``_torch_layer_norm`` (normalization/layer_norm.py:65-66)."""
    return F.layer_norm(x, (x.shape[-1],), weight.to(x.dtype), bias.to(x.dtype), eps)


def layer_norm_fp32(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """fp32 statistics, one rounding (normalization/kernels/triton.py:224-247)."""
    out = F.layer_norm(x.float(), (x.shape[-1],), weight.to(x.dtype).float(), bias.to(x.dtype).float(), eps)
    return out.to(x.dtype)


# ---- masks and pooling -----------------------------------------------------------------------------------------------


def make_padding_mask(lengths: torch.Tensor, max_len: int) -> torch.Tensor:
    """modeling/sequence.py:32-34: True = padding."""
    positions = torch.arange(max_len, device=lengths.device).unsqueeze(0)
    return positions >= lengths.unsqueeze(1)


def safe_key_padding_mask(mask: torch.Tensor) -> torch.Tensor:
    """modeling/sequence.py:37-45."""
    if mask.numel() == 0 or mask.shape[1] == 0:
        return mask
    all_masked = mask.all(dim=1, keepdim=True)
    first_column = torch.zeros_like(mask)
    first_column[:, :1] = True
    return torch.where(all_masked, mask & ~first_column, mask)


def masked_mean(tokens: torch.Tensor, padding_mask: torch.Tensor | None = None) -> torch.Tensor:
    """modeling/sequence.py:54-60."""
    if tokens.shape[1] == 0:
        return tokens.new_zeros(tokens.shape[0], tokens.shape[-1])
    if padding_mask is None:
        return tokens.mean(dim=1)
    valid = (~padding_mask).to(tokens.dtype).unsqueeze(-1)
    return (tokens * valid).sum(dim=1) / valid.sum(dim=1).clamp_min(1.0)


def key_length_mask(key_lengths: torch.Tensor, heads: int, query_len: int, kv_len: int) -> torch.Tensor:
    """(B, H, Tq, Tk) bool mask, True = attend, for per-sample valid key prefixes - the mask family the reference's
    planner reduces to ``key_lengths`` (attention/flash_attention.py:172-181)."""
    key_valid = torch.arange(kv_len).unsqueeze(0) < key_lengths.unsqueeze(1).to(torch.int64)
    return key_valid[:, None, None, :].expand(key_lengths.shape[0], heads, query_len, kv_len)


def causal_valid_attention_mask(padding_mask: torch.Tensor, num_heads: int) -> torch.Tensor:
    """modeling/sequence.py:119-127."""
    batch_size, token_count = padding_mask.shape
    causal = torch.ones(token_count, token_count, dtype=torch.bool).tril()
    mask = causal.unsqueeze(0) & (~padding_mask).unsqueeze(1)
    fallback = torch.eye(token_count, dtype=torch.bool).unsqueeze(0)
    mask = torch.where(padding_mask.unsqueeze(-1), fallback, mask)
    return mask.unsqueeze(1).expand(batch_size, num_heads, token_count, token_count)


# ---- attention -------------------------------------------------------------------------------------------------------


def sdpa(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, attn_mask: torch.Tensor | None = None,
         is_causal: bool = False) -> torch.Tensor:
    """``_torch_flash_attention`` in eval mode (attention/flash_attention.py:552-570)."""
    return F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask, dropout_p=0.0,
                                          is_causal=is_causal if attn_mask is None else False)


def attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    key_lengths: torch.Tensor | None = None,
    *,
    is_causal: bool = False,
    zero_padded_queries: bool = False,
) -> torch.Tensor:
    """fp32 ``softmax(q k^T / sqrt(d) masked_fill -inf) v`` on (B, H, T, d) inputs, result in v's dtype.

    The explicit form the reference's GPU tests compare against
    (tests/gpu/infrastructure/accelerators/test_tilelang_ops_cuda.py:37-57). Rows whose visible key set is empty
    give 0, as the reference kernel does (attention/kernels/tilelang.py:127-133). With ``zero_padded_queries`` rows
    ``t >= key_lengths[b]`` are set to 0 (the benchmark configuration's definition of padded query rows).
    """
    batch, heads, query_len, head_dim = q.shape
    kv_len = k.shape[2]
    scores = torch.matmul(q.float(), k.float().transpose(-1, -2)) * (1.0 / math.sqrt(head_dim))
    visible = torch.ones(batch, 1, query_len, kv_len, dtype=torch.bool)
    if key_lengths is not None:
        visible = visible & (torch.arange(kv_len)[None, None, None, :] < key_lengths.to(torch.int64)[:, None, None, None])
    if is_causal:
        visible = visible & (torch.arange(query_len)[:, None] >= torch.arange(kv_len)[None, :])[None, None]
    scores = scores.masked_fill(~visible, float("-inf"))
    row_max = scores.amax(dim=-1, keepdim=True)
    row_max = torch.where(torch.isinf(row_max), torch.zeros_like(row_max), row_max)
    weights = torch.exp(scores - row_max)
    denom = weights.sum(dim=-1, keepdim=True)
    probs = torch.where(denom > 0, weights / denom.clamp_min(1e-38), torch.zeros_like(weights))
    out = torch.matmul(probs, v.float())
    if zero_padded_queries and key_lengths is not None:
        keep = torch.arange(query_len)[None, :] < key_lengths.to(torch.int64)[:, None]
        out = out * keep[:, None, :, None].to(out.dtype)
    return out.to(v.dtype)


def attention_dropout(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, key_lengths: torch.Tensor | None,
                      dropout_mask: torch.Tensor, dropout_p: float, *, is_causal: bool = False,
                      zero_padded_queries: bool = False, attn_mask: torch.Tensor | None = None) -> torch.Tensor:
    """Training attention with dropout on the probabilities under a fixed keep mask, (B, H, T, d) tensors:
    ``softmax(scores)`` over the visible keys, then ``P * keep / (1 - p)``, then ``@ v`` - the semantics of the
    reference's training kernel (attention/kernels/tilelang.py:224-247: the normaliser sums the undropped probabilities)
    and of the manual reference its own test compares with
    (tests/gpu/infrastructure/accelerators/test_tilelang_ops_cuda.py:103-141). Differentiable; evaluate in float64 for
    gradient targets. Rows without a visible key give 0. ``attn_mask``: a bool mask of the models on top (what
    ``F.scaled_dot_product_attention(attn_mask=, dropout_p=)`` computes for them, with the keep mask fixed)."""
    batch, heads, query_len, dim = q.shape
    kv_len = k.shape[2]
    scores = torch.matmul(q, k.transpose(-1, -2)) * (dim ** -0.5)
    visible = torch.ones(batch, 1, query_len, kv_len, dtype=torch.bool)
    if key_lengths is not None:
        visible = visible & (torch.arange(kv_len)[None, None, None, :] < key_lengths.to(torch.int64)[:, None, None, None])
    if is_causal:
        visible = visible & (torch.arange(kv_len)[None, None, None, :] <= torch.arange(query_len)[None, None, :, None])
    if attn_mask is not None:  # a bool mask (B, 1 or H, Tq, Tk), True = attend, as the models build them
        visible = visible & attn_mask
    scores = scores.masked_fill(~visible, float("-inf"))
    probs = torch.softmax(scores, dim=-1)
    probs = torch.where(visible.any(dim=-1, keepdim=True), probs, torch.zeros_like(probs))
    probs = probs * dropout_mask.to(probs.dtype) / (1.0 - dropout_p)
    out = torch.matmul(probs, v)
    if zero_padded_queries and key_lengths is not None:
        keep_rows = torch.arange(query_len)[None, :] < key_lengths.to(torch.int64)[:, None]
        out = out * keep_rows[:, None, :, None].to(out.dtype)
    return out


def scaled_dot_product_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, num_heads: int,
                                 key_lengths: torch.Tensor | None = None, zero_padded_queries: bool = False) -> torch.Tensor:
    """modeling/sequence.py:81-116 on (B, T, D) projections, with the key-length mask."""
    batch, query_len, d_model = q.shape
    head_dim = d_model // num_heads
    q4 = q.view(batch, query_len, num_heads, head_dim).transpose(1, 2)
    k4 = k.view(batch, k.shape[1], num_heads, head_dim).transpose(1, 2)
    v4 = v.view(batch, v.shape[1], num_heads, head_dim).transpose(1, 2)
    out = attention(q4, k4, v4, key_lengths, zero_padded_queries=zero_padded_queries)
    return out.transpose(1, 2).contiguous().view(batch, query_len, d_model)


# ---- embedding bag -------------------------------------------------------------------------------------------------------


def embedding_bag_mean(weight: torch.Tensor, values: torch.Tensor) -> torch.Tensor:
    """``_torch_embedding_bag_mean`` (accelerators/embedding/embedding_bag.py:82-83): mean of the rows named by the
    non-zero ids of each bag, zeros for a bag of padding only."""
    return F.embedding_bag(values.long(), weight, mode="mean", padding_idx=0)


def embedding_bag_mean_closed_form(weight: torch.Tensor, values: torch.Tensor) -> torch.Tensor:
    """The expression the reference's own test and benchmark compare against (tests/unit/infrastructure/accelerators/
    test_tilelang_ops.py:134-137, application/benchmarking/pcvr_tilelang_ops_benchmark.py:171-174), in float32."""
    embedded = F.embedding(values.long(), weight.float(), padding_idx=0)
    valid = values.ne(0).to(embedded.dtype).unsqueeze(-1)
    return (embedded * valid).sum(dim=1) / valid.sum(dim=1).clamp_min(1.0)


# ---- model-level structured masks ------------------------------------------------------------------------------------


def bfts_attention_mask(padding_mask: torch.Tensor, role_ids: torch.Tensor, layer_index: int, num_layers: int, *,
                        seq_causal: bool, seq_keep_per_domain: int) -> torch.Tensor:
    """``PCVRTokenFormer._bfts_attention_mask`` (experiments/tokenformer/model.py:474-503) restated element by element
    (small inputs only): (B, 1, T, T) bool, True = attend. Roles: 3 = target, 4 = separator (model.py:32-37)."""
    batch, tokens = padding_mask.shape
    bottom = max(1, num_layers // 2)
    window = None if layer_index < bottom else max(4, math.ceil(seq_keep_per_domain / (2 ** (layer_index - bottom))))
    safe = safe_key_padding_mask(padding_mask)
    mask = torch.zeros(batch, 1, tokens, tokens, dtype=torch.bool)
    for b in range(batch):
        for i in range(tokens):
            if bool(padding_mask[b, i]):
                mask[b, 0, i, i] = True  # a padded query attends to itself only
                continue
            for j in range(tokens):
                if window is None:
                    seen = j <= i if seq_causal else True
                else:
                    seen = 0 <= i - j <= window if seq_causal else abs(i - j) <= window
                seen = seen or i == j or int(role_ids[i]) == 3 or int(role_ids[j]) == 4
                mask[b, 0, i, j] = seen and not bool(safe[b, j])
    return mask


_METADATA_VISIBLE_KEY_ROLES = {
    # query role -> key roles it may read (experiments/symbiosis/attention.py:29-58; roles: tokenization.py:22-30)
    0: set(range(8)), 1: set(range(8)), 7: set(range(8)),
    2: {0, 1, 2, 3, 4, 5, 7}, 3: {0, 1, 2, 3, 4, 5, 7}, 4: {0, 1, 2, 3, 4, 5, 7}, 5: {0, 1, 2, 3, 4, 5, 7},
    6: {0, 1, 3, 6, 5, 7},
}


def metadata_attention_mask(padding_mask: torch.Tensor, role_ids: torch.Tensor, *, enabled: bool = True) -> torch.Tensor:
    """``MetadataAttentionMask.forward`` (experiments/symbiosis/attention.py:22-60) restated element by element (small
    inputs only): (B, 1, T, T) bool."""
    batch, tokens = padding_mask.shape
    safe = safe_key_padding_mask(padding_mask)
    mask = torch.zeros(batch, 1, tokens, tokens, dtype=torch.bool)
    for b in range(batch):
        for i in range(tokens):
            for j in range(tokens):
                seen = True if not enabled else (i == j or int(role_ids[j]) in _METADATA_VISIBLE_KEY_ROLES[int(role_ids[i])])
                mask[b, 0, i, j] = seen and not bool(safe[b, j])
    return mask


# ---- query / key normalisation and rotary embedding ------------------------------------------------------------------


def rotate_half_pairs(values: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """``_rotate_half_pairs`` (experiments/tokenformer/model.py:131-136): features (2i, 2i + 1) are one plane, rotated
    by the angle of frequency i; evaluated in the dtype of ``values`` as the reference does."""
    even = values[..., 0::2]
    odd = values[..., 1::2]
    return torch.stack((even * cos - odd * sin, even * sin + odd * cos), dim=-1).flatten(-2)


def rope_tables(token_count: int, head_dim: int, rope_base: float, dtype: torch.dtype) -> tuple[torch.Tensor, torch.Tensor]:
    """cos / sin of ``position * rope_base ** (-2i / rotary_dim)`` rounded to the activation dtype
    (experiments/tokenformer/model.py:174-179): shape (tokens, rotary_dim / 2), rotary_dim = 2 * (head_dim // 2)."""
    rotary_dim = (head_dim // 2) * 2
    positions = torch.arange(token_count, dtype=torch.float32)
    frequencies = torch.arange(0, rotary_dim, 2, dtype=torch.float32)
    inv_freq = torch.pow(torch.tensor(float(rope_base)), -frequencies / max(1, rotary_dim))
    angles = positions[:, None] * inv_freq[None, :]
    return angles.cos().to(dtype), angles.sin().to(dtype)


def apply_rope(query: torch.Tensor, key: torch.Tensor, *, num_heads: int, rope_base: float) -> tuple[torch.Tensor, torch.Tensor]:
    """``BFTSAttention._apply_rope`` (experiments/tokenformer/model.py:165-192) on (B, T, D) projections: positions
    are the token indices 0..T-1, each head rotates its first rotary_dim features and keeps an odd last one."""
    batch, token_count, d_model = query.shape
    head_dim = d_model // num_heads
    rotary_dim = (head_dim // 2) * 2
    if rotary_dim <= 0:
        return query, key
    cos, sin = rope_tables(token_count, head_dim, rope_base, query.dtype)
    cos = cos.view(1, token_count, 1, -1)
    sin = sin.view(1, token_count, 1, -1)

    def rotate(values: torch.Tensor) -> torch.Tensor:
        heads = values.reshape(batch, token_count, num_heads, head_dim)
        rotated = rotate_half_pairs(heads[..., :rotary_dim], cos, sin)
        if rotary_dim != head_dim:
            rotated = torch.cat([rotated, heads[..., rotary_dim:]], dim=-1)
        return rotated.reshape(batch, token_count, d_model)

    return rotate(query), rotate(key)


def qk_norm_rope(query: torch.Tensor, key: torch.Tensor, query_weight: torch.Tensor | None,
                 key_weight: torch.Tensor | None, *, num_heads: int, eps: float = 1e-6, rope_base: float | None = None,
                 fp32: bool = False) -> tuple[torch.Tensor, torch.Tensor]:
    """What ``UnifiedSelfAttention.forward`` (experiments/symbiosis/backbone.py:33-36) and ``BFTSAttention.forward``
    (experiments/tokenformer/model.py:149-154) do to the query and key projections before attention: RMSNorm over the
    whole model width (not per head), then the rotary embedding when ``rope_base`` is given. ``fp32=True`` evaluates
    the same expressions in float32 from the stored inputs (tables still rounded to the storage dtype) and rounds once:
    the parity target of a fused kernel, as ``rms_norm_fp32`` is for the norm alone."""
    dtype = query.dtype
    if fp32:
        query, key = query.float(), key.float()
    if query_weight is not None:
        query = rms_norm(query, query_weight.to(dtype).to(query.dtype), eps)
        key = rms_norm(key, key_weight.to(dtype).to(key.dtype), eps)
    if rope_base is not None:
        if fp32:
            batch, token_count, d_model = query.shape
            head_dim = d_model // num_heads
            cos, sin = rope_tables(token_count, head_dim, rope_base, dtype)
            cos = cos.float().view(1, token_count, 1, -1)
            sin = sin.float().view(1, token_count, 1, -1)
            rotary_dim = (head_dim // 2) * 2

            def rotate(values: torch.Tensor) -> torch.Tensor:
                heads = values.reshape(batch, token_count, num_heads, head_dim)
                rotated = rotate_half_pairs(heads[..., :rotary_dim], cos, sin)
                if rotary_dim != head_dim:
                    rotated = torch.cat([rotated, heads[..., rotary_dim:]], dim=-1)
                return rotated.reshape(batch, token_count, d_model)

            query, key = rotate(query), rotate(key)
        else:
            query, key = apply_rope(query, key, num_heads=num_heads, rope_base=rope_base)
    return query.to(dtype), key.to(dtype)


# ---- readout ---------------------------------------------------------------------------------------------------------------


def candidate_readout(tokens: torch.Tensor, padding_mask: torch.Tensor | None, *, cls_index: int,
                      candidate_index: int | None, token_norm_weight: torch.Tensor | None,
                      pool_norm_weight: torch.Tensor | None, eps: float = 1e-6,
                      classifier: tuple[torch.Tensor, torch.Tensor | None, torch.Tensor, torch.Tensor | None] | None = None,
                      fp32: bool = True) -> tuple[torch.Tensor, torch.Tensor | None]:
    """``final_norm`` -> ``CandidateClsPooler.forward`` -> classifier of ``PCVRSymbiosis`` (experiments/symbiosis/
    model.py:215-222, 291, 309, 316-317; experiments/symbiosis/pooling.py:24-32): the pieces are ``rms_norm``,
    ``masked_mean`` and ``F.linear`` / ``F.silu`` above. ``fp32=True`` evaluates them in float32 from the stored operands
    (the parity target of a fused kernel), ``fp32=False`` in the tensors' own dtype as the reference does.
    Returns (pooled embedding (B, 3D), logits (B, actions) or None)."""
    cast = (lambda t: None if t is None else t.float()) if fp32 else (lambda t: t)
    x = cast(tokens)
    if token_norm_weight is not None:
        x = rms_norm(x, cast(token_norm_weight), eps)
    cls_summary = x[:, cls_index, :]
    candidate_summary = x[:, candidate_index, :] if candidate_index is not None else torch.zeros_like(cls_summary)
    pooled = torch.cat([cls_summary, candidate_summary, masked_mean(x, padding_mask)], dim=-1)
    if pool_norm_weight is not None:
        pooled = rms_norm(pooled, cast(pool_norm_weight), eps)
    if classifier is None:
        return pooled, None
    w1, b1, w2, b2 = (cast(t) for t in classifier)
    return pooled, F.linear(F.silu(F.linear(pooled, w1, b1)), w2, b2)


# ---- dense layers ----------------------------------------------------------------------------------------------------


def swiglu_ffn(x: torch.Tensor, up_weight: torch.Tensor, up_bias: torch.Tensor | None, down_weight: torch.Tensor,
               down_bias: torch.Tensor | None, *, gate_first: bool = True) -> torch.Tensor:
    """``SwiGLUFeedForward.forward`` in eval mode (experiments/symbiosis/backbone.py:19-21); ``gate_first=False`` is
    the Baseline convention ``x1 * silu(x2)`` (experiments/baseline/model.py:108-113)."""
    gate, value = F.linear(x, up_weight, up_bias).chunk(2, dim=-1)
    hidden = F.silu(gate) * value if gate_first else gate * F.silu(value)
    return F.linear(hidden, down_weight, down_bias)


def swiglu_hidden(x: torch.Tensor, up_weight: torch.Tensor, up_bias: torch.Tensor | None, *, gate_first: bool = True) -> torch.Tensor:
    gate, value = F.linear(x, up_weight, up_bias).chunk(2, dim=-1)
    return F.silu(gate) * value if gate_first else gate * F.silu(value)


def block(x: torch.Tensor, key_lengths: torch.Tensor, w: dict[str, torch.Tensor], *, num_heads: int, eps: float = 1e-6,
          rope_base: float | None = None) -> torch.Tensor:
    """One canonical pre-norm block: the recipe of ``UnifiedInteractionBlock.forward``
    (experiments/symbiosis/backbone.py:58-68) without the padding multiply on the updates (padded rows are
    don't-care), attention over the valid key prefix with padded query rows set to 0. The benchmark recipe has no
    QK-norm; with ``query_norm.weight`` / ``key_norm.weight`` in ``w`` the query and key are normalised over the model
    width as the reference layer does (backbone.py:33-36), with ``rope_base`` they are rotated (tokenformer/model.py:
    153-154)."""
    h = rms_norm(x, w["attn_norm.weight"], eps)
    q, k, v = F.linear(h, w["qkv.weight"], w.get("qkv.bias")).chunk(3, dim=-1)
    if "query_norm.weight" in w or rope_base is not None:
        q, k = qk_norm_rope(q, k, w.get("query_norm.weight"), w.get("key_norm.weight"), num_heads=num_heads, eps=eps,
                            rope_base=rope_base)
    a = scaled_dot_product_attention(q, k, v, num_heads=num_heads, key_lengths=key_lengths, zero_padded_queries=True)
    x = x + F.linear(a, w["out.weight"], w.get("out.bias"))
    h2 = rms_norm(x, w["ffn_norm.weight"], eps)
    return x + swiglu_ffn(h2, w["up.weight"], w.get("up.bias"), w["down.weight"], w.get("down.bias"))


def interaction_block(tokens: torch.Tensor, padding_mask: torch.Tensor, attention_mask: torch.Tensor | None,
                      w: dict[str, torch.Tensor], *, num_heads: int, eps: float = 1e-6,
                      rope_base: float | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """``UnifiedInteractionBlock.forward`` as written (experiments/symbiosis/backbone.py:58-68): both updates are
    multiplied by ``~padding_mask``, so padded rows pass through unchanged; ``attention_mask`` is the bool
    (B, 1 or H, T, T) mask the model's mask module built (True = attend) or None. Composed from the pinned pieces
    above. Returns (output, attn_tokens)."""
    batch, token_count, d_model = tokens.shape
    keep = (~padding_mask).unsqueeze(-1).to(tokens.dtype)
    h = rms_norm(tokens, w["attn_norm.weight"], eps)
    q, k, v = F.linear(h, w["qkv.weight"], w.get("qkv.bias")).chunk(3, dim=-1)
    if "query_norm.weight" in w or rope_base is not None:
        q, k = qk_norm_rope(q, k, w.get("query_norm.weight"), w.get("key_norm.weight"), num_heads=num_heads, eps=eps,
                            rope_base=rope_base)
    heads = lambda t: t.view(batch, token_count, num_heads, d_model // num_heads).transpose(1, 2)  # noqa: E731
    a = sdpa(heads(q), heads(k), heads(v), attn_mask=attention_mask).transpose(1, 2).reshape(batch, token_count, d_model)
    attn_tokens = tokens + F.linear(a, w["out.weight"], w.get("out.bias")) * keep
    h2 = rms_norm(attn_tokens, w["ffn_norm.weight"], eps)
    output = attn_tokens + swiglu_ffn(h2, w["up.weight"], w.get("up.bias"), w["down.weight"], w.get("down.bias")) * keep
    return output, attn_tokens


def tokenformer_block(tokens: torch.Tensor, padding_mask: torch.Tensor, attention_mask: torch.Tensor | None,
                      w: dict[str, torch.Tensor], *, num_heads: int, eps: float = 1e-6,
                      rope_base: float | None = None) -> torch.Tensor:
    """``TokenFormerBlock.forward`` as written (experiments/tokenformer/model.py:203-215): the attention layer
    (``BFTSAttention.forward``, :150-163: packed projection, RMSNorm(d_model) of query and key, optional rotary
    embedding, attention, out projection) reads ``attn_norm(tokens)``; its update is multiplied by
    ``sigmoid(nlir_gate(attn_norm(tokens)))`` and by ``~padding_mask`` before it joins the stream; the SwiGLU feed-forward
    update is multiplied by ``~padding_mask`` as well. ``w`` holds the block's parameters under the names of
    :func:`interaction_block` plus ``nlir_gate.weight`` / ``nlir_gate.bias``."""
    batch, token_count, d_model = tokens.shape
    keep = (~padding_mask).unsqueeze(-1).to(tokens.dtype)
    h = rms_norm(tokens, w["attn_norm.weight"], eps)
    q, k, v = F.linear(h, w["qkv.weight"], w.get("qkv.bias")).chunk(3, dim=-1)
    q, k = qk_norm_rope(q, k, w.get("query_norm.weight"), w.get("key_norm.weight"), num_heads=num_heads, eps=eps,
                        rope_base=rope_base)
    heads = lambda t: t.view(batch, token_count, num_heads, d_model // num_heads).transpose(1, 2)  # noqa: E731
    a = sdpa(heads(q), heads(k), heads(v), attn_mask=attention_mask).transpose(1, 2).reshape(batch, token_count, d_model)
    attention_update = F.linear(a, w["out.weight"], w.get("out.bias"))
    nlir_update = torch.sigmoid(F.linear(h, w["nlir_gate.weight"], w.get("nlir_gate.bias"))) * attention_update
    tokens = tokens + nlir_update * keep
    h2 = rms_norm(tokens, w["ffn_norm.weight"], eps)
    return tokens + swiglu_ffn(h2, w["up.weight"], w.get("up.bias"), w["down.weight"], w.get("down.bias")) * keep


def silu_mlp(x: torch.Tensor, fc1_weight: torch.Tensor, fc1_bias: torch.Tensor | None, fc2_weight: torch.Tensor,
             fc2_bias: torch.Tensor | None) -> torch.Tensor:
    """OneTrans' ``FeedForward.forward`` in eval mode (experiments/onetrans/model.py:33-44):
    ``Linear(d_model, d_model * hidden_mult) -> SiLU -> Dropout -> Linear(d_model * hidden_mult, d_model)``."""
    return F.linear(F.silu(F.linear(x, fc1_weight, fc1_bias)), fc2_weight, fc2_bias)


def mixed_feed_forward(tokens: torch.Tensor, seq_token_count: int, shared: tuple, ns_specific: list[tuple]) -> torch.Tensor:
    """OneTrans' ``MixedFeedForward.forward`` (experiments/onetrans/model.py:87-94): the shared feed-forward over every
    token, then the token at position ``seq_token_count + i`` is replaced by the output of the i-th token-specific
    feed-forward on that token (positions beyond the sequence are skipped). ``shared`` and every entry of
    ``ns_specific`` are ``(fc1_weight, fc1_bias, fc2_weight, fc2_bias)``."""
    output = silu_mlp(tokens, *shared).clone()
    for ns_index, weights in enumerate(ns_specific):
        position = seq_token_count + ns_index
        if position >= tokens.shape[1]:
            continue
        output[:, position, :] = silu_mlp(tokens[:, position, :], *weights)
    return output


def backbone(emb: torch.Tensor, key_lengths: torch.Tensor, blocks: list[dict[str, torch.Tensor]],
             head_weight: torch.Tensor, head_bias: torch.Tensor | None, *, num_heads: int, eps: float = 1e-6,
             return_hidden: bool = False, rope_base: float | None = None):
    """n pre-norm blocks (``_run_backbone``, experiments/symbiosis/model.py:283-292) + masked mean-pool
    (modeling/sequence.py:54-60) -> Linear(D, 1) -> sigmoid. Returns float32 probabilities [B]."""
    x = emb
    for w in blocks:
        x = block(x, key_lengths, w, num_heads=num_heads, eps=eps, rope_base=rope_base)
    padding = make_padding_mask(key_lengths.to(torch.int64), x.shape[1])
    pooled = masked_mean(x, padding)
    logits = F.linear(pooled, head_weight.reshape(1, -1), head_bias).squeeze(-1)
    probs = torch.sigmoid(logits.float())
    return (probs, x) if return_hidden else probs


# ---- FP8 emulation (no reference counterpart; parity unpinned, see the module docstring) -------------------------------


def fp8_scale(t: torch.Tensor) -> torch.Tensor:
    return t.float().abs().max().clamp_min(1e-12) / FP8_MAX


def fp8_quantize(t: torch.Tensor, scale: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """``q = (t / s).to(float8_e4m3fn)`` with ``s = amax / 448``. Returns (q, s)."""
    if scale is None:
        scale = fp8_scale(t)
    q = (t.float() / scale).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, scale


def linear_fp8(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None, *,
               residual: torch.Tensor | None = None, swiglu: bool = False, gate_first: bool = True,
               x_scale: torch.Tensor | None = None, w_scale: torch.Tensor | None = None) -> torch.Tensor:
    """quantize -> matmul -> dequantize emulation: ``y = (qx.float() @ qw.float().T) * s_x * s_w`` (+ bias), then the
    fp32 epilogue (SiLU-gate or residual) and one rounding to bf16."""
    qx, sx = fp8_quantize(x, x_scale)
    qw, sw = fp8_quantize(weight, w_scale)
    y = torch.matmul(qx.float(), qw.float().t()) * (sx * sw)
    if bias is not None:
        y = y + bias.float()
    if swiglu:
        gate, value = y.chunk(2, dim=-1)
        y = F.silu(gate) * value if gate_first else gate * F.silu(value)
    if residual is not None:
        y = y + residual.float()
    return y.to(torch.bfloat16)


def swiglu_ffn_fp8(x: torch.Tensor, norm_weight: torch.Tensor | None, up_weight: torch.Tensor, up_bias: torch.Tensor | None,
                   down_weight: torch.Tensor, down_bias: torch.Tensor | None, *, residual: torch.Tensor | None = None,
                   eps: float = 1e-6, gate_first: bool = True) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """The feed-forward half as a chain of two ``linear_fp8`` layers on bf16 tensors (FP8 configuration of the dense
    layers; experiments/symbiosis/backbone.py:19-21, 66-67 for the recipe): ``h = rmsnorm(x)`` in fp32 statistics, one
    rounding; ``hidden = linear_fp8(h, up, swiglu=True)``; ``out = linear_fp8(hidden, down, residual=residual)``, every
    tensor quantised with its own ``amax / 448``. Returns (out, hidden, h). Parity unpinned by the reference like
    ``linear_fp8`` itself; composed from it only."""
    h = x if norm_weight is None else rms_norm_fp32(x, norm_weight, eps)
    hidden = linear_fp8(h, up_weight, up_bias, swiglu=True, gate_first=gate_first)
    out = linear_fp8(hidden, down_weight, down_bias, residual=residual)
    return out, hidden, h


def block_fp8(x: torch.Tensor, key_lengths: torch.Tensor, w: dict[str, torch.Tensor], *, num_heads: int, eps: float = 1e-6,
              valid_only: bool = False, maxima: dict[str, torch.Tensor] | None = None) -> torch.Tensor:
    """``block`` with its four dense layers replaced by ``linear_fp8`` (qkv, out, up, down; the recipe of
    experiments/symbiosis/backbone.py:58-68, plain attention layer). ``valid_only=True`` takes every activation scale
    over the rows before ``key_lengths`` only, which is what a route that never touches the padded positions computes;
    the padded rows of the result are then don't-care. ``maxima`` fixes the per-tensor maxima of the four activations
    (keys "attn_norm", "attention", "ffn_norm", "hidden") instead of taking them from ``x`` - for a slice of a batch
    whose scales were taken over the whole batch. Parity unpinned like ``linear_fp8``; composed from it only."""
    keep = ~make_padding_mask(key_lengths.to(torch.int64), x.shape[1])

    def scale_of(name: str, t: torch.Tensor) -> torch.Tensor | None:
        if maxima is not None:
            return maxima[name].float().clamp_min(1e-12) / FP8_MAX
        return fp8_scale(t[keep]) if valid_only else None

    h = rms_norm_fp32(x, w["attn_norm.weight"], eps)
    q, k, v = linear_fp8(h, w["qkv.weight"], w.get("qkv.bias"), x_scale=scale_of("attn_norm", h)).chunk(3, dim=-1)
    a = scaled_dot_product_attention(q, k, v, num_heads=num_heads, key_lengths=key_lengths, zero_padded_queries=True)
    x = linear_fp8(a, w["out.weight"], w.get("out.bias"), residual=x, x_scale=scale_of("attention", a))
    h2 = rms_norm_fp32(x, w["ffn_norm.weight"], eps)
    hidden = linear_fp8(h2, w["up.weight"], w.get("up.bias"), swiglu=True, x_scale=scale_of("ffn_norm", h2))
    return linear_fp8(hidden, w["down.weight"], w.get("down.bias"), residual=x, x_scale=scale_of("hidden", hidden))


def backbone_fp8(emb: torch.Tensor, key_lengths: torch.Tensor, blocks: list[dict[str, torch.Tensor]],
                 head_weight: torch.Tensor, head_bias: torch.Tensor | None, *, num_heads: int, eps: float = 1e-6,
                 return_hidden: bool = False, valid_only: bool = False,
                 maxima: list[dict[str, torch.Tensor]] | None = None):
    """``backbone`` over ``block_fp8``; the pooled readout stays in the activation dtype."""
    x = emb
    for index, w in enumerate(blocks):
        x = block_fp8(x, key_lengths, w, num_heads=num_heads, eps=eps, valid_only=valid_only,
                      maxima=None if maxima is None else maxima[index])
    padding = make_padding_mask(key_lengths.to(torch.int64), x.shape[1])
    pooled = masked_mean(x, padding)
    logits = F.linear(pooled, head_weight.reshape(1, -1), head_bias).squeeze(-1)
    probs = torch.sigmoid(logits.float())
    return (probs, x) if return_hidden else probs
