"""GPU parity: attention under structured masks (structural[query, key] & key_valid[batch, key], optional self-only query
rows) through the C ABI, against the library SDPA with the dense bool mask and the oracle's per-element mask rules."""

from __future__ import annotations

from dataclasses import replace

import pytest
import torch
import torch.nn.functional as F

from oracle import reference as oracle
from taac_2026_amd.api import (
    MetadataAttentionMask,
    bfts_attention_mask,
    build_structured_mask,
    flash_attention,
    scaled_dot_product_attention,
)

pytestmark = pytest.mark.gpu

BF16_TOL = dict(rtol=2e-2, atol=2e-2)


def _qkv(batch, heads, tokens, dim, seed):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(batch, heads, tokens, dim, generator=g).to(torch.bfloat16) for _ in range(3))


def _expected(q, k, v, dense):
    """Library SDPA with the bool mask (the reference's torch backend, flash_attention.py:552-570); rows without any
    visible key are defined as zeros, as the kernel and the reference's TileLang kernel define them."""
    empty = ~dense.any(dim=-1, keepdim=True)
    out = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=dense | empty)
    return torch.where(empty.expand(-1, q.shape[1], -1, -1), torch.zeros_like(out), out)


@pytest.mark.parametrize("sparse", [False, True])
@pytest.mark.parametrize("tokens,dim", [(50, 32), (130, 64), (300, 32), (512, 32), (97, 128)])
def test_random_structured_masks(device, tokens, dim, sparse):
    """``sparse``: the kernel that gives every 32-query tile its own wavefront (head dims 32 and 64; 128 runs the chunked
    kernel either way)."""
    batch, heads = 3, 2
    q, k, v = _qkv(batch, heads, tokens, dim, tokens + dim)
    g = torch.Generator().manual_seed(tokens)
    structural = torch.rand(tokens, tokens, generator=g) < 0.4
    structural[tokens // 3] = False                     # a query row that sees nothing: zeros
    key_valid = torch.rand(batch, tokens, generator=g) < 0.7
    key_valid[1] = True
    query_self = torch.rand(batch, tokens, generator=g) < 0.1
    with torch.no_grad():
        plain = build_structured_mask(structural.to(device), key_valid.to(device), sparse=sparse)
        with_self = build_structured_mask(structural.to(device), key_valid.to(device), query_self.to(device), sparse=sparse)
        only_structural = build_structured_mask(structural.to(device), sparse=sparse)
        args = (q.to(device), k.to(device), v.to(device))
        got = flash_attention(*args, structured_mask=plain).cpu()
        got_self = flash_attention(*args, structured_mask=with_self).cpu()
        got_struct = flash_attention(*args, structured_mask=only_structural).cpu()
    dense = (structural[None] & key_valid[:, None, :])[:, None]
    assert torch.equal(plain.dense().cpu(), dense)
    torch.testing.assert_close(got.float(), _expected(q, k, v, dense), **BF16_TOL)
    assert got[:, :, tokens // 3].abs().max().item() == 0.0
    torch.testing.assert_close(got_struct.float(), _expected(q, k, v, structural[None, None].expand(batch, 1, -1, -1)), **BF16_TOL)
    # self-only rows return their value row bit for bit; the other rows are unchanged
    flagged = query_self[:, None, :, None].expand_as(got_self)
    assert torch.equal(got_self[flagged], v[flagged])
    assert torch.equal(got_self[~flagged], got[~flagged])
    assert torch.equal(with_self.dense().cpu(), torch.where(query_self[:, None, :, None], torch.eye(tokens, dtype=torch.bool)[None, None], dense))


@pytest.mark.parametrize("seq_causal", [True, False])
def test_tokenformer_layer_masks(device, seq_causal):
    """Every layer's mask of a TokenFormer-like token layout (bottom layers full, upper layers sliding windows that shrink
    by halves; separators seen by everyone, the target sees everyone, padded queries keep themselves): the factored mask
    equals the oracle's per-element rule, and attention under it equals SDPA with the dense mask. At 512 tokens the
    narrow windows leave most (query block, key chunk) pairs empty - those are skipped by the kernel."""
    batch, heads, dim, layers = 3, 2, 32, 6
    roles = torch.tensor([0] * 20 + [4] + [1] * 460 + [4] + [2] * 20 + [5] * 9 + [3])
    tokens = roles.numel()
    assert tokens == 512
    g = torch.Generator().manual_seed(3)
    padding = torch.zeros(batch, tokens, dtype=torch.bool)
    padding[1, 200:481] = True
    padding[2, 21 + 37:481] = True
    padding[2, 5] = True
    q, k, v = _qkv(batch, heads, tokens, dim, 5)
    for layer in range(layers):
        with torch.no_grad():
            mask = bfts_attention_mask(padding.to(device), roles.to(device), layer, layers, seq_causal=seq_causal,
                                       seq_keep_per_domain=64)
            got = flash_attention(q.to(device), k.to(device), v.to(device), structured_mask=mask).cpu()
            other = flash_attention(q.to(device), k.to(device), v.to(device),
                                    structured_mask=replace(mask, sparse=not mask.sparse)).cpu()
        assert mask.sparse == (layer >= 3)               # the window layers prefer the per-tile kernel
        dense = mask.dense().cpu()
        torch.testing.assert_close(other.float(), got.float(), rtol=2 ** -6, atol=2 ** -6)   # same result from either kernel
        if layer in (0, 3, 5):  # the per-element oracle is slow: three layers cover full, first and narrowest window
            assert torch.equal(dense[:1], oracle.bfts_attention_mask(padding[:1], roles, layer, layers, seq_causal=seq_causal,
                                                                      seq_keep_per_domain=64))
        torch.testing.assert_close(got.float(), _expected(q, k, v, dense), **BF16_TOL)
        if layer == 5:  # window max(4, 64 / 4) = 16: far-away key chunks of the sequence span are empty for a query block
            assert mask.block_any.cpu()[1].tolist().count(0) >= 2


def test_symbiosis_metadata_mask(device):
    batch, heads, dim = 4, 4, 64
    roles = torch.tensor([0, 1] + [2] * 9 + [3] * 7 + [4] * 3 + [5] * 2 + [6] * 150 + [7] * 4)
    tokens = roles.numel()
    g = torch.Generator().manual_seed(1)
    padding = torch.rand(batch, tokens, generator=g) < 0.3
    padding[:, :2] = False
    padding[3] = True                                           # an all-padded sample keeps key 0 (safe mask)
    q, k, v = _qkv(batch, heads, tokens, dim, 2)
    for enabled in (True, False):
        module = MetadataAttentionMask(enabled=enabled)
        with torch.no_grad():
            mask = module(padding.to(device), roles.to(device))
            got = flash_attention(q.to(device), k.to(device), v.to(device), structured_mask=mask).cpu()
            per_tile = flash_attention(q.to(device), k.to(device), v.to(device), structured_mask=replace(mask, sparse=True)).cpu()
        dense = mask.dense().cpu()
        torch.testing.assert_close(per_tile.float(), _expected(q, k, v, dense), **BF16_TOL)
        assert torch.equal(dense[:2], oracle.metadata_attention_mask(padding[:2], roles, enabled=enabled))
        assert dense[:, :, 0, :].any(dim=-1).all() and dense[:, :, 1, :].any(dim=-1).all()   # the reference's own check
        torch.testing.assert_close(got.float(), _expected(q, k, v, dense), **BF16_TOL)


def test_dense_bool_masks_are_factored(device):
    """A (B, 1, T, T) or (B, H, T, T) bool mask that is neither a key prefix nor causal-valid is factored and verified by
    the planner (the reference's accelerated path rejects it and runs torch SDPA); masks without the factored form are
    refused with a RuntimeError."""
    batch, heads, tokens, dim = 3, 2, 70, 32
    roles = torch.tensor([0] * 5 + [4] + [1] * 50 + [4] + [2] * 12 + [3])
    padding = torch.zeros(batch, tokens, dtype=torch.bool)
    padding[1, 30:56] = True
    q, k, v = _qkv(batch, heads, tokens, dim, 9)
    dense = oracle.bfts_attention_mask(padding, roles, 2, 4, seq_causal=True, seq_keep_per_domain=8)
    expected = _expected(q, k, v, dense)
    with torch.no_grad():
        args = (q.to(device), k.to(device), v.to(device))
        got1 = flash_attention(*args, attn_mask=dense.to(device)).cpu()
        got_h = flash_attention(*args, attn_mask=dense.expand(-1, heads, -1, -1).contiguous().to(device)).cpu()
        torch.testing.assert_close(got1.float(), expected, **BF16_TOL)
        assert torch.equal(got1, got_h)
        # (B, T, D) front end used by the model packages
        q3, k3, v3 = (t.transpose(1, 2).reshape(batch, tokens, heads * dim).to(device) for t in (q, k, v))
        got3 = scaled_dot_product_attention(q3, k3, v3, num_heads=heads, attn_mask=dense.to(device), dropout_p=0.0,
                                            training=False).cpu()
        torch.testing.assert_close(got3.view(batch, tokens, heads, dim).transpose(1, 2).float(), expected, **BF16_TOL)
        bad = dense.clone()
        bad[0, 0, 10, 3] = ~bad[0, 0, 10, 3]        # differs between samples in a way no key_valid explains
        bad[1, 0, 10, 3] = ~bad[0, 0, 10, 3]
        with pytest.raises(RuntimeError, match="structural"):
            flash_attention(*args, attn_mask=bad.to(device))
        per_head = dense.expand(-1, heads, -1, -1).clone()
        per_head[:, 1, 4, 2] = ~per_head[:, 1, 4, 2]
        with pytest.raises(RuntimeError, match="shared across heads"):
            flash_attention(*args, attn_mask=per_head.to(device))


@pytest.mark.parametrize("sparse", [False, True])
@pytest.mark.parametrize("dim", [32, 64])
def test_structured_mask_with_key_lengths_and_row_factors(device, sparse, dim):
    from taac_2026_amd.accelerators.attention import hip_flash_attention_kernel

    batch, heads, tokens = 3, 2, 160
    q, k, v = _qkv(batch, heads, tokens, dim, 4)
    g = torch.Generator().manual_seed(6)
    structural = (torch.arange(tokens)[:, None] - torch.arange(tokens)[None, :]).abs() <= 20
    lengths = torch.tensor([160, 33, 97], dtype=torch.int32)
    sq = 0.5 + torch.rand(batch, tokens, generator=g)
    sk = 0.5 + torch.rand(batch, tokens, generator=g)
    key_valid = torch.arange(tokens)[None, :] < lengths[:, None]
    dense = (structural[None] & key_valid[:, None, :])[:, None]
    expected = _expected(q.float() * sq[:, None, :, None], k.float() * sk[:, None, :, None], v, dense)
    expected = expected * key_valid[:, None, :, None]     # zero_padded_queries
    with torch.no_grad():
        mask = build_structured_mask(structural.to(device), sparse=sparse)
        got = hip_flash_attention_kernel(q.to(device), k.to(device), v.to(device), lengths.to(device),
                                         zero_padded_queries=True, q_row_scale=sq.to(device), k_row_scale=sk.to(device),
                                         structured_mask=mask).cpu()
        with pytest.raises(ValueError, match="causal"):
            hip_flash_attention_kernel(q.to(device), k.to(device), v.to(device), None, is_causal=True, structured_mask=mask)
    torch.testing.assert_close(got.float(), expected, **BF16_TOL)


@pytest.mark.parametrize("dim", [32, 64])
def test_per_tile_kernel_ignores_the_rows_of_invalid_keys_and_padded_queries(device, dim):
    """Scattered padding, NaN in the q / k / v rows of padded positions (a caller that skips them never writes them): the
    valid rows are unchanged, padded query rows return their value row (self-only), tiles nobody sees cost nothing."""
    batch, heads, tokens = 4, 2, 200
    q, k, v = _qkv(batch, heads, tokens, dim, 11)
    g = torch.Generator().manual_seed(12)
    padding = torch.rand(batch, tokens, generator=g) < 0.4
    padding[0] = False
    padding[3, 40:] = True
    positions = torch.arange(tokens)
    distance = positions[:, None] - positions[None, :]
    structural = ((distance >= 0) & (distance <= 9)) | (positions[None, :] == 7) | (positions[:, None] == tokens - 1)
    poisoned = [t.clone() for t in (q, k, v)]
    for t in poisoned[:2]:
        t[padding[:, None, :, None].expand_as(t)] = float("nan")
    with torch.no_grad():
        mask = build_structured_mask(structural.to(device), (~padding).to(device), padding.to(device), sparse=True)
        clean = flash_attention(q.to(device), k.to(device), v.to(device), structured_mask=mask).cpu()
        got = flash_attention(*(t.to(device) for t in poisoned), structured_mask=mask).cpu()
        chunked = flash_attention(q.to(device), k.to(device), v.to(device), structured_mask=replace(mask, sparse=False)).cpu()
    dense = (structural[None] & ~padding[:, None, :])[:, None]
    valid = (~padding)[:, None, :, None].expand_as(got)
    assert torch.equal(got[valid], clean[valid]) and torch.isfinite(got[valid]).all()
    torch.testing.assert_close(clean.float()[valid], _expected(q, k, v, dense)[valid], **BF16_TOL)
    assert torch.equal(clean[~valid], v[~valid])                 # self-only rows: the value row, bit for bit
    torch.testing.assert_close(clean.float(), chunked.float(), rtol=2 ** -6, atol=2 ** -6)


def test_per_tile_kernel_at_the_headline_attention_shape(device):
    """B=1024, H=8, T=512, head dim 32 under TokenFormer's narrowest window layer (2.3 % of the pairs visible): the
    per-tile kernel against the chunked kernel on every sample, and a slice of samples against SDPA with the dense mask."""
    batch, heads, tokens, dim, layers = 1024, 8, 512, 32, 6
    g = torch.Generator().manual_seed(42)
    qkv = torch.randn(batch, tokens, 3 * heads * dim, generator=g).to(torch.bfloat16).to(device)
    q, k, v = (t.view(batch, tokens, heads, dim).transpose(1, 2) for t in qkv.chunk(3, dim=-1))
    roles = torch.tensor([0] * 20 + [4] + [1] * 460 + [4] + [2] * 20 + [5] * 9 + [3], device=device)
    span = torch.randint(32, 461, (batch,), generator=g).to(device)
    positions = torch.arange(tokens, device=device)
    padding = (positions[None, :] >= 21 + span[:, None]) & (positions[None, :] < 481)
    with torch.no_grad():
        mask = bfts_attention_mask(padding, roles, 5, layers, seq_causal=True, seq_keep_per_domain=64)
        assert mask.sparse
        got = flash_attention(q, k, v, structured_mask=mask)
        chunked = flash_attention(q, k, v, structured_mask=replace(mask, sparse=False))
    torch.testing.assert_close(got.float(), chunked.float(), rtol=2 ** -6, atol=2 ** -6)
    pick = torch.tensor([0, 333, 1023])
    dense = mask.dense()[pick.to(device)].cpu()
    want = _expected(q[pick.to(device)].cpu(), k[pick.to(device)].cpu(), v[pick.to(device)].cpu(), dense)
    self_rows = padding[pick.to(device)].cpu()[:, None, :, None].expand_as(want)
    torch.testing.assert_close(got[pick.to(device)].cpu().float()[~self_rows], want[~self_rows], **BF16_TOL)
    assert torch.equal(got[pick.to(device)].cpu()[self_rows], v[pick.to(device)].cpu()[self_rows])


def test_compact_tables_follow_their_definition(device):
    """``taac_mask_compact``: per 32-query tile the ascending list of visible key columns, per compact tile of 32 such keys
    the key words it draws from, per query row one word per compact tile - against loops over a random structure."""
    from taac_2026_amd.accelerators.attention import _compact_tables

    tokens_q, tokens_k = 70, 200
    g = torch.Generator().manual_seed(5)
    structural = torch.rand(tokens_q, tokens_k, generator=g) < 0.08
    structural[40:] &= torch.arange(tokens_k)[None, :] < 90            # a tile with few columns
    mask = build_structured_mask(structural.to(device), sparse=True)
    bits, keys, tile_words = (t.cpu() for t in _compact_tables(mask, 1))
    words = (tokens_k + 31) // 32
    assert bits.shape == (1, tokens_q, words) and keys.shape == (1, 3, 32 * words) and tile_words.shape == (1, 3, 64)
    for tile in range(3):
        rows = structural[tile * 32:(tile + 1) * 32]
        columns = rows.any(dim=0).nonzero().flatten().tolist()
        assert keys[0, tile, :len(columns)].tolist() == columns and (keys[0, tile, len(columns):] == -1).all()
        for c in range(64):
            chunk = columns[c * 32:(c + 1) * 32]
            expected = 0
            for key in chunk:
                expected |= 1 << (key // 32)
            assert int(tile_words[0, tile, c]) == expected
        for r in range(rows.shape[0]):
            for c in range(words):
                chunk = columns[c * 32:(c + 1) * 32]
                expected = sum(1 << j for j, key in enumerate(chunk) if bool(rows[r, key]))
                assert int(bits[0, tile * 32 + r, c]) & 0xffffffff == expected


# ---- training under structured masks ---------------------------------------------------------------------------------

# Gradient tolerance of the reference's GPU tests for 16-bit attention (tests/gpu/infrastructure/accelerators/
# test_tilelang_ops_cuda.py:98-141): 3e-2.
GRAD_TOL = dict(rtol=3e-2, atol=3e-2)


def _autograd_expected(q, k, v, dense, grad_out):
    """float64 autograd of the oracle's SDPA under the dense bool mask (what the reference's models train with,
    flash_attention.py:552-570); rows without a visible key are zeros and pass no gradient."""
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    empty = ~dense.any(dim=-1, keepdim=True)
    out = oracle.sdpa(qr, kr, vr, dense | empty)
    out = torch.where(empty.expand(-1, q.shape[1], -1, -1), torch.zeros_like(out), out)
    out.backward(grad_out.double())
    return out.detach(), qr.grad, kr.grad, vr.grad


def _check_training(device, q, k, v, mask, grad_out, key_lengths=None, dense=None):
    dense = mask.dense().cpu() if dense is None else dense
    want_out, *want_grads = _autograd_expected(q, k, v, dense, grad_out)
    qd, kd, vd = (t.to(device).requires_grad_(True) for t in (q, k, v))
    out = flash_attention(qd, kd, vd, structured_mask=mask, key_lengths=key_lengths)
    with torch.no_grad():
        serving = flash_attention(qd, kd, vd, structured_mask=mask, key_lengths=key_lengths)
    if mask.sparse:                                    # serving prefers the per-tile kernel there; training runs the chunked one
        torch.testing.assert_close(out.detach().float(), serving.float(), rtol=2 ** -6, atol=2 ** -6)
    else:                                              # the training forward is the serving kernel plus the log-sum-exp
        assert torch.equal(out.detach(), serving)
    out.backward(grad_out.to(device))
    torch.testing.assert_close(out.detach().cpu().double(), want_out, **BF16_TOL)
    for got, want, name in zip((qd.grad, kd.grad, vd.grad), want_grads, ("dq", "dk", "dv")):
        assert got.dtype == q.dtype and got.shape == want.shape
        torch.testing.assert_close(got.cpu().double(), want, msg=lambda m, n=name: f"{n}: {m}", **GRAD_TOL)
    return qd.grad.cpu(), kd.grad.cpu(), vd.grad.cpu()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tokens,dim", [(50, 32), (130, 64), (300, 32), (257, 16), (96, 48), (1100, 32)])
def test_structured_masks_take_a_gradient(device, dtype, tokens, dim):
    """Random structure, invalid keys, self-only queries and a query that sees nothing: the gradients equal float64
    autograd under the dense mask; invisible keys and the empty query row receive exactly zero."""
    batch, heads = 3, 2
    g = torch.Generator().manual_seed(tokens * 3 + dim)
    q, k, v, grad_out = (torch.randn(batch, heads, tokens, dim, generator=g).to(dtype) for _ in range(4))
    structural = torch.rand(tokens, tokens, generator=g) < 0.4
    structural[tokens // 3] = False
    key_valid = torch.rand(batch, tokens, generator=g) < 0.7
    key_valid[1] = True
    query_self = torch.rand(batch, tokens, generator=g) < 0.1
    query_self[:, tokens // 3] = False
    for mask in (build_structured_mask(structural.to(device), key_valid.to(device), query_self.to(device)),
                 build_structured_mask(structural.to(device), key_valid.to(device)),
                 build_structured_mask(structural.to(device))):
        dq, dk, dv = _check_training(device, q, k, v, mask, grad_out)
        assert dq[:, :, tokens // 3].abs().max().item() == 0.0
        if mask.key_valid is not None and mask.query_self is None:
            dead = ~key_valid[:, None, :, None].expand_as(dk)
            assert dk[dead].abs().max().item() == 0.0 and dv[dead].abs().max().item() == 0.0
        if mask.query_self is not None:                # a self-only query passes its gradient to its own value row only
            flagged = query_self[:, None, :, None].expand_as(dq)
            assert dq[flagged].abs().max().item() == 0.0


def test_model_masks_take_a_gradient(device):
    """The masks the reference's models build: TokenFormer layers (full, first and narrowest window, padded queries keep
    themselves - experiments/tokenformer/model.py:474-503) and the Symbiosis role mask
    (experiments/symbiosis/attention.py:21-60)."""
    batch, heads, dim, layers = 3, 2, 32, 6
    roles = torch.tensor([0] * 20 + [4] + [1] * 460 + [4] + [2] * 20 + [5] * 9 + [3])
    tokens = roles.numel()
    padding = torch.zeros(batch, tokens, dtype=torch.bool)
    padding[1, 200:481] = True
    padding[2, 21 + 37:481] = True
    padding[2, 5] = True
    g = torch.Generator().manual_seed(11)
    q, k, v, grad_out = (torch.randn(batch, heads, tokens, dim, generator=g).to(torch.bfloat16) for _ in range(4))
    for layer in (0, 3, 5):
        mask = bfts_attention_mask(padding.to(device), roles.to(device), layer, layers, seq_causal=True, seq_keep_per_domain=64)
        _check_training(device, q, k, v, mask, grad_out)
    roles = torch.tensor([0, 1] + [2] * 9 + [3] * 7 + [4] * 3 + [5] * 2 + [6] * 150 + [7] * 4)
    tokens = roles.numel()
    padding = torch.rand(4, tokens, generator=g) < 0.3
    padding[:, :2] = False
    padding[3] = True
    q, k, v, grad_out = (torch.randn(4, 4, tokens, 64, generator=g).to(torch.bfloat16) for _ in range(4))
    mask = MetadataAttentionMask(enabled=True)(padding.to(device), roles.to(device))
    _check_training(device, q, k, v, mask, grad_out)


def test_structured_mask_gradient_with_key_lengths(device):
    """``key_lengths`` on top of the structure (keys beyond the prefix invisible, padded query rows zero)."""
    batch, heads, tokens, dim = 3, 2, 200, 32
    g = torch.Generator().manual_seed(4)
    q, k, v, grad_out = (torch.randn(batch, heads, tokens, dim, generator=g).to(torch.bfloat16) for _ in range(4))
    structural = torch.tril(torch.ones(tokens, tokens, dtype=torch.bool)) & (torch.rand(tokens, tokens, generator=g) < 0.8)
    structural |= torch.eye(tokens, dtype=torch.bool)
    lengths = torch.tensor([200, 33, 129], dtype=torch.int32)
    inside = torch.arange(tokens)[None, :] < lengths[:, None]
    dense = (structural[None] & inside[:, None, :])[:, None]
    mask = build_structured_mask(structural.to(device))
    _check_training(device, q, k, v, mask, grad_out, key_lengths=lengths.to(device), dense=dense)


@pytest.mark.parametrize("per_head,per_sample,with_valid", [(True, True, False), (False, True, False), (True, False, False),
                                                          (False, False, False), (False, False, True), (True, False, True)])
def test_mask_bwd_abi_reads_any_bool_mask(device, per_head, per_sample, with_valid):
    """``taac_flash_attn_mask_bwd`` alone: a random mask per sample and / or head (strides 0 = shared), optionally times a
    key validity per sample, the log-sum-exp and the output taken from the float64 reference."""
    from taac_2026_amd import _native

    batch, heads, tokens, dim = 2, 3, 150, 64
    g = torch.Generator().manual_seed(int(per_head) * 2 + int(per_sample))
    q, k, v, grad_out = (torch.randn(batch, heads, tokens, dim, generator=g).to(torch.bfloat16) for _ in range(4))
    visible = torch.rand(batch if per_sample else 1, heads if per_head else 1, tokens, tokens, generator=g) < 0.5
    visible[..., 0] = True                              # every query sees a key
    dense = visible.expand(batch, heads, -1, -1)
    key_valid = None
    if with_valid:
        key_valid = torch.rand(batch, tokens, generator=g) < 0.7
        key_valid[:, 0] = True
        dense = dense & key_valid[:, None, None, :]
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    scores = (qr @ kr.transpose(-1, -2)) / dim ** 0.5
    scores = scores.masked_fill(~dense, float("-inf"))
    lse = torch.logsumexp(scores, dim=-1)
    out = torch.softmax(scores, dim=-1) @ vr
    out.backward(grad_out.double())
    dev = [t.to(device) for t in (q, k, v, out.detach().to(torch.bfloat16), grad_out)]
    lse_d = lse.detach().float().to(device)
    vis_d = visible.to(torch.uint8).contiguous().to(device)
    valid_d = None if key_valid is None else key_valid.to(torch.uint8).contiguous().to(device)
    grads = [torch.empty_like(dev[0]) for _ in range(3)]
    delta = torch.empty_like(lse_d)
    strides = [_native.Int64x4(*t.stride()) for t in (*dev, *grads)]
    status = _native.load_library().taac_flash_attn_mask_bwd(
        *(t.data_ptr() for t in dev), lse_d.data_ptr(), None, vis_d.data_ptr(),
        heads * tokens * tokens if per_sample and per_head else (tokens * tokens if per_sample else 0),
        tokens * tokens if per_head else 0, None if key_valid is None else valid_d.data_ptr(),
        *(t.data_ptr() for t in grads), delta.data_ptr(), batch, heads, tokens,
        tokens, dim, *strides, 0, _native.dtype_code(torch.bfloat16), _native.current_stream(dev[0].device))
    _native.check(status, "taac_flash_attn_mask_bwd")
    for got, want, name in zip(grads, (qr.grad, kr.grad, vr.grad), ("dq", "dk", "dv")):
        torch.testing.assert_close(got.cpu().double(), want, msg=lambda m, n=name: f"{n}: {m}", **GRAD_TOL)


@pytest.mark.parametrize("tokens,dim,with_lengths", [(130, 32, False), (200, 64, True), (96, 16, False)])
def test_structured_mask_with_dropout_takes_a_gradient(device, tokens, dim, with_lengths):
    """Dropout on the probabilities under a structured mask with a fixed keep mask - what the reference's models train
    with by default (``F.scaled_dot_product_attention(attn_mask=, dropout_p=)``, experiments/symbiosis/__init__.py:87):
    output and gradients against float64 autograd of the oracle's closed form (normaliser over the visible keys, then
    keep / (1 - p))."""
    batch, heads, dropout_p = 3, 2, 0.125
    g = torch.Generator().manual_seed(tokens + dim)
    q, k, v, grad_out = (torch.randn(batch, heads, tokens, dim, generator=g).to(torch.bfloat16) for _ in range(4))
    structural = (torch.rand(tokens, tokens, generator=g) < 0.5) | torch.eye(tokens, dtype=torch.bool)
    structural[tokens // 2] = False                     # a query that sees nothing
    key_valid = torch.rand(batch, tokens, generator=g) < 0.7
    key_valid[1] = True
    keep = (torch.rand(batch, heads, tokens, tokens, generator=g) >= dropout_p).to(torch.uint8)
    lengths = torch.tensor([tokens, tokens // 3, tokens - 5], dtype=torch.int32) if with_lengths else None
    dense = (structural[None] & key_valid[:, None, :])[:, None]
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    want = oracle.attention_dropout(qr, kr, vr, lengths, keep, dropout_p, attn_mask=dense)
    want.backward(grad_out.double())
    mask = build_structured_mask(structural.to(device), key_valid.to(device))
    qd, kd, vd = (t.to(device).requires_grad_(True) for t in (q, k, v))
    out = flash_attention(qd, kd, vd, structured_mask=mask, key_lengths=None if lengths is None else lengths.to(device),
                          dropout_p=dropout_p, training=True, dropout_mask=keep.to(device))
    out.backward(grad_out.to(device))
    torch.testing.assert_close(out.detach().cpu().double(), want.detach(), **BF16_TOL)
    assert out[:, :, tokens // 2].abs().max().item() == 0.0
    for got, ref, name in zip((qd.grad, kd.grad, vd.grad), (qr.grad, kr.grad, vr.grad), ("dq", "dk", "dv")):
        torch.testing.assert_close(got.cpu().double(), ref, msg=lambda m, n=name: f"{n}: {m}", **GRAD_TOL)
    # a keep mask of ones at a vanishing rate is the plain masked attention
    ones = torch.ones_like(keep).to(device)
    same = flash_attention(qd.detach(), kd.detach(), vd.detach(), structured_mask=mask,
                           key_lengths=None if lengths is None else lengths.to(device), dropout_p=1e-9, training=True,
                           dropout_mask=ones)
    plain = flash_attention(qd.detach(), kd.detach(), vd.detach(), structured_mask=mask,
                            key_lengths=None if lengths is None else lengths.to(device))
    torch.testing.assert_close(same.float(), plain.float(), rtol=2 ** -6, atol=2 ** -6)
    # self-only queries: probability 1 on their own key, kept or dropped like any other
    if lengths is None:
        query_self = torch.rand(batch, tokens, generator=g) < 0.2
        eye = torch.eye(tokens, dtype=torch.bool)
        dense_self = torch.where(query_self[:, None, :, None], eye[None, None], dense)
        qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
        want = oracle.attention_dropout(qr, kr, vr, None, keep, dropout_p, attn_mask=dense_self)
        want.backward(grad_out.double())
        with_self = build_structured_mask(structural.to(device), key_valid.to(device), query_self.to(device))
        qd, kd, vd = (t.to(device).requires_grad_(True) for t in (q, k, v))
        out = flash_attention(qd, kd, vd, structured_mask=with_self, dropout_p=dropout_p, training=True,
                              dropout_mask=keep.to(device))
        out.backward(grad_out.to(device))
        torch.testing.assert_close(out.detach().cpu().double(), want.detach(), **BF16_TOL)
        for got, ref, name in zip((qd.grad, kd.grad, vd.grad), (qr.grad, kr.grad, vr.grad), ("dq", "dk", "dv")):
            torch.testing.assert_close(got.cpu().double(), ref, msg=lambda m, n=name: f"{n} (self rows): {m}", **GRAD_TOL)


def test_reference_block_trains_with_its_default_dropout(device):
    """``UnifiedInteractionBlock`` in training mode with dropout (the reference's default hyperparameters) under the role
    mask: the layer-by-layer route runs on the HIP attention with a drawn keep mask; same seed, same result; every
    parameter receives a finite gradient."""
    from taac_2026_amd.api import UnifiedInteractionBlock

    batch, d_model, heads = 3, 128, 4
    roles = torch.tensor([0, 1] + [2] * 5 + [3] * 4 + [4] * 3 + [5] * 2 + [6] * 40 + [7] * 4)
    tokens = roles.numel()
    g = torch.Generator().manual_seed(2)
    block = UnifiedInteractionBlock(d_model, heads, 2, 0.04).to(torch.bfloat16).to(device).train()
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    padding = (torch.rand(batch, tokens, generator=g) < 0.3).to(device)
    padding[:, :2] = False
    mask = MetadataAttentionMask(enabled=True)(padding, roles.to(device))
    results = []
    for _ in range(2):
        torch.manual_seed(7)
        block.zero_grad(set_to_none=True)
        xd = x.clone().requires_grad_(True)
        out, _ = block(xd, padding, mask)
        out.float().square().mean().backward()
        results.append((out.detach().clone(), xd.grad.clone()))
        for name, parameter in block.named_parameters():
            assert parameter.grad is not None and torch.isfinite(parameter.grad).all(), name
    assert torch.equal(results[0][0], results[1][0]) and torch.equal(results[0][1], results[1][1])
    assert torch.isfinite(results[0][0]).all() and torch.isfinite(results[0][1]).all()
