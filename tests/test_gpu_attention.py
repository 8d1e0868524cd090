"""GPU parity: key-padding-masked attention HIP kernel (through the C ABI) against the CPU oracle."""

from __future__ import annotations

import pytest
import torch
import torch.nn.functional as F

from oracle import reference as oracle
from taac_2026_amd import workloads
from taac_2026_amd.api import causal_valid_attention_mask, flash_attention, scaled_dot_product_attention

pytestmark = pytest.mark.gpu

BF16_TOL = dict(rtol=2e-2, atol=2e-2)


def _qkv(batch, heads, tq, tk, dim, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(batch, heads, tq, dim, generator=g).to(dtype)
    k = torch.randn(batch, heads, tk, dim, generator=g).to(dtype)
    v = torch.randn(batch, heads, tk, dim, generator=g).to(dtype)
    return q, k, v


def _run(q, k, v, device, **kwargs):
    with torch.no_grad():
        return flash_attention(q.to(device), k.to(device), v.to(device), **kwargs).cpu()


def test_unmasked_fp16_small_matches_sdpa(device):
    # shape and tolerance of the reference's GPU test (test_tilelang_ops_cuda.py:61-73)
    q, k, v = _qkv(2, 4, 32, 32, 16, torch.float16, 0)
    got = _run(q, k, v, device)
    expected = F.scaled_dot_product_attention(q.float(), k.float(), v.float())
    torch.testing.assert_close(got.float(), expected, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dim", [8, 16, 32, 64, 96, 128])
@pytest.mark.parametrize("tokens", [1, 31, 32, 33, 64, 100, 128, 129, 300])
def test_key_lengths_bf16(device, dim, tokens):
    batch, heads = 5, 3
    q, k, v = _qkv(batch, heads, tokens, tokens, dim, torch.bfloat16, dim * 1000 + tokens)
    lengths = torch.tensor([tokens, 1, max(1, tokens // 2), 0, max(1, tokens - 1)], dtype=torch.int32)
    expected = oracle.attention(q, k, v, lengths)
    got = _run(q, k, v, device, key_lengths=lengths.to(device))
    torch.testing.assert_close(got.float(), expected.float(), **BF16_TOL)
    expected_zero = oracle.attention(q, k, v, lengths, zero_padded_queries=True)
    got_zero = _run(q, k, v, device, key_lengths=lengths.to(device), zero_padded_queries=True)
    torch.testing.assert_close(got_zero.float(), expected_zero.float(), **BF16_TOL)
    # padded query rows are exactly zero
    for b in range(batch):
        assert got_zero[b, :, int(lengths[b]):].abs().max().item() == 0.0 if lengths[b] < tokens else True


@pytest.mark.parametrize("dim", [32, 64])
@pytest.mark.parametrize("tokens", [129, 300, 512, 640])
def test_workgroups_that_take_two_query_blocks(device, dim, tokens):
    """Under key lengths (or a causal triangle) a workgroup of the direct-transfer kernel takes query blocks g and
    nqc - 1 - g: 2, 3, 4 and 5 blocks of 128 queries here (odd counts leave the middle block alone), with samples whose
    second block is full, partly valid, empty, and whose first block is empty too."""
    batch, heads = 6, 2
    q, k, v = _qkv(batch, heads, tokens, tokens, dim, torch.bfloat16, 7 * tokens + dim)
    lengths = torch.tensor([tokens, 0, 1, 128, min(tokens, 200), tokens - 1], dtype=torch.int32)
    for zero_pad in (False, True):
        expected = oracle.attention(q, k, v, lengths, zero_padded_queries=zero_pad)
        got = _run(q, k, v, device, key_lengths=lengths.to(device), zero_padded_queries=zero_pad)
        torch.testing.assert_close(got.float(), expected.float(), **BF16_TOL)
    # rows left alone (the backbone's mode): the valid rows as above
    got = _run(q, k, v, device, key_lengths=lengths.to(device), zero_padded_queries=2)
    expected = oracle.attention(q, k, v, lengths, zero_padded_queries=True)
    for b in range(batch):
        n = int(lengths[b])
        torch.testing.assert_close(got[b, :, :n].float(), expected[b, :, :n].float(), **BF16_TOL)
    # the causal triangle pairs blocks as well (no key lengths: every sample full)
    causal = torch.ones(tokens, tokens, dtype=torch.bool).tril()
    want = oracle.sdpa(q.float(), k.float(), v.float(), attn_mask=causal[None, None])
    got = _run(q, k, v, device, is_causal=True)
    torch.testing.assert_close(got.float(), want, **BF16_TOL)


def test_cross_attention_lengths_differ(device):
    q, k, v = _qkv(2, 3, 5, 7, 8, torch.bfloat16, 11)
    got = _run(q, k, v, device)
    torch.testing.assert_close(got.float(), oracle.attention(q, k, v).float(), **BF16_TOL)
    q, k, v = _qkv(3, 2, 150, 77, 64, torch.bfloat16, 12)
    lengths = torch.tensor([77, 40, 3], dtype=torch.int32)
    got = _run(q, k, v, device, key_lengths=lengths.to(device))
    torch.testing.assert_close(got.float(), oracle.attention(q, k, v, lengths).float(), **BF16_TOL)


def test_bool_mask_forms(device):
    q, k, v = _qkv(2, 3, 4, 6, 8, torch.bfloat16, 5)
    key_valid = torch.tensor([[True, True, True, True, False, False], [True, True, False, False, False, False]])
    mask4 = key_valid[:, None, None, :].expand(2, 3, 4, 6)
    expected = oracle.sdpa(q.float(), k.float(), v.float(), attn_mask=mask4)
    for mask in (mask4, key_valid, key_valid[:, None, None, :]):
        got = _run(q, k, v, device, attn_mask=mask.to(device))
        torch.testing.assert_close(got.float(), expected, **BF16_TOL)


@pytest.mark.parametrize("tokens,dim", [(5, 8), (64, 32), (130, 64), (257, 32)])
def test_causal_valid_mask(device, tokens, dim):
    batch, heads = 3, 2
    q, k, v = _qkv(batch, heads, tokens, tokens, dim, torch.bfloat16, tokens)
    lengths = torch.tensor([tokens, max(1, tokens // 3), 1])
    padding = oracle.make_padding_mask(lengths, tokens)
    mask = oracle.causal_valid_attention_mask(padding, heads)
    expected = oracle.sdpa(q.float(), k.float(), v.float(), attn_mask=mask)
    got = _run(q, k, v, device, attn_mask=causal_valid_attention_mask(padding.to(device), heads))
    torch.testing.assert_close(got.float(), expected, **BF16_TOL)
    # plain causal without lengths
    got = _run(q, k, v, device, is_causal=True)
    torch.testing.assert_close(got.float(), oracle.attention(q, k, v, is_causal=True).float(), **BF16_TOL)


def test_float32_callers_are_computed_in_bf16(device):
    q, k, v = _qkv(2, 4, 32, 32, 16, torch.float32, 3)
    got = _run(q, k, v, device)
    assert got.dtype == torch.float32
    torch.testing.assert_close(got, F.scaled_dot_product_attention(q, k, v), rtol=1.5e-2, atol=1.5e-2)


def test_projection_layout_is_read_in_place(device):
    """(B, T, 3D) fused projection -> strided (B, H, T, dh) views, no copies, result (B, T, D)."""
    batch, tokens, heads, dh = 3, 70, 8, 32
    g = torch.Generator().manual_seed(9)
    qkv = torch.randn(batch, tokens, 3 * heads * dh, generator=g).to(torch.bfloat16)
    lengths = torch.tensor([70, 33, 1], dtype=torch.int32)
    q, k, v = qkv.chunk(3, dim=-1)
    expected = oracle.scaled_dot_product_attention(q, k, v, num_heads=heads, key_lengths=lengths, zero_padded_queries=True)
    dq, dk, dv = qkv.to(device).chunk(3, dim=-1)
    with torch.no_grad():
        got = scaled_dot_product_attention(dq, dk, dv, num_heads=heads, attn_mask=None, dropout_p=0.0, training=False,
                                           key_lengths=lengths.to(device), zero_padded_queries=True)
    assert got.shape == (batch, tokens, heads * dh)
    torch.testing.assert_close(got.cpu().float(), expected.float(), **BF16_TOL)


def test_special_cases(device):
    # identical keys -> uniform softmax -> mean of the valid values; len == 1 -> v[0]
    batch, heads, tokens, dim = 2, 2, 96, 64
    q, k, v = _qkv(batch, heads, tokens, tokens, dim, torch.bfloat16, 21)
    k = k[:, :, :1].expand(-1, -1, tokens, -1).contiguous()
    lengths = torch.tensor([50, 1], dtype=torch.int32)
    got = _run(q, k, v, device, key_lengths=lengths.to(device)).float()
    torch.testing.assert_close(got[0], v[0, :, :50].float().mean(dim=1, keepdim=True).expand(-1, tokens, -1), **BF16_TOL)
    torch.testing.assert_close(got[1], v[1, :, :1].float().expand(-1, tokens, -1), **BF16_TOL)


def test_config3_full_size(device):
    """Config 3 (B=2048, H=4, T=256, d=64, lengths ~ U{16..256}) at full size: a slice of samples against the oracle,
    padded rows exactly zero, everything finite."""
    q, k, v, lengths = workloads.attention_inputs()
    with torch.no_grad():
        got = flash_attention(q.to(device), k.to(device), v.to(device), key_lengths=lengths.to(device),
                              zero_padded_queries=True)
        assert torch.isfinite(got).all()
        positions = torch.arange(256, device=device)[None, :] >= lengths.to(device)[:, None]
        assert got.float().abs().amax(dim=(1, 3))[positions].max().item() == 0.0
    got = got.cpu()
    pick = torch.arange(0, 2048, 53)
    expected = oracle.attention(q[pick], k[pick], v[pick], lengths[pick], zero_padded_queries=True)
    torch.testing.assert_close(got[pick].float(), expected.float(), **BF16_TOL)


def test_errors(device):
    q, k, v = _qkv(2, 3, 5, 5, 8, torch.bfloat16, 1)
    with pytest.raises(ValueError, match="matching head dimensions"):
        flash_attention(q.to(device), k.to(device), v[..., :4].to(device))
    bad = torch.tensor([[True, False, True, False, False]]).expand(2, 5)[:, None, None, :].expand(2, 3, 5, 5)
    # the reference's planner refuses a key mask that is not a prefix (flash_attention.py:171-173), and so does its
    # restatement here; flash_attention itself then serves the mask through the structured-mask kernel, as the
    # reference serves it through its torch backend
    from taac_2026_amd.accelerators.attention import plan_flash_attention_mask

    with pytest.raises(RuntimeError, match="prefix-valid"):
        plan_flash_attention_mask(q.to(device), k.to(device), bad.to(device), is_causal=False)
    got = flash_attention(q.to(device), k.to(device), v.to(device), attn_mask=bad.to(device)).cpu()
    expected = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=bad)
    torch.testing.assert_close(got.float(), expected, **BF16_TOL)
    with pytest.raises(RuntimeError, match="requires CUDA tensors"):
        flash_attention(q, k, v)
    q7 = torch.randn(1, 1, 4, 12, dtype=torch.bfloat16, device=device)
    with pytest.raises(RuntimeError, match="head_dim"):
        flash_attention(q7, q7, q7)


@pytest.mark.parametrize("dim,tokens,causal", [(32, 150, False), (64, 70, False), (128, 33, False), (32, 130, True)])
def test_row_factors_of_queries_and_keys(device, dim, tokens, causal):
    """One positive factor per query row and per key row (shared by the heads) applied inside the kernel equals attention
    over the scaled tensors; factors at padded rows are never read (NaN there changes nothing); either may be absent."""
    from taac_2026_amd.accelerators.attention import hip_flash_attention_kernel

    batch, heads = 4, 3
    q, k, v = _qkv(batch, heads, tokens, tokens, dim, torch.bfloat16, dim + tokens)
    g = torch.Generator().manual_seed(9)
    sq = 0.25 + 2.0 * torch.rand(batch, tokens, generator=g)
    sk = 0.25 + 2.0 * torch.rand(batch, tokens, generator=g)
    lengths = torch.tensor([tokens, 7, tokens // 2, 0], dtype=torch.int32)
    expected = oracle.attention(q.float() * sq[:, None, :, None], k.float() * sk[:, None, :, None], v, lengths,
                                is_causal=causal, zero_padded_queries=True)
    valid = torch.arange(tokens)[None, :] < lengths[:, None]
    sq_nan = torch.where(valid, sq, torch.full_like(sq, float("nan")))
    sk_nan = torch.where(valid, sk, torch.full_like(sk, float("nan")))
    with torch.no_grad():
        args = (q.to(device), k.to(device), v.to(device), lengths.to(device))
        got = hip_flash_attention_kernel(*args, is_causal=causal, zero_padded_queries=True,
                                         q_row_scale=sq_nan.to(device), k_row_scale=sk_nan.to(device)).cpu()
        only_q = hip_flash_attention_kernel(*args, is_causal=causal, zero_padded_queries=True,
                                            q_row_scale=sq.to(device)).cpu()
        only_k = hip_flash_attention_kernel(*args, is_causal=causal, zero_padded_queries=True,
                                            k_row_scale=sk.to(device)).cpu()
    assert torch.isfinite(got.float()).all()
    torch.testing.assert_close(got.float(), expected.float(), **BF16_TOL)
    expected_q = oracle.attention(q.float() * sq[:, None, :, None], k, v, lengths, is_causal=causal, zero_padded_queries=True)
    expected_k = oracle.attention(q, k.float() * sk[:, None, :, None], v, lengths, is_causal=causal, zero_padded_queries=True)
    torch.testing.assert_close(only_q.float(), expected_q.float(), **BF16_TOL)
    torch.testing.assert_close(only_k.float(), expected_k.float(), **BF16_TOL)
    with pytest.raises(ValueError, match="q_row_scale"):
        hip_flash_attention_kernel(*args, q_row_scale=sq[:, :-1].contiguous().to(device))
    # one factor per query feature (the product of a query and a key norm weight)
    col = 0.5 + torch.rand(heads * dim, generator=g)
    expected_c = oracle.attention(q.float() * col.view(1, heads, 1, dim) * sq[:, None, :, None], k, v, lengths,
                                  is_causal=causal, zero_padded_queries=True)
    with torch.no_grad():
        with_col = hip_flash_attention_kernel(*args, is_causal=causal, zero_padded_queries=True,
                                              q_row_scale=sq.to(device), q_col_scale=col.to(device)).cpu()
        only_col = hip_flash_attention_kernel(*args, is_causal=causal, zero_padded_queries=True,
                                              q_col_scale=col.to(device)).cpu()
    torch.testing.assert_close(with_col.float(), expected_c.float(), **BF16_TOL)
    expected_oc = oracle.attention(q.float() * col.view(1, heads, 1, dim), k, v, lengths, is_causal=causal,
                                   zero_padded_queries=True)
    torch.testing.assert_close(only_col.float(), expected_oc.float(), **BF16_TOL)
    with pytest.raises(ValueError, match="q_col_scale"):
        hip_flash_attention_kernel(*args, q_col_scale=col[:-1].contiguous().to(device))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("head_dim", [32, 64])
@pytest.mark.parametrize("causal", [False, True])
def test_direct_transfer_kernel_agrees_with_general_kernel(device, dtype, head_dim, causal):
    """Head dims 32 and 64 run a kernel that stages K and V by direct global->LDS transfers (swizzled rows, transposed
    LDS reads) and a softmax whose reference moves lazily (query pre-multiplied by the softmax scale, row sums through the
    matrix unit); kv_staging="registers" selects the general kernel with the textbook running maximum. The two differ by
    one more rounding of the scaled query and by the order of the sums: a few steps of the storage type, for ragged
    lengths (0, 1, not a multiple of the chunk), strided views of a packed projection and row factors. Rows a kernel must
    not touch or must zero are identical."""
    from taac_2026_amd.api import flash_attention
    from taac_2026_amd.accelerators.attention import hip_flash_attention_kernel

    g = torch.Generator().manual_seed(head_dim + int(causal))
    batch, heads, tokens = 5, 3, 200
    qkv = torch.randn(batch, tokens, 3 * heads * head_dim, generator=g).to(dtype).to(device)
    q, k, v = (t.view(batch, tokens, heads, head_dim).transpose(1, 2) for t in qkv.chunk(3, dim=-1))
    lengths = torch.tensor([200, 0, 1, 65, 130], dtype=torch.int32, device=device)
    q_rows = (0.5 + torch.rand(batch, tokens, generator=g)).to(device)
    k_rows = (0.5 + torch.rand(batch, tokens, generator=g)).to(device)
    q_cols = (0.5 + torch.rand(heads * head_dim, generator=g)).to(device)

    def run(staging):
        with torch.no_grad():
            plain = flash_attention(q, k, v, key_lengths=lengths, is_causal=causal, zero_padded_queries=True,
                                    kv_staging=staging)
            full = flash_attention(q, k, v, is_causal=causal, kv_staging=staging)
            scaled = hip_flash_attention_kernel(q, k, v, lengths, is_causal=causal, zero_padded_queries=True,
                                                q_row_scale=q_rows, k_row_scale=k_rows, q_col_scale=q_cols,
                                                kv_staging=staging)
        return plain, full, scaled

    direct = run("direct")
    general = run("registers")
    step = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    for a, b in zip(direct, general):
        torch.testing.assert_close(a.float(), b.float(), rtol=4 * step, atol=4 * step)
        assert torch.equal(a == 0, b == 0) or (a.float() - b.float()).abs().max().item() <= 4 * step
    padded = torch.arange(tokens, device=device)[None, :] >= lengths[:, None]
    assert (direct[0].transpose(1, 2)[padded] == 0).all() and (direct[2].transpose(1, 2)[padded] == 0).all()


@pytest.mark.parametrize("head_dim,zero_pad", [(32, 2), (64, 1), (16, 0)])
def test_attention_reduces_the_scale_of_its_output(device, head_dim, zero_pad):
    """``amax_out`` receives max |o| over the rows the kernel writes (the FP8 scale of the layer behind it), from both
    kernels (direct-transfer and general), with the output itself unchanged."""
    from taac_2026_amd.accelerators.attention import hip_flash_attention_kernel

    g = torch.Generator().manual_seed(head_dim)
    batch, heads, tokens = 6, 3, 190
    q, k, v = (torch.randn(batch, heads, tokens, head_dim, generator=g).to(torch.bfloat16).to(device) for _ in range(3))
    lengths = torch.tensor([190, 1, 64, 65, 130, 17], dtype=torch.int32, device=device)
    for staging in ("direct", "registers"):
        amax = torch.full((), -1.0, dtype=torch.float32, device=device)
        with torch.no_grad():
            plain = hip_flash_attention_kernel(q, k, v, lengths, zero_padded_queries=zero_pad, kv_staging=staging)
            got = hip_flash_attention_kernel(q, k, v, lengths, zero_padded_queries=zero_pad, kv_staging=staging, amax_out=amax)
        valid = torch.arange(tokens, device=device)[None, :] < lengths[:, None]
        rows = valid[:, None, :, None].expand_as(got) if zero_pad else torch.ones_like(got, dtype=torch.bool)
        assert torch.equal(got[rows], plain[rows])
        assert amax.item() == got[rows].float().abs().max().item()
