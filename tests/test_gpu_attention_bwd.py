"""GPU parity: attention training forward (log-sum-exp) and backward (through the C ABI) against torch autograd of the
CPU oracle's closed form evaluated in float64."""

from __future__ import annotations

import pytest
import torch

from oracle import reference as oracle
from taac_2026_amd.api import flash_attention, scaled_dot_product_attention

pytestmark = pytest.mark.gpu

# Gradient tolerance of the reference's GPU tests for 16-bit attention (tests/gpu/infrastructure/accelerators/
# test_tilelang_ops_cuda.py:98-141): 3e-2.
TOL = dict(rtol=3e-2, atol=3e-2)


def _reference(q, k, v, lengths, grad_out, *, causal, zero_pad):
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    out = oracle.attention(qr, kr, vr, lengths, is_causal=causal, zero_padded_queries=zero_pad)
    out.backward(grad_out.double())
    return out.detach(), qr.grad, kr.grad, vr.grad


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tokens,dim", [(50, 32), (130, 64), (300, 32), (64, 16), (257, 64), (33, 8), (150, 48)])
@pytest.mark.parametrize("causal,zero_pad", [(False, False), (False, True), (True, False)])
def test_backward_matches_autograd_of_the_oracle(device, dtype, tokens, dim, causal, zero_pad):
    batch, heads = 4, 2
    g = torch.Generator().manual_seed(tokens * 7 + dim)
    q, k, v = (torch.randn(batch, heads, tokens, dim, generator=g).to(dtype) for _ in range(3))
    grad_out = torch.randn(batch, heads, tokens, dim, generator=g).to(dtype)
    lengths = torch.tensor([tokens, 1, max(1, tokens // 2), max(1, tokens - 3)], dtype=torch.int32)
    ref_out, ref_dq, ref_dk, ref_dv = _reference(q, k, v, lengths, grad_out, causal=causal, zero_pad=zero_pad)
    qd, kd, vd = (t.to(device).requires_grad_(True) for t in (q, k, v))
    out = flash_attention(qd, kd, vd, key_lengths=lengths.to(device), is_causal=causal, zero_padded_queries=zero_pad)
    out.backward(grad_out.to(device))
    torch.testing.assert_close(out.detach().cpu().double(), ref_out, rtol=2e-2, atol=2e-2)
    for got, ref, name in ((qd.grad, ref_dq, "dq"), (kd.grad, ref_dk, "dk"), (vd.grad, ref_dv, "dv")):
        assert got.dtype == dtype and got.shape == ref.shape
        torch.testing.assert_close(got.cpu().double(), ref, msg=lambda m, n=name: f"{n}: {m}", **TOL)
    # keys in the padding receive exactly zero gradient
    for b in range(batch):
        if lengths[b] < tokens:
            assert kd.grad[b, :, int(lengths[b]):].abs().max().item() == 0.0
            assert vd.grad[b, :, int(lengths[b]):].abs().max().item() == 0.0
            if zero_pad:
                assert qd.grad[b, :, int(lengths[b]):].abs().max().item() == 0.0


def test_backward_is_reproducible_and_reads_the_projection_layout(device):
    """(B, T, D) projections that are chunk views of one packed tensor, as the model packages produce them; two runs
    give bit-identical gradients (one writer per element, fixed summation order)."""
    batch, tokens, heads, dim = 3, 200, 4, 32
    g = torch.Generator().manual_seed(0)
    packed = torch.randn(batch, tokens, 3 * heads * dim, generator=g).to(torch.bfloat16)
    lengths = torch.tensor([200, 77, 130], dtype=torch.int32)
    grad_out = torch.randn(batch, tokens, heads * dim, generator=g).to(torch.bfloat16)
    grads = []
    for _ in range(2):
        pd = packed.to(device).requires_grad_(True)
        q, k, v = pd.chunk(3, dim=-1)
        out = scaled_dot_product_attention(q, k, v, num_heads=heads, attn_mask=None, dropout_p=0.0, training=True,
                                           key_lengths=lengths.to(device), zero_padded_queries=True)
        out.backward(grad_out.to(device))
        grads.append(pd.grad.clone())
    assert torch.equal(grads[0], grads[1])
    pr = packed.double().requires_grad_(True)
    q, k, v = pr.chunk(3, dim=-1)
    ref = oracle.scaled_dot_product_attention(q, k, v, num_heads=heads, key_lengths=lengths, zero_padded_queries=True)
    ref.backward(grad_out.double())
    torch.testing.assert_close(grads[0].cpu().double(), pr.grad, **TOL)


@pytest.mark.parametrize("dim,causal", [(32, False), (64, False), (64, True)])
def test_direct_transfer_backward_equals_register_staged_backward(device, dim, causal):
    """Full head dims stream their chunks from global memory straight into LDS, where rows beyond the valid length repeat
    the last valid row instead of zeros; their products are cancelled by zero probabilities, so both backward routes give
    the same bits from the same saved forward (taac_flash_attn_bwd through the C ABI with and without
    TAAC_ATTN_REGISTER_STAGING; the two forwards differ by roundings, see test_gpu_attention.py, so one forward feeds
    both)."""
    from taac_2026_amd import _native

    batch, heads, tokens = 5, 2, 333
    g = torch.Generator().manual_seed(dim + causal)
    q, k, v, grad_out = (torch.randn(batch, heads, tokens, dim, generator=g).to(torch.bfloat16).to(device) for _ in range(4))
    lengths = torch.tensor([333, 1, 64, 65, 200], dtype=torch.int32, device=device)
    library = _native.load_library()
    stream = _native.current_stream(q.device)
    out = torch.empty_like(q)
    lse = torch.empty(batch, heads, tokens, dtype=torch.float32, device=device)
    strides = lambda *ts: [_native.Int64x4(*t.stride()) for t in ts]  # noqa: E731
    flags = _native.ATTN_CAUSAL if causal else 0
    zero_pad = int(not causal)
    _native.check(library.taac_flash_attn_train_fwd(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), lengths.data_ptr(), out.data_ptr(), lse.data_ptr(), batch, heads, tokens,
        tokens, dim, *strides(q, k, v, out), flags, zero_pad, _native.dtype_code(q.dtype), stream), "train_fwd")
    grads = {}
    for name, route in (("direct", 0), ("registers", _native.ATTN_REGISTER_STAGING)):
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        delta = torch.empty_like(lse)
        _native.check(library.taac_flash_attn_bwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), grad_out.data_ptr(), lse.data_ptr(),
            lengths.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), delta.data_ptr(), batch, heads, tokens, tokens,
            dim, *strides(q, k, v, out, grad_out, dq, dk, dv), flags | route, zero_pad, _native.dtype_code(q.dtype), stream),
            "bwd")
        grads[name] = (dq, dk, dv)
    for direct, staged in zip(grads["direct"], grads["registers"]):
        assert torch.isfinite(direct.float()).all()
        assert torch.equal(direct, staged)
    # and the module-level route switch reaches both kernels: gradients of the two routes agree to rounding
    for staging in ("direct", "registers"):
        qd, kd, vd = (t.clone().requires_grad_(True) for t in (q, k, v))
        flash_attention(qd, kd, vd, key_lengths=lengths, is_causal=causal, zero_padded_queries=not causal,
                        kv_staging=staging).backward(grad_out)
        for got, want in zip((qd.grad, kd.grad, vd.grad), grads["direct"]):
            # (a step or two of bf16 at the largest gradients: the two forwards round differently)
            torch.testing.assert_close(got.float(), want.float(), rtol=2 ** -5, atol=2 ** -6 * want.float().abs().max().item())


def test_backward_envelope(device):
    q = torch.randn(1, 1, 16, 128, device=device, dtype=torch.bfloat16, requires_grad=True)
    with pytest.raises(RuntimeError, match="head_dim"):
        flash_attention(q, q, q).sum().backward()
    q32 = torch.randn(1, 1, 16, 32, device=device, requires_grad=True)
    with pytest.raises(RuntimeError, match="backward covers"):
        flash_attention(q32, q32, q32)


@pytest.mark.parametrize("dtype,dim,causal,tokens", [(torch.float16, 16, False, 32), (torch.bfloat16, 32, False, 150),
                                                     (torch.bfloat16, 64, True, 200), (torch.float16, 64, False, 77)])
def test_training_dropout_with_a_fixed_keep_mask(device, dtype, dim, causal, tokens):
    """Dropout on the attention probabilities with the caller's uint8 keep mask, forward and backward, against float64
    autograd of the oracle under the same mask - the check the reference runs on its TileLang kernels
    (tests/gpu/infrastructure/accelerators/test_tilelang_ops_cuda.py:103-141: output 2e-2, gradients 3e-2), here also with
    ragged key lengths, a causal triangle and a key count that is no multiple of four (unaligned mask rows)."""
    batch, heads, dropout_p = 3, 4, 0.125
    g = torch.Generator().manual_seed(tokens + dim)
    q, k, v, grad_out = (torch.randn(batch, heads, tokens, dim, generator=g).to(dtype) for _ in range(4))
    lengths = torch.tensor([tokens, max(1, tokens // 3), tokens - 5], dtype=torch.int32)
    mask = (torch.rand(batch, heads, tokens, tokens, generator=g) >= dropout_p).to(torch.uint8)
    qd, kd, vd = (t.to(device).requires_grad_(True) for t in (q, k, v))
    out = flash_attention(qd, kd, vd, key_lengths=lengths.to(device), is_causal=causal, zero_padded_queries=not causal,
                          dropout_p=dropout_p, training=True, dropout_mask=mask.to(device))
    out.backward(grad_out.to(device))
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    want = oracle.attention_dropout(qr, kr, vr, lengths, mask, dropout_p, is_causal=causal, zero_padded_queries=not causal)
    want.backward(grad_out.double())
    torch.testing.assert_close(out.detach().cpu().double(), want.detach(), rtol=2e-2, atol=2e-2)
    for got, ref in ((qd.grad, qr.grad), (kd.grad, kr.grad), (vd.grad, vr.grad)):
        torch.testing.assert_close(got.cpu().double(), ref, rtol=3e-2, atol=3e-2)
    # the mask matters (a run without it differs) and an all-ones mask at p -> 0 is the plain training path
    plain = flash_attention(qd.detach(), kd.detach(), vd.detach(), key_lengths=lengths.to(device), is_causal=causal,
                            zero_padded_queries=not causal)
    assert (plain.float() - out.detach().float()).abs().max().item() > 5e-2
    ones = torch.ones_like(mask).to(device)
    q1 = qd.detach().clone().requires_grad_(True)
    same = flash_attention(q1, kd.detach(), vd.detach(), key_lengths=lengths.to(device), is_causal=causal,
                           zero_padded_queries=not causal, dropout_p=1e-9, training=True, dropout_mask=ones)
    torch.testing.assert_close(same.detach().float(), plain.float(), rtol=2e-2, atol=2e-2)


def test_dropout_draws_its_own_mask_and_rejects_what_it_does_not_cover(device):
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(2, 2, 64, 32, generator=g).to(torch.bfloat16).to(device) for _ in range(3))
    torch.manual_seed(0)
    a = flash_attention(q, k, v, dropout_p=0.5, training=True)
    torch.manual_seed(0)
    b = flash_attention(q, k, v, dropout_p=0.5, training=True)
    c = flash_attention(q, k, v, dropout_p=0.5, training=True)
    assert torch.equal(a, b) and not torch.equal(a, c)
    with pytest.raises(RuntimeError, match="only supports dropout during training"):
        flash_attention(q, k, v, dropout_p=0.5, training=False)
    with pytest.raises(ValueError, match="dropout_mask must be uint8"):
        flash_attention(q, k, v, dropout_p=0.5, training=True, dropout_mask=torch.ones(2, 2, 64, 63, dtype=torch.uint8, device=device))
