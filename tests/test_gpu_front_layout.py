"""GPU parity of the pieces that move every sample's valid tokens to the front of its rows: the second row index, the
structural mask gathered per sample, dense layers that read one layout and write the other, and attention under the
gathered mask against attention under the original one."""

from __future__ import annotations

import pytest
import torch

from oracle import reference as oracle
from taac_2026_amd.api import (
    build_structured_mask,
    flash_attention,
    front_rows,
    front_structured_mask,
    norm_linear,
    qkv_projection,
    valid_rows,
)

pytestmark = pytest.mark.gpu


def _padding(batch, tokens, seed):
    g = torch.Generator().manual_seed(seed)
    padding = torch.rand(batch, tokens, generator=g) < 0.4
    padding[0] = False            # nothing padded
    if batch > 1:
        padding[1] = True         # everything padded
    if batch > 2:
        padding[2, 1:] = True     # at most one valid token
    return padding


@pytest.mark.parametrize("batch,tokens", [(6, 100), (3, 32), (4, 513), (1, 1)])
def test_front_rows(device, batch, tokens):
    padding = _padding(batch, tokens, seed=tokens)
    index = valid_rows(None, tokens, padding_mask=padding.to(device))
    front, lengths = front_rows(index, batch, tokens)
    valid = ~padding
    assert torch.equal(lengths.cpu().long(), valid.sum(1))
    rank = valid.long().cumsum(1) - 1
    expected = (torch.arange(batch)[:, None] * tokens + rank)[valid]
    assert torch.equal(front[:expected.numel()].cpu().long(), expected)


@pytest.mark.parametrize("batch,tokens", [(5, 70), (3, 200), (2, 33)])
def test_front_structured_mask_bits(device, batch, tokens):
    g = torch.Generator().manual_seed(tokens)
    padding = _padding(batch, tokens, seed=tokens + 1)
    structural = torch.rand(tokens, tokens, generator=g) < 0.6
    mask = build_structured_mask(structural.to(device), (~padding).to(device))
    index = valid_rows(None, tokens, padding_mask=padding.to(device))
    front = front_structured_mask(mask, index, batch)
    words = (tokens + 31) // 32
    assert front.sample_stride == tokens * words and front.struct_bits.shape == (batch * tokens, words)
    bits = front.struct_bits.cpu().view(batch, tokens, words)
    shifts = torch.arange(32)
    got = ((bits[..., None] >> shifts) & 1).bool().view(batch, tokens, words * 32)[..., :tokens]
    for b in range(batch):
        positions = (~padding[b]).nonzero().flatten()
        n = positions.numel()
        # written: rows below n, and of those the words up to the end of the 64-key group of key n - 1
        written = min(tokens, 64 * ((n + 63) // 64))
        want = torch.zeros(n, written, dtype=torch.bool)
        want[:, :n] = structural[positions][:, positions]
        assert torch.equal(got[b, :n, :written], want), b
    with pytest.raises(RuntimeError, match="front layout"):
        front.dense()
    with pytest.raises(ValueError, match="front layout already"):
        front_structured_mask(front, index, batch)


def test_dense_layers_between_the_two_layouts(device):
    """norm_linear reading the caller's layout and writing the front layout, and back: the same values as the layer over
    positions, moved."""
    batch, tokens, d_model = 4, 90, 256
    g = torch.Generator().manual_seed(3)
    padding = _padding(batch, tokens, seed=5)
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    weight = (0.05 * torch.randn(3 * d_model, d_model, generator=g)).to(torch.bfloat16).to(device)
    norm_weight = (1 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16).to(device)
    index = valid_rows(None, tokens, padding_mask=padding.to(device))
    front, lengths = front_rows(index, batch, tokens)
    by_position = norm_linear(x, weight, None, norm_weight=norm_weight, token_rows=index)
    moved = torch.zeros(batch * tokens, 3 * d_model, dtype=torch.bfloat16, device=device)
    norm_linear(x, weight, None, norm_weight=norm_weight, token_rows=(front, index[1]), input_rows=index[0], out=moved)
    count = int(index[1].item())
    rows, front_cpu = index[0][:count].long(), front[:count].long()
    assert torch.equal(moved[front_cpu], by_position.view(-1, 3 * d_model)[rows])
    untouched = torch.ones(batch * tokens, dtype=torch.bool, device=device)
    untouched[front_cpu] = False
    assert moved[untouched].abs().max().item() == 0.0
    # and back: a square layer reading the front layout, adding to and writing the caller's layout
    square = (0.05 * torch.randn(d_model, d_model, generator=g)).to(torch.bfloat16).to(device)
    attn_front = moved[:, :d_model].contiguous()
    attn_position = by_position.view(-1, 3 * d_model)[:, :d_model].contiguous()
    want = norm_linear(attn_position, square, None, residual=x.view(-1, d_model), token_rows=index, out=x.view(-1, d_model).clone())
    got = norm_linear(attn_front, square, None, residual=x.view(-1, d_model), token_rows=index, input_rows=front,
                      out=x.view(-1, d_model).clone())
    assert torch.equal(got, want)
    with pytest.raises(ValueError, match="input_rows needs token_rows"):
        norm_linear(attn_front, square, None, input_rows=front)


def test_qkv_projection_into_the_front_layout_keeps_positions_and_factors(device):
    """Rotary positions follow the rows of the input, the norm factors the rows of the output."""
    batch, tokens, d_model, heads = 3, 64, 128, 4
    g = torch.Generator().manual_seed(11)
    padding = _padding(batch, tokens, seed=12)
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    weight = (0.1 * torch.randn(3 * d_model, d_model, generator=g)).to(torch.bfloat16).to(device)
    qw, kw = ((1 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16).to(device) for _ in range(2))
    index = valid_rows(None, tokens, padding_mask=padding.to(device))
    front, _ = front_rows(index, batch, tokens)
    common = dict(num_heads=heads, query_weight=qw, key_weight=kw, rope_base=10000.0)
    by_position, q_scale, k_scale, _ = qkv_projection(x, weight, None, token_rows=index, **common)
    moved, q_front, k_front, _ = qkv_projection(x, weight, None, token_rows=(front, index[1]), input_rows=index[0], **common)
    count = int(index[1].item())
    rows, front_cpu = index[0][:count].long(), front[:count].long()
    assert torch.equal(moved.view(-1, 3 * d_model)[front_cpu], by_position.view(-1, 3 * d_model)[rows])
    assert torch.equal(q_front.flatten()[front_cpu], q_scale.flatten()[rows])
    assert torch.equal(k_front.flatten()[front_cpu], k_scale.flatten()[rows])


@pytest.mark.parametrize("tokens,dim", [(150, 32), (96, 64)])
def test_attention_over_the_front_layout_matches_the_masked_attention_over_positions(device, tokens, dim):
    batch, heads = 5, 2
    g = torch.Generator().manual_seed(tokens + dim)
    padding = _padding(batch, tokens, seed=tokens)
    padding[1, 0] = False                                  # keep one valid token: a sample without any has no output rows
    structural = (torch.rand(tokens, tokens, generator=g) < 0.5) | torch.eye(tokens, dtype=torch.bool)
    q, k, v = (torch.randn(batch, heads, tokens, dim, generator=g).to(torch.bfloat16) for _ in range(3))
    dense = structural[None, None] & (~padding)[:, None, None, :]
    want = oracle.sdpa(q.float(), k.float(), v.float(), dense)
    mask = build_structured_mask(structural.to(device), (~padding).to(device))
    index = valid_rows(None, tokens, padding_mask=padding.to(device))
    front, lengths = front_rows(index, batch, tokens)
    front_mask = front_structured_mask(mask, index, batch)
    count = int(index[1].item())
    rows, front_cpu = index[0][:count].long().cpu(), front[:count].long().cpu()

    def moved(t):  # (B, H, T, d) -> the same with every sample's valid tokens at the front
        flat = t.transpose(1, 2).reshape(batch * tokens, heads, dim)
        out = torch.full_like(flat, float("nan"))         # rows beyond a sample's length are never read
        out[front_cpu] = flat[rows]
        return out.view(batch, tokens, heads, dim).transpose(1, 2).to(device)

    got_front = flash_attention(moved(q), moved(k), moved(v), key_lengths=lengths, structured_mask=front_mask,
                                zero_padded_queries=2)
    got = got_front.transpose(1, 2).reshape(batch * tokens, heads, dim).cpu().float()[front_cpu]
    expected = want.transpose(1, 2).reshape(batch * tokens, heads, dim)[rows]
    torch.testing.assert_close(got, expected, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("tokens,dim", [(150, 32), (96, 64)])
def test_attention_over_the_front_layout_takes_a_gradient(device, tokens, dim):
    """The same comparison for the backward: gradients of attention over the front layout (structure bits per sample,
    key lengths = the samples' numbers of valid tokens, rows beyond them never read: they hold NaN here) against
    float64 autograd under the dense mask over the positions."""
    batch, heads = 5, 2
    g = torch.Generator().manual_seed(tokens + dim + 1)
    padding = _padding(batch, tokens, seed=tokens)
    padding[1, 0] = False
    structural = (torch.rand(tokens, tokens, generator=g) < 0.5) | torch.eye(tokens, dtype=torch.bool)
    q, k, v, grad_out = (torch.randn(batch, heads, tokens, dim, generator=g).to(torch.bfloat16) for _ in range(4))
    dense = structural[None, None] & (~padding)[:, None, None, :]
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    keep = (~padding)[:, None, :, None].double()           # padded query rows carry no loss
    (oracle.sdpa(qr, kr, vr, dense) * keep).backward(grad_out.double())
    mask = build_structured_mask(structural.to(device), (~padding).to(device))
    index = valid_rows(None, tokens, padding_mask=padding.to(device))
    front, lengths = front_rows(index, batch, tokens)
    front_mask = front_structured_mask(mask, index, batch)
    count = int(index[1].item())
    rows, front_cpu = index[0][:count].long().cpu(), front[:count].long().cpu()

    def moved(t, fill):
        flat = t.transpose(1, 2).reshape(batch * tokens, heads, dim)
        out = torch.full_like(flat, fill)
        out[front_cpu] = flat[rows]
        return out.view(batch, tokens, heads, dim).transpose(1, 2).to(device)

    qd, kd, vd = (moved(t, float("nan")).requires_grad_(True) for t in (q, k, v))
    out = flash_attention(qd, kd, vd, key_lengths=lengths, structured_mask=front_mask, zero_padded_queries=True)
    out.backward(moved(grad_out, float("nan")))
    for got, want, name in zip((qd.grad, kd.grad, vd.grad), (qr.grad, kr.grad, vr.grad), ("dq", "dk", "dv")):
        got = got.transpose(1, 2).reshape(batch * tokens, heads, dim).cpu().double()[front_cpu]
        want = want.transpose(1, 2).reshape(batch * tokens, heads, dim)[rows]
        assert torch.isfinite(got).all(), name
        torch.testing.assert_close(got, want, rtol=3e-2, atol=3e-2, msg=lambda m, n=name: f"{n}: {m}")
