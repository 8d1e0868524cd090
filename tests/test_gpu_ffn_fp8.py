"""GPU parity: the fused FP8 feed-forward layer (taac_swiglu_ffn_fp8_fwd) against the chain of two quantize -> matmul ->
dequantize layers of the CPU oracle. Tolerance of the FP8 configuration: 5e-2 relative to the largest expected value."""

from __future__ import annotations

import pytest
import torch

from oracle import reference as oracle
from taac_2026_amd.api import (amax, linear_fp8, norm_linear_fp8, pack_ffn_weights_fp8, quantize_fp8, rms_norm,
                               swiglu_ffn_fp8, valid_rows)

pytestmark = pytest.mark.gpu


def _case(m, d, f, seed, bias=True):
    g = torch.Generator().manual_seed(seed)
    bf = lambda t: t.to(torch.bfloat16)  # noqa: E731
    x = bf(torch.randn(m, d, generator=g) * (0.5 + torch.rand(m, 1, generator=g)))
    norm_w = bf(1 + 0.1 * torch.randn(d, generator=g))
    up_w = bf(torch.randn(2 * f, d, generator=g) * d ** -0.5)
    down_w = bf(torch.randn(d, f, generator=g) * f ** -0.5)
    up_b = bf(0.1 * torch.randn(2 * f, generator=g)) if bias else None
    down_b = bf(0.1 * torch.randn(d, generator=g)) if bias else None
    return x, norm_w, up_w, up_b, down_w, down_b


def _rel(got, expected):
    return ((got.float() - expected.float()).abs().max() / expected.float().abs().max()).item()


def _to(device, *tensors):
    return [None if t is None else t.to(device) for t in tensors]


@pytest.mark.parametrize("m,d,f", [(1, 256, 64), (300, 256, 1024), (64, 128, 64), (1000, 256, 192), (257, 128, 256),
                                   (777, 256, 512)])
@pytest.mark.parametrize("gate_first", [True, False])
@pytest.mark.parametrize("with_norm", [True, False])
def test_fused_fp8_ffn_matches_the_chain_of_emulated_layers(device, m, d, f, gate_first, with_norm):
    x, norm_w, up_w, up_b, down_w, down_b = _case(m, d, f, seed=m + f)
    want, hidden, h = oracle.swiglu_ffn_fp8(x, norm_w if with_norm else None, up_w, up_b, down_w, down_b, residual=x,
                                            gate_first=gate_first)
    xd, nw, uw, ub, dw, db = _to(device, x, norm_w, up_w, up_b, down_w, down_b)
    with torch.no_grad():
        packed = pack_ffn_weights_fp8(uw, dw, gate_first=gate_first)
        h_dev = rms_norm(xd, nw) if with_norm else xd
        got, amax_hidden, amax_next = swiglu_ffn_fp8(xd, packed, ub, db, amax(h_dev), hidden_size=f, residual=xd,
                                                     gate_first=gate_first, norm_weight=nw if with_norm else None,
                                                     want_amax_next=True)
    assert _rel(got.cpu(), want) <= 5e-2
    torch.testing.assert_close(got.cpu().float(), want.float(), rtol=0, atol=5e-2 * want.float().abs().max().item())
    # the scale the layer found for the hidden state is the maximum of the emulated hidden state (up to its rounding)
    assert abs(amax_hidden.item() - hidden.float().abs().max().item()) <= 2e-2 * hidden.float().abs().max().item()
    # and the scale handed to the next layer is the maximum of what the layer wrote
    assert amax_next.item() == got.float().abs().max().item()
    assert packed[1].item() == up_w.float().abs().max().item() and packed[2].item() == down_w.float().abs().max().item()


def test_fused_fp8_ffn_is_tight_against_the_emulation_with_its_own_scales(device):
    """With the oracle given the scales the kernel used, only accumulation order and the double rounding of the hidden
    state separate the two: far inside the 5e-2 of the configuration."""
    m, d, f = 512, 256, 1024
    x, norm_w, up_w, up_b, down_w, down_b = _case(m, d, f, seed=5)
    xd, nw, uw, ub, dw, db = _to(device, x, norm_w, up_w, up_b, down_w, down_b)
    with torch.no_grad():
        packed = pack_ffn_weights_fp8(uw, dw)
        h_dev = rms_norm(xd, nw)
        ax = amax(h_dev)
        got, amax_hidden, _ = swiglu_ffn_fp8(xd, packed, ub, db, ax, hidden_size=f, residual=xd, norm_weight=nw)
    h = h_dev.cpu()
    hidden = oracle.linear_fp8(h, up_w, up_b, swiglu=True, x_scale=ax.cpu() / 448.0)
    want = oracle.linear_fp8(hidden, down_w, down_b, residual=x, x_scale=amax_hidden.cpu() / 448.0)
    assert abs(amax_hidden.item() - hidden.float().abs().max().item()) <= 2 ** -7 * hidden.float().abs().max().item()
    assert _rel(got.cpu(), want) <= 1e-2


def test_fused_fp8_ffn_walks_valid_rows_only_and_hands_over_the_next_scale(device):
    batch, tokens, d, f = 6, 100, 256, 256
    x, norm_w, up_w, up_b, down_w, down_b = _case(batch * tokens, d, f, seed=9)
    lengths = torch.tensor([100, 1, 37, 64, 0, 99], dtype=torch.int32)
    valid = (torch.arange(tokens)[None, :] < lengths[:, None]).flatten()
    next_w = (1 + 0.2 * torch.randn(d, generator=torch.Generator().manual_seed(1))).to(torch.bfloat16)
    want, _, _ = oracle.swiglu_ffn_fp8(x[valid], norm_w, up_w, up_b, down_w, down_b, residual=x[valid])
    poisoned = x.clone()
    poisoned[~valid] = float("nan")
    xd, nw, uw, ub, dw, db, nxt = _to(device, poisoned, norm_w, up_w, up_b, down_w, down_b, next_w)
    with torch.no_grad():
        index = valid_rows(lengths.to(device), tokens)
        packed = pack_ffn_weights_fp8(uw, dw)
        ax = amax(rms_norm(x[valid].to(device), nw))
        out = xd.clone()
        got, _, amax_next = swiglu_ffn_fp8(xd, packed, ub, db, ax, hidden_size=f, residual=xd, norm_weight=nw,
                                           token_rows=index, out=out, next_norm_weight=nxt)
        again, _, amax_again = swiglu_ffn_fp8(xd, packed, ub, db, ax, hidden_size=f, residual=xd, norm_weight=nw,
                                              token_rows=index, out=xd.clone(), next_norm_weight=nxt)
    got = got.cpu()
    assert torch.isnan(got[~valid].float()).all()                      # padded rows are never touched
    assert _rel(got[valid], want) <= 5e-2
    assert torch.equal(again.cpu()[valid], got[valid]) and amax_again.item() == amax_next.item()
    expected_next = rms_norm(got[valid].to(device), nxt).float().abs().max().item()
    assert amax_next.item() == expected_next


def test_fused_fp8_ffn_errors(device):
    x, norm_w, up_w, up_b, down_w, down_b = _case(8, 256, 64, seed=1)
    xd, uw, dw = _to(device, x, up_w, down_w)
    packed = pack_ffn_weights_fp8(uw, dw)
    with pytest.raises(ValueError, match="do not match"):
        swiglu_ffn_fp8(xd, packed, None, None, amax(xd), hidden_size=128)
    with pytest.raises(RuntimeError, match="unsupported shape"):
        pack_ffn_weights_fp8(torch.zeros(2 * 48, 256, dtype=torch.bfloat16, device=device),
                             torch.zeros(256, 48, dtype=torch.bfloat16, device=device))
    with pytest.raises(RuntimeError, match="same device|CUDA"):
        swiglu_ffn_fp8(x, packed, None, None, amax(xd), hidden_size=64)


@pytest.mark.parametrize("workgroups", [None, 2])
@pytest.mark.parametrize("n,with_norm,with_residual", [(768, True, False), (256, False, True), (256, True, True), (64, False, False)])
def test_norm_linear_fp8_fuses_norm_rows_and_the_next_scale(device, test_hooks, n, with_norm, with_residual, workgroups):
    """RMSNorm -> quantise -> e4m3 product -> (+ residual) in one kernel, over a row index, with the scale of the consuming
    layer reduced in the epilogue; against the emulated layer on the normalised rows, and against the two-kernel route
    (stand-alone norm, taac_linear_fp8), which computes the same thing."""
    if workgroups is not None:
        test_hooks(max_workgroups=workgroups)
    batch, tokens, k = 9, 150, 256
    g = torch.Generator().manual_seed(n + with_norm)
    bf = lambda t: t.to(torch.bfloat16)  # noqa: E731
    x = bf(torch.randn(batch * tokens, k, generator=g) * (0.5 + torch.rand(batch * tokens, 1, generator=g)))
    w = bf(torch.randn(n, k, generator=g) * k ** -0.5)
    b = bf(0.1 * torch.randn(n, generator=g))
    norm_w = bf(1 + 0.1 * torch.randn(k, generator=g))
    next_w = bf(1 + 0.2 * torch.randn(n, generator=g))
    res = bf(torch.randn(batch * tokens, n, generator=g)) if with_residual else None
    lengths = torch.tensor([150, 0, 1, 77, 149, 150, 3, 64, 100], dtype=torch.int32)
    valid = (torch.arange(tokens)[None, :] < lengths[:, None]).flatten()
    h = oracle.rms_norm_fp32(x[valid], norm_w) if with_norm else x[valid]
    want = oracle.linear_fp8(h, w, b, residual=None if res is None else res[valid])
    poisoned = x.clone()
    poisoned[~valid] = float("nan")
    xd, wd, bd, nw, nxt = _to(device, poisoned, w, b, norm_w, next_w)
    resd = None if res is None else res.to(device)
    with torch.no_grad():
        index = valid_rows(lengths.to(device), tokens)
        wq, wa = quantize_fp8(wd)
        h_dev = rms_norm(x[valid].to(device), nw) if with_norm else x[valid].to(device)
        ax = amax(h_dev)
        out = torch.full((batch * tokens, n), float("nan"), dtype=torch.bfloat16, device=device)
        got, amax_out = norm_linear_fp8(xd, wq, ax, wa, bd, norm_weight=nw if with_norm else None, residual=resd,
                                        token_rows=index, out=out, out_norm_weight=nxt)
        plain, amax_plain = norm_linear_fp8(xd, wq, ax, wa, bd, norm_weight=nw if with_norm else None, residual=resd,
                                            token_rows=index, out=out.clone(), want_amax_out=True)
        two_kernels = linear_fp8(h_dev, wq, ax, wa, bd, residual=None if resd is None else resd[valid.to(device)])
    got = got.cpu()
    assert torch.isnan(got[~valid].float()).all()
    assert _rel(got[valid], want) <= 5e-2
    assert torch.equal(got[valid], two_kernels.cpu())
    assert torch.equal(plain.cpu()[valid], got[valid])
    assert amax_plain.item() == got[valid].float().abs().max().item()
    expected_next = rms_norm(got[valid].to(device), nxt).float().abs().max().item()
    assert abs(amax_out.item() - expected_next) <= 2 ** -7 * expected_next
