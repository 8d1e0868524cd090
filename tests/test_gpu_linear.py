"""GPU parity: dense-layer HIP kernels (bf16 and FP8 MFMA, fused epilogues) against the CPU oracle."""

from __future__ import annotations

import pytest
import torch
import torch.nn.functional as F

from oracle import reference as oracle
from taac_2026_amd.api import (
    SwiGLUFeedForward,
    amax,
    linear,
    linear_fp8,
    quantize_fp8,
    swiglu_ffn,
    swiglu_linear,
)

pytestmark = pytest.mark.gpu

BF16_TOL = dict(rtol=2e-2, atol=2e-2)


def _draw(m, n, k, seed, *, x_scale=1.0):
    g = torch.Generator().manual_seed(seed)
    x = (x_scale * torch.randn(m, k, generator=g)).to(torch.bfloat16)
    bound = (6.0 / (n + k)) ** 0.5
    w = ((torch.rand(n, k, generator=g) * 2 - 1) * bound).to(torch.bfloat16)
    b = (0.1 * torch.randn(n, generator=g)).to(torch.bfloat16)
    return x, w, b


@pytest.mark.parametrize("m,n,k", [(1, 8, 8), (127, 768, 256), (128, 256, 256), (300, 256, 1024), (513, 264, 72),
                                   (1000, 768, 256), (64, 2048, 256)])
@pytest.mark.parametrize("use_bias", [False, True])
def test_linear_matches_oracle(device, m, n, k, use_bias):
    x, w, b = _draw(m, n, k, seed=m + n + k)
    bias = b if use_bias else None
    expected = F.linear(x.float(), w.float(), None if bias is None else bias.float())
    with torch.no_grad():
        got = linear(x.to(device), w.to(device), None if bias is None else bias.to(device))
    assert got.dtype == torch.bfloat16 and got.shape == (m, n)
    torch.testing.assert_close(got.cpu().float(), expected, **BF16_TOL)
    # the reference's bf16 torch path is inside the same tolerance
    torch.testing.assert_close(got.cpu().float(), F.linear(x, w, bias).float(), **BF16_TOL)


@pytest.mark.parametrize("m,n,k", [(1024, 256, 512), (1500, 256, 2048), (1025, 136, 520), (4096, 192, 768)])
@pytest.mark.parametrize("epilogue", ["none", "bias", "residual"])
def test_linear_long_contraction_into_a_narrow_output(device, m, n, k, epilogue):
    """Shapes served by the 256-token x all-features kernel (128 < N <= 256, K >= 512, M >= 1024): ragged token, feature
    and contraction tails, bias and residual epilogues."""
    x, w, b = _draw(m, n, k, seed=m + n + k)
    res = torch.randn(m, n, generator=torch.Generator().manual_seed(k)).to(torch.bfloat16)
    bias = None if epilogue == "none" else b
    expected = F.linear(x.float(), w.float(), None if bias is None else bias.float())
    if epilogue == "residual":
        expected = expected + res.float()
    with torch.no_grad():
        got = linear(x.to(device), w.to(device), None if bias is None else bias.to(device),
                     residual=res.to(device) if epilogue == "residual" else None)
    torch.testing.assert_close(got.cpu().float(), expected, **BF16_TOL)


def test_linear_residual_and_batch_dims(device):
    x, w, b = _draw(6 * 50, 256, 256, seed=4)
    x3 = x.view(6, 50, 256)
    g = torch.Generator().manual_seed(5)
    res = torch.randn(6, 50, 256, generator=g).to(torch.bfloat16)
    expected = res.float() + F.linear(x3.float(), w.float(), b.float())
    with torch.no_grad():
        got = linear(x3.to(device), w.to(device), b.to(device), residual=res.to(device))
    assert got.shape == (6, 50, 256)
    torch.testing.assert_close(got.cpu().float(), expected, **BF16_TOL)


@pytest.mark.parametrize("m,f,k", [(1, 8, 8), (200, 1024, 256), (129, 72, 64), (512, 64, 256)])
@pytest.mark.parametrize("gate_first", [True, False])
def test_swiglu_linear(device, m, f, k, gate_first):
    x, w, b = _draw(m, 2 * f, k, seed=m + f)
    expected = oracle.swiglu_hidden(x.float(), w.float(), b.float(), gate_first=gate_first)
    with torch.no_grad():
        got = swiglu_linear(x.to(device), w.to(device), b.to(device), gate_first=gate_first)
    assert got.shape == (m, f)
    torch.testing.assert_close(got.cpu().float(), expected, **BF16_TOL)


def test_swiglu_ffn_module_matches_reference_formula(device):
    torch.manual_seed(0)
    module = SwiGLUFeedForward(256, 4, 0.0).eval()
    x = (torch.randn(3, 40, 256)).to(torch.bfloat16)
    weights = {name: p.detach().to(torch.bfloat16) for name, p in module.named_parameters()}
    expected = oracle.swiglu_ffn(x, weights["up.weight"], weights["up.bias"], weights["down.weight"], weights["down.bias"])
    module = module.to(device)
    with torch.no_grad():
        got = module(x.to(device))
        got_fn = swiglu_ffn(x.to(device), weights["up.weight"].to(device), weights["up.bias"].to(device),
                            weights["down.weight"].to(device), weights["down.bias"].to(device))
    torch.testing.assert_close(got.cpu().float(), expected.float(), **BF16_TOL)
    torch.testing.assert_close(got_fn.cpu().float(), expected.float(), **BF16_TOL)


# ---- FP8 ---------------------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n", [1, 7, 8, 1000, 65536 + 3])
def test_amax_and_quantize_fp8(device, dtype, n):
    g = torch.Generator().manual_seed(n)
    x = (3.0 * torch.randn(n, generator=g)).to(dtype)
    with torch.no_grad():
        a = amax(x.to(device))
        q, a2 = quantize_fp8(x.to(device))
    assert a.item() == x.float().abs().max().item() == a2.item()
    expected_q, _ = oracle.fp8_quantize(x)
    assert torch.equal(q.cpu().view(torch.uint8), expected_q.view(torch.uint8))


def _rel_err(got, expected):
    return ((got.float() - expected.float()).abs().max() / expected.float().abs().max()).item()


@pytest.mark.parametrize("m,n,k", [(256, 768, 256), (130, 256, 256), (77, 256, 1024), (64, 64, 16)])
def test_linear_fp8_matches_emulation(device, m, n, k):
    x, w, b = _draw(m, n, k, seed=m * 3 + n)
    expected = oracle.linear_fp8(x, w, b)
    with torch.no_grad():
        wq, wa = quantize_fp8(w.to(device))
        xa = amax(x.to(device))
        got = linear_fp8(x.to(device), wq, xa, wa, b.to(device))
        # pre-quantised activations take the same path
        xq, _ = quantize_fp8(x.to(device), xa)
        got_q = linear_fp8(xq, wq, xa, wa, b.to(device))
    assert _rel_err(got.cpu(), expected) <= 5e-2
    assert _rel_err(got_q.cpu(), expected) <= 5e-2
    torch.testing.assert_close(got.cpu().float(), expected.float(), rtol=0, atol=5e-2 * expected.float().abs().max().item())


def test_linear_fp8_epilogues(device):
    m, f, k = 200, 1024, 256
    x, w, b = _draw(m, 2 * f, k, seed=77)
    expected = oracle.linear_fp8(x, w, b, swiglu=True)
    with torch.no_grad():
        wq, wa = quantize_fp8(w.to(device))
        xa = amax(x.to(device))
        got = linear_fp8(x.to(device), wq, xa, wa, b.to(device), swiglu=True)
    assert got.shape == (m, f)
    assert _rel_err(got.cpu(), expected) <= 5e-2
    x2, w2, b2 = _draw(m, 256, 1024, seed=78)
    res = torch.randn(m, 256, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    expected = oracle.linear_fp8(x2, w2, b2, residual=res)
    with torch.no_grad():
        wq, wa = quantize_fp8(w2.to(device))
        xa = amax(x2.to(device))
        got = linear_fp8(x2.to(device), wq, xa, wa, b2.to(device), residual=res.to(device))
    assert _rel_err(got.cpu(), expected) <= 5e-2


@pytest.mark.parametrize("workgroups", [None, 1, 2])
@pytest.mark.parametrize("epilogue", ["none", "residual", "swiglu", "swiglu_value_first"])
def test_linear_fp8_token_stationary_path(device, test_hooks, epilogue, workgroups):
    """K = 256 layers run on the token-stationary e4m3 kernel: every epilogue, bf16 and pre-quantised activations,
    ragged M, one and several token tiles per workgroup; and the tiled kernel (forced) gives the same numbers up to the
    rounding of the output."""
    if workgroups is not None:
        test_hooks(max_workgroups=workgroups)
    m, k = 1333, 256
    swiglu = epilogue.startswith("swiglu")
    gate_first = epilogue != "swiglu_value_first"
    n = 512 if swiglu else 320
    x, w, b = _draw(m, n, k, seed=len(epilogue) + (workgroups or 0))
    res = torch.randn(m, n, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16) if epilogue == "residual" else None
    expected = oracle.linear_fp8(x, w, b, residual=res, swiglu=swiglu, gate_first=gate_first)
    kwargs = dict(swiglu=swiglu, gate_first=gate_first, residual=None if res is None else res.to(device))
    with torch.no_grad():
        wq, wa = quantize_fp8(w.to(device))
        xa = amax(x.to(device))
        got = linear_fp8(x.to(device), wq, xa, wa, b.to(device), **kwargs)
        xq, _ = quantize_fp8(x.to(device), xa)
        got_q = linear_fp8(xq, wq, xa, wa, b.to(device), **kwargs)
        no_bias = linear_fp8(x.to(device), wq, xa, wa, None, **kwargs)
        test_hooks(fp8_tiled=True)
        tiled = linear_fp8(x.to(device), wq, xa, wa, b.to(device), **kwargs)
        tiled_no_bias = linear_fp8(x.to(device), wq, xa, wa, None, **kwargs)
    assert got.shape == expected.shape
    assert _rel_err(got.cpu(), expected) <= 5e-2
    assert _rel_err(got_q.cpu(), expected) <= 5e-2
    scale = expected.float().abs().max().item()
    torch.testing.assert_close(got.cpu().float(), tiled.cpu().float(), rtol=0, atol=2.0 ** -7 * scale)
    torch.testing.assert_close(no_bias.cpu().float(), tiled_no_bias.cpu().float(), rtol=0, atol=2.0 ** -7 * scale)


@pytest.mark.parametrize("epilogue", ["none", "residual"])
@pytest.mark.parametrize("workgroups", [None, 2])
def test_linear_fp8_token_stationary_long_reduction(device, test_hooks, epilogue, workgroups):
    """K = 1024 (the FFN down projection) on the token-stationary e4m3 kernel: one 32-row weight block per step, ragged
    M, several token tiles per workgroup, bf16 and pre-quantised activations, against the oracle and the tiled kernel."""
    if workgroups is not None:
        test_hooks(max_workgroups=workgroups)
    m, n, k = 1111, 96, 1024
    x, w, b = _draw(m, n, k, seed=17 + (workgroups or 0))
    res = torch.randn(m, n, generator=torch.Generator().manual_seed(6)).to(torch.bfloat16) if epilogue == "residual" else None
    expected = oracle.linear_fp8(x, w, b, residual=res)
    kwargs = dict(residual=None if res is None else res.to(device))
    with torch.no_grad():
        wq, wa = quantize_fp8(w.to(device))
        xa = amax(x.to(device))
        got = linear_fp8(x.to(device), wq, xa, wa, b.to(device), **kwargs)
        xq, _ = quantize_fp8(x.to(device), xa)
        got_q = linear_fp8(xq, wq, xa, wa, b.to(device), **kwargs)
        test_hooks(fp8_tiled=True)
        tiled = linear_fp8(x.to(device), wq, xa, wa, b.to(device), **kwargs)
    assert _rel_err(got.cpu(), expected) <= 5e-2
    assert _rel_err(got_q.cpu(), expected) <= 5e-2
    scale = expected.float().abs().max().item()
    torch.testing.assert_close(got.cpu().float(), tiled.cpu().float(), rtol=0, atol=2.0 ** -7 * scale)
    torch.testing.assert_close(got_q.cpu().float(), got.cpu().float(), rtol=0, atol=2.0 ** -7 * scale)


# ---- token-stationary fused kernels --------------------------------------------------------------------------------


@pytest.mark.parametrize("m,d,f", [(1, 256, 32), (300, 256, 1024), (64, 128, 64), (1000, 256, 96), (257, 128, 256)])
@pytest.mark.parametrize("gate_first", [True, False])
def test_fused_swiglu_ffn(device, m, d, f, gate_first):
    """RMSNorm -> up -> SiLU-gate -> down -> + residual in one kernel against the oracle's pieces evaluated in fp32."""
    from taac_2026_amd.api import swiglu_ffn

    g = torch.Generator().manual_seed(m + d + f)
    x = torch.randn(m, d, generator=g).to(torch.bfloat16)
    nw = (1 + 0.1 * torch.randn(d, generator=g)).to(torch.bfloat16)
    wu = (torch.randn(2 * f, d, generator=g) * (2.0 / (d + 2 * f)) ** 0.5).to(torch.bfloat16)
    bu = (0.1 * torch.randn(2 * f, generator=g)).to(torch.bfloat16)
    wd = (torch.randn(d, f, generator=g) * (2.0 / (d + f)) ** 0.5).to(torch.bfloat16)
    bd = (0.1 * torch.randn(d, generator=g)).to(torch.bfloat16)
    h = oracle.rms_norm_fp32(x, nw)
    expected = x.float() + oracle.swiglu_ffn(h.float(), wu.float(), bu.float(), wd.float(), bd.float(), gate_first=gate_first)
    with torch.no_grad():
        got = swiglu_ffn(x.to(device), wu.to(device), bu.to(device), wd.to(device), bd.to(device), residual=x.to(device),
                         norm_weight=nw.to(device), gate_first=gate_first)
        plain = swiglu_ffn(x.to(device), wu.to(device), None, wd.to(device), None)
    torch.testing.assert_close(got.cpu().float(), expected, **BF16_TOL)
    torch.testing.assert_close(plain.cpu().float(), oracle.swiglu_ffn(x.float(), wu.float(), None, wd.float(), None), **BF16_TOL)
    # the reference's bf16 evaluation of the same expression stays inside the same tolerance
    ref_bf16 = x + oracle.swiglu_ffn(oracle.rms_norm(x, nw), wu, bu, wd, bd, gate_first=gate_first)
    torch.testing.assert_close(got.cpu().float(), ref_bf16.float(), rtol=4e-2, atol=4e-2)


@pytest.mark.parametrize("m,d,f", [(300, 256, 1024), (65, 128, 96)])
@pytest.mark.parametrize("gate_first", [True, False])
@pytest.mark.parametrize("with_norm", [True, False])
def test_fused_ffn_with_the_activation_constants_in_the_packed_weights(device, m, d, f, gate_first, with_norm):
    """``fold_activation``: the packed up projection carries -log2(e) (gated half) and -ln(2) (other half), the kernel
    evaluates ``g' * u' / (1 + 2^g')``. Both forms against the oracle's fp32 evaluation, with biases, either gate order,
    with and without the norm in front (whose weight shares the rounding); the two forms differ by rounding only. The
    block tail (rows and per-head planes) likewise. A hidden size that leaves no room for the kernels' third weight
    buffer takes the plain blob."""
    from taac_2026_amd.api import attention_out_ffn, swiglu_ffn
    from taac_2026_amd.accelerators.linear import attention_out_ffn_heads, ffn_activation_fold_supported

    assert ffn_activation_fold_supported(d, f) and not ffn_activation_fold_supported(256, 4096)
    attn, h, nw, wo, bo, wu, bu, wd, bd = _block_tail_inputs(m, d, f, seed=m + f + int(gate_first))
    norm = nw if with_norm else None
    x = h
    xin = oracle.rms_norm_fp32(x, nw).float() if with_norm else x.float()
    expected = x.float() + oracle.swiglu_ffn(xin, wu.float(), bu.float(), wd.float(), bd.float(), gate_first=gate_first)
    dev = lambda t: None if t is None else t.to(device)
    results = {}
    with torch.no_grad():
        for fold in (False, True, None):
            results[fold] = swiglu_ffn(dev(x), dev(wu), dev(bu), dev(wd), dev(bd), residual=dev(x), norm_weight=dev(norm),
                                       gate_first=gate_first, fold_activation=fold).cpu().float()
            torch.testing.assert_close(results[fold], expected, **BF16_TOL)
    assert torch.equal(results[None], results[True])
    step = 2.0 ** -7
    assert (results[True] - results[False]).abs().max().item() <= 4 * step * max(1.0, expected.abs().max().item())
    assert (results[True] - expected).abs().mean().item() <= 1.25 * (results[False] - expected).abs().mean().item() + 1e-4
    if gate_first:
        heads = d // 32
        planes = attn.view(m, heads, 32).transpose(0, 1).contiguous()
        with torch.no_grad():
            tails = {fold: attention_out_ffn(dev(attn), dev(wo), dev(bo), dev(h), dev(wu), dev(bu), dev(wd), dev(bd),
                                             norm_weight=dev(norm), fold_activation=fold).cpu().float() for fold in (False, True)}
            from_planes = attention_out_ffn_heads(dev(planes), dev(wo), dev(bo), dev(h), dev(wu), dev(bu), dev(wd), dev(bd),
                                                  norm_weight=dev(norm), fold_activation=True).cpu().float()
        assert torch.equal(from_planes, tails[True])
        x1 = (h.float() + (attn.float() @ wo.float().t() + bo.float()).to(torch.bfloat16).float()).to(torch.bfloat16)
        x1n = oracle.rms_norm_fp32(x1, nw).float() if with_norm else x1.float()
        tail_expected = x1.float() + oracle.swiglu_ffn(x1n, wu.float(), bu.float(), wd.float(), bd.float())
        for fold in (False, True):
            torch.testing.assert_close(tails[fold], tail_expected, **BF16_TOL)
    # no room for three weight buffers: the wrappers fall back to the plain blob, an explicit request is refused
    wide_up = (torch.randn(2 * 4096, 256, generator=torch.Generator().manual_seed(1)) * 0.02).to(torch.bfloat16)
    wide_down = (torch.randn(256, 4096, generator=torch.Generator().manual_seed(2)) * 0.02).to(torch.bfloat16)
    xs = torch.randn(8, 256, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    with torch.no_grad():
        wide = swiglu_ffn(dev(xs), dev(wide_up), None, dev(wide_down), None).cpu().float()
        torch.testing.assert_close(wide, oracle.swiglu_ffn(xs.float(), wide_up.float(), None, wide_down.float(), None), **BF16_TOL)
        with pytest.raises(RuntimeError):
            swiglu_ffn(dev(xs), dev(wide_up), None, dev(wide_down), None, fold_activation=True)


def _block_tail_inputs(m, d, f, seed):
    g = torch.Generator().manual_seed(seed)
    attn = torch.randn(m, d, generator=g).to(torch.bfloat16)
    h = torch.randn(m, d, generator=g).to(torch.bfloat16)
    nw = (1 + 0.1 * torch.randn(d, generator=g)).to(torch.bfloat16)
    wo = (torch.randn(d, d, generator=g) * (1.0 / d) ** 0.5).to(torch.bfloat16)
    bo = (0.1 * torch.randn(d, generator=g)).to(torch.bfloat16)
    wu = (torch.randn(2 * f, d, generator=g) * (2.0 / (d + 2 * f)) ** 0.5).to(torch.bfloat16)
    bu = (0.1 * torch.randn(2 * f, generator=g)).to(torch.bfloat16)
    wd = (torch.randn(d, f, generator=g) * (2.0 / (d + f)) ** 0.5).to(torch.bfloat16)
    bd = (0.1 * torch.randn(d, generator=g)).to(torch.bfloat16)
    return attn, h, nw, wo, bo, wu, bu, wd, bd


@pytest.mark.parametrize("m,d,f", [(1, 256, 32), (300, 256, 1024), (64, 128, 64), (1000, 256, 96), (257, 128, 256),
                                   (2500, 256, 64)])
@pytest.mark.parametrize("workgroups", [None, 3])
def test_fused_attention_out_ffn(device, test_hooks, m, d, f, workgroups):
    """out projection + residual -> RMSNorm -> up -> SiLU-gate -> down -> + residual in one kernel, against the oracle's
    pieces (dense layers evaluated in fp32 from the stored operands, the residual stream rounded to bf16 in between) and
    against the two-kernel route of the same library."""
    from taac_2026_amd.api import attention_out_ffn, norm_linear, swiglu_ffn

    if workgroups is not None:
        test_hooks(max_workgroups=workgroups)
    attn, h, nw, wo, bo, wu, bu, wd, bd = _block_tail_inputs(m, d, f, seed=m + d + f)
    lin = F.linear(attn.float(), wo.float(), bo.float()).to(torch.bfloat16)
    x1 = (lin.float() + h.float()).to(torch.bfloat16)
    expected = x1.float() + oracle.swiglu_ffn(oracle.rms_norm_fp32(x1, nw).float(), wu.float(), bu.float(), wd.float(), bd.float())
    to = lambda t: t.to(device)
    with torch.no_grad():
        got = attention_out_ffn(to(attn), to(wo), to(bo), to(h), to(wu), to(bu), to(wd), to(bd), norm_weight=to(nw))
        mid = norm_linear(to(attn), to(wo), to(bo), residual=to(h))
        two = swiglu_ffn(mid, to(wu), to(bu), to(wd), to(bd), residual=mid, norm_weight=to(nw))
        bare = attention_out_ffn(to(attn), to(wo), None, to(h), to(wu), None, to(wd), None)
    assert got.shape == attn.shape and got.dtype == torch.bfloat16
    torch.testing.assert_close(got.cpu().float(), expected, **BF16_TOL)
    # x1 is bit-identical on both routes; the one-kernel route rounds x1 + down + b_down once, the other twice
    torch.testing.assert_close(got.cpu().float(), two.cpu().float(), rtol=2 ** -6, atol=2 ** -6)
    x1_bare = (F.linear(attn.float(), wo.float()).to(torch.bfloat16).float() + h.float()).to(torch.bfloat16)
    expected_bare = x1_bare.float() + oracle.swiglu_ffn(x1_bare.float(), wu.float(), None, wd.float(), None)
    torch.testing.assert_close(bare.cpu().float(), expected_bare, **BF16_TOL)


def test_fused_attention_out_ffn_in_place_on_valid_rows(device):
    """With a row index and out = residual the kernel updates the residual stream in place: valid rows equal the dense
    run bit for bit, padded rows (NaN in every operand here) are neither read nor written."""
    from taac_2026_amd.api import attention_out_ffn, valid_rows

    batch, tokens, d, f = 7, 150, 256, 64
    lengths = torch.tensor([150, 0, 1, 77, 149, 33, 64], dtype=torch.int32)
    valid = (torch.arange(tokens)[None, :] < lengths[:, None]).flatten()
    attn, h, nw, wo, bo, wu, bu, wd, bd = _block_tail_inputs(batch * tokens, d, f, seed=5)
    to = lambda t: t.to(device)
    with torch.no_grad():
        dense = attention_out_ffn(to(attn), to(wo), to(bo), to(h), to(wu), to(bu), to(wd), to(bd), norm_weight=to(nw))
        attn_p, h_p = attn.clone(), h.clone()
        attn_p[~valid] = float("nan")
        h_p[~valid] = float("nan")
        stream = to(h_p)
        result = attention_out_ffn(to(attn_p), to(wo), to(bo), stream, to(wu), to(bu), to(wd), to(bd), norm_weight=to(nw),
                                   token_rows=valid_rows(to(lengths), tokens), out=stream)
    assert result.data_ptr() == stream.data_ptr()
    assert torch.equal(result.cpu()[valid], dense.cpu()[valid])
    assert torch.isnan(result.cpu()[~valid].float()).all()


def test_fused_attention_out_ffn_rejects_other_shapes(device):
    from taac_2026_amd.api import attention_out_ffn

    attn, h, nw, wo, bo, wu, bu, wd, bd = _block_tail_inputs(8, 64, 32, seed=1)
    to = lambda t: t.to(device)
    with pytest.raises(RuntimeError, match="width 128 / 256"):
        attention_out_ffn(to(attn), to(wo), to(bo), to(h), to(wu), to(bu), to(wd), to(bd))


@pytest.mark.parametrize("m,k,n", [(1, 256, 64), (300, 256, 768), (64, 128, 256), (1000, 256, 256), (513, 128, 768)])
def test_fused_norm_linear(device, m, k, n):
    from taac_2026_amd.api import norm_linear

    x, w, b = _draw(m, n, k, seed=m + n)
    g = torch.Generator().manual_seed(7)
    nw = (1 + 0.1 * torch.randn(k, generator=g)).to(torch.bfloat16)
    res = torch.randn(m, n, generator=g).to(torch.bfloat16)
    expected = res.float() + F.linear(oracle.rms_norm_fp32(x, nw).float(), w.float(), b.float())
    with torch.no_grad():
        got = norm_linear(x.to(device), w.to(device), b.to(device), norm_weight=nw.to(device), residual=res.to(device))
        plain = norm_linear(x.to(device), w.to(device))
    torch.testing.assert_close(got.cpu().float(), expected, **BF16_TOL)
    torch.testing.assert_close(plain.cpu().float(), F.linear(x.float(), w.float()), **BF16_TOL)


@pytest.mark.parametrize("workgroups", [1, 2, 3])
@pytest.mark.parametrize("m,k,n", [(3000, 256, 768), (2049, 128, 256), (1500, 256, 64)])
def test_fused_norm_linear_walks_several_token_tiles(device, test_hooks, workgroups, m, k, n):
    """The linear kernel is persistent: with few workgroups each one walks several token tiles (what happens at full
    size on 256 compute units), including the out-of-phase tile changes of its two wavefront groups and the residual
    pieces requested one step ahead across a tile boundary."""
    from taac_2026_amd.api import norm_linear

    test_hooks(max_workgroups=workgroups)
    x, w, b = _draw(m, n, k, seed=m + n + workgroups)
    g = torch.Generator().manual_seed(11)
    nw = (1 + 0.1 * torch.randn(k, generator=g)).to(torch.bfloat16)
    res = torch.randn(m, n, generator=g).to(torch.bfloat16)
    expected = res.float() + F.linear(oracle.rms_norm_fp32(x, nw).float(), w.float(), b.float())
    with torch.no_grad():
        got = norm_linear(x.to(device), w.to(device), b.to(device), norm_weight=nw.to(device), residual=res.to(device))
        plain = norm_linear(x.to(device), w.to(device))
    torch.testing.assert_close(got.cpu().float(), expected, **BF16_TOL)
    torch.testing.assert_close(plain.cpu().float(), F.linear(x.float(), w.float()), **BF16_TOL)


def test_valid_rows_index(device):
    """Row index of a padded batch: valid rows in increasing order, count, per-sample offsets; lengths are clamped to
    [0, T]."""
    from taac_2026_amd.api import valid_rows

    tokens = 37
    lengths = torch.tensor([5, 0, 37, 12, 99, -3, 1], dtype=torch.int32)
    rows, count = valid_rows(lengths.to(device), tokens)
    clamped = lengths.clamp(0, tokens)
    expected = torch.cat([b * tokens + torch.arange(int(n)) for b, n in enumerate(clamped)]).to(torch.int32)
    n = int(count.item())
    assert n == int(clamped.sum())
    assert torch.equal(rows[:n].cpu(), expected)
    offsets = rows[len(lengths) * tokens:len(lengths) * tokens + len(lengths) + 1].cpu()
    assert torch.equal(offsets, torch.cat([torch.zeros(1, dtype=torch.int64), clamped.cumsum(0)]).to(torch.int32))
    big = torch.randint(0, 513, (3000,), dtype=torch.int32, generator=torch.Generator().manual_seed(0))
    rows, count = valid_rows(big.to(device), 512)
    assert int(count.item()) == int(big.sum())
    mask = torch.arange(512)[None, :] < big[:, None]
    assert torch.equal(rows[:int(count.item())].cpu().long(), mask.flatten().nonzero().flatten())


@pytest.mark.parametrize("workgroups", [None, 2])
def test_fused_layers_skip_padded_rows(device, test_hooks, workgroups):
    """With a row index the fused layers process exactly the valid rows of a padded batch: those rows are bit-identical
    to the dense run, all other rows are neither read (they hold NaN here) nor written."""
    from taac_2026_amd.api import norm_linear, swiglu_ffn, valid_rows

    if workgroups is not None:
        test_hooks(max_workgroups=workgroups)
    g = torch.Generator().manual_seed(21)
    batch, tokens, d, f = 9, 200, 256, 96
    lengths = torch.tensor([200, 1, 0, 77, 128, 199, 33, 64, 160], dtype=torch.int32)
    valid = (torch.arange(tokens)[None, :] < lengths[:, None]).flatten()
    x = torch.randn(batch * tokens, d, generator=g).to(torch.bfloat16)
    res = torch.randn(batch * tokens, d, generator=g).to(torch.bfloat16)
    nw = (1 + 0.1 * torch.randn(d, generator=g)).to(torch.bfloat16)
    _, w, b = _draw(1, 768, d, seed=1)
    _, wo, bo = _draw(1, d, d, seed=2)
    _, wu, bu = _draw(1, 2 * f, d, seed=3)
    _, wd, bd = _draw(1, d, f, seed=4)
    poisoned = x.clone()
    poisoned[~valid] = float("nan")
    res_poisoned = res.clone()
    res_poisoned[~valid] = float("nan")
    to = lambda t: t.to(device)
    with torch.no_grad():
        index = valid_rows(to(lengths), tokens)
        dense_qkv = norm_linear(to(x), to(w), to(b), norm_weight=to(nw))
        skip_qkv = norm_linear(to(poisoned), to(w), to(b), norm_weight=to(nw), token_rows=index)
        dense_out = norm_linear(to(x), to(wo), to(bo), residual=to(res))
        skip_out = norm_linear(to(poisoned), to(wo), to(bo), residual=to(res_poisoned), token_rows=index)
        dense_ffn = swiglu_ffn(to(x), to(wu), to(bu), to(wd), to(bd), residual=to(res), norm_weight=to(nw))
        skip_ffn = swiglu_ffn(to(poisoned), to(wu), to(bu), to(wd), to(bd), residual=to(res_poisoned), norm_weight=to(nw),
                              token_rows=index)
    for dense, skipped in ((dense_qkv, skip_qkv), (dense_out, skip_out), (dense_ffn, skip_ffn)):
        assert torch.equal(skipped.cpu()[valid], dense.cpu()[valid])
        assert (skipped.cpu()[~valid] == 0).all()


def test_fused_paths_fall_back_for_other_widths(device):
    from taac_2026_amd.api import norm_linear, swiglu_ffn

    x, w, b = _draw(100, 72, 96, seed=3)  # K = 96, N = 72: not a token-stationary shape
    with torch.no_grad():
        got = norm_linear(x.to(device), w.to(device), b.to(device))
    torch.testing.assert_close(got.cpu().float(), F.linear(x.float(), w.float(), b.float()), **BF16_TOL)
    _, wu, _ = _draw(1, 2 * 40, 96, seed=4)
    _, wd, _ = _draw(1, 96, 40, seed=5)
    with torch.no_grad():
        got = swiglu_ffn(x.to(device), wu.to(device), None, wd.to(device), None, residual=x.to(device))
    expected = x.float() + oracle.swiglu_ffn(x.float(), wu.float(), None, wd.float(), None)
    torch.testing.assert_close(got.cpu().float(), expected, **BF16_TOL)
