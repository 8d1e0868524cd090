"""GPU parity of the float16 dense layers (the tiled MFMA kernel with float16 operands) and of the modules on float16 tokens."""

from __future__ import annotations

import pytest
import torch
import torch.nn.functional as F

from oracle import reference as oracle
from taac_2026_amd.api import SwiGLUFeedForward, UnifiedSelfAttention, linear, norm_linear, silu_mlp, swiglu_ffn, swiglu_linear

pytestmark = pytest.mark.gpu

# float16 tolerance of the reference's GPU tests (tests/gpu/infrastructure/accelerators/test_tilelang_ops_cuda.py:205)
TOL = dict(rtol=5e-3, atol=5e-3)


def _draw(m, n, k, seed):
    g = torch.Generator().manual_seed(seed)
    h = lambda t: t.to(torch.float16)  # noqa: E731
    return (h(torch.randn(m, k, generator=g)), h(torch.randn(n, k, generator=g) * k ** -0.5), h(0.1 * torch.randn(n, generator=g)))


@pytest.mark.parametrize("m,n,k", [(1, 8, 8), (77, 200, 96), (300, 768, 256), (1031, 256, 1024), (129, 136, 264)])
def test_linear_f16_epilogues(device, m, n, k):
    x, w, b = _draw(m, n, k, seed=m + n)
    res = torch.randn(m, n, generator=torch.Generator().manual_seed(1)).to(torch.float16)
    to = lambda t: t.to(device)  # noqa: E731
    with torch.no_grad():
        plain = linear(to(x), to(w), to(b))
        no_bias = linear(to(x), to(w))
        with_res = linear(to(x), to(w), to(b), residual=to(res))
    assert plain.dtype == torch.float16
    want = F.linear(x.float(), w.float(), b.float())
    torch.testing.assert_close(plain.cpu().float(), want, **TOL)
    torch.testing.assert_close(no_bias.cpu().float(), F.linear(x.float(), w.float()), **TOL)
    torch.testing.assert_close(with_res.cpu().float(), want + res.float(), **TOL)
    if n % 2 == 0 and (n // 2) % 8 == 0:
        for gate_first in (True, False):
            with torch.no_grad():
                gated = swiglu_linear(to(x), to(w), to(b), gate_first=gate_first)
            torch.testing.assert_close(gated.cpu().float(),
                                       oracle.swiglu_hidden(x.float(), w.float(), b.float(), gate_first=gate_first), **TOL)


@pytest.mark.parametrize("d,f", [(256, 1024), (128, 384), (64, 96)])
def test_composed_layers_on_float16(device, d, f):
    """``norm_linear``, ``swiglu_ffn`` and ``silu_mlp`` on float16 tensors (layer by layer on the tiled kernel, also at the
    widths whose bfloat16 form is one fused kernel) against the fp32 evaluation of the same formulas."""
    g = torch.Generator().manual_seed(d + f)
    h = lambda t: t.to(torch.float16)  # noqa: E731
    m = 333
    x = h(torch.randn(m, d, generator=g))
    wn = h(1 + 0.1 * torch.randn(d, generator=g))
    wu, bu = h(torch.randn(2 * f, d, generator=g) * d ** -0.5), h(0.1 * torch.randn(2 * f, generator=g))
    wd, bd = h(torch.randn(d, f, generator=g) * f ** -0.5), h(0.1 * torch.randn(d, generator=g))
    w1, b1 = h(torch.randn(f, d, generator=g) * d ** -0.5), h(0.1 * torch.randn(f, generator=g))
    to = lambda t: t.to(device)  # noqa: E731
    with torch.no_grad():
        ffn = swiglu_ffn(to(x), to(wu), to(bu), to(wd), to(bd), residual=to(x), norm_weight=to(wn))
        mlp = silu_mlp(to(x), to(w1), to(b1), to(wd), to(bd), residual=to(x), norm_weight=to(wn))
        proj = norm_linear(to(x), to(wu), to(bu), norm_weight=to(wn))
    assert ffn.dtype == mlp.dtype == proj.dtype == torch.float16
    n = oracle.rms_norm_fp32(x, wn).float()
    f32 = lambda *ts: [t.float() for t in ts]  # noqa: E731
    torch.testing.assert_close(ffn.cpu().float(), x.float() + oracle.swiglu_ffn(n, *f32(wu, bu, wd, bd)), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(mlp.cpu().float(), x.float() + oracle.silu_mlp(n, *f32(w1, b1, wd, bd)), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(proj.cpu().float(), F.linear(n, wu.float(), bu.float()), rtol=1e-2, atol=1e-2)


def test_modules_keep_float16_tokens_in_float16(device):
    """A float16 model (weights and tokens) runs its feed-forward and attention layers in float16: results against the fp32
    evaluation at the float16 tolerance (a bfloat16 detour would miss it), and a gradient is refused with a clear message."""
    torch.manual_seed(5)
    d, heads, tokens, batch = 128, 4, 48, 3
    ffn = SwiGLUFeedForward(d, 4, 0.0).to(torch.float16).eval()
    attention = UnifiedSelfAttention(d, heads, 0.0, qk_norm=True).to(torch.float16).eval()
    x = (0.7 * torch.randn(batch, tokens, d)).to(torch.float16)
    lengths = torch.tensor([48, 20, 1], dtype=torch.int32)
    sd = {k: v.detach().float() for k, v in ffn.state_dict().items()}
    want_ffn = oracle.swiglu_ffn(x.float(), sd["up.weight"], sd["up.bias"], sd["down.weight"], sd["down.bias"])
    sa = {k: v.detach().float() for k, v in attention.state_dict().items()}
    q, k, v = F.linear(x.float(), sa["qkv.weight"], sa["qkv.bias"]).chunk(3, -1)
    q, k = oracle.rms_norm(q, sa["query_norm.weight"]), oracle.rms_norm(k, sa["key_norm.weight"])
    a = oracle.scaled_dot_product_attention(q, k, v, num_heads=heads, key_lengths=lengths)
    want_attn = F.linear(a, sa["out.weight"], sa["out.bias"])
    ffn, attention = ffn.to(device), attention.to(device)
    with torch.no_grad():
        got_ffn = ffn(x.to(device))
        got_attn = attention(x.to(device), None, key_lengths=lengths.to(device))
    assert got_ffn.dtype == got_attn.dtype == torch.float16
    torch.testing.assert_close(got_ffn.cpu().float(), want_ffn, rtol=1e-2, atol=1e-2)
    valid = torch.arange(tokens)[None, :] < lengths[:, None]
    torch.testing.assert_close(got_attn.cpu().float()[valid], want_attn[valid], rtol=1e-2, atol=1e-2)
    with pytest.raises(RuntimeError, match="forward-only"):
        ffn(x.to(device).requires_grad_(True))
    with pytest.raises(RuntimeError, match="one 16-bit dtype"):
        linear(x.to(device), ffn.up.weight.detach().to(torch.bfloat16))
