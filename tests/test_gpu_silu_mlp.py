"""GPU parity of the plain SiLU feed-forward (OneTrans) on the fused kernel and of its modules."""

from __future__ import annotations

import pytest
import torch

from oracle import reference as oracle
from taac_2026_amd.api import FeedForward, MixedFeedForward, silu_mlp, valid_rows

pytestmark = pytest.mark.gpu


def _draw(m, d, f, seed):
    g = torch.Generator().manual_seed(seed)
    bf = lambda t: t.to(torch.bfloat16)  # noqa: E731
    x = bf(torch.randn(m, d, generator=g))
    w1, b1 = bf(torch.randn(f, d, generator=g) * d ** -0.5), bf(0.2 * torch.randn(f, generator=g))
    w2, b2 = bf(torch.randn(d, f, generator=g) * f ** -0.5), bf(0.2 * torch.randn(d, generator=g))
    wn = bf(1 + 0.1 * torch.randn(d, generator=g))
    return x, w1, b1, w2, b2, wn


@pytest.mark.parametrize("workgroups", [None, 2])
@pytest.mark.parametrize("m,d,f", [(1, 128, 32), (300, 128, 512), (257, 256, 96), (1111, 256, 1024)])
def test_silu_mlp_fused_kernel(device, test_hooks, m, d, f, workgroups):
    """``taac_silu_mlp_fwd`` against the oracle: plain, with the norm in front and the residual behind, without biases,
    ragged M, one and several token tiles per workgroup."""
    if workgroups is not None:
        test_hooks(max_workgroups=workgroups)
    x, w1, b1, w2, b2, wn = _draw(m, d, f, seed=m + f)
    to = lambda t: t.to(device)  # noqa: E731
    with torch.no_grad():
        plain = silu_mlp(to(x), to(w1), to(b1), to(w2), to(b2))
        no_bias = silu_mlp(to(x), to(w1), None, to(w2), None)
        full = silu_mlp(to(x), to(w1), to(b1), to(w2), to(b2), residual=to(x), norm_weight=to(wn))
    f32 = lambda *ts: [t.float() for t in ts]  # noqa: E731
    torch.testing.assert_close(plain.cpu().float(), oracle.silu_mlp(*f32(x, w1, b1, w2, b2)), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(no_bias.cpu().float(), oracle.silu_mlp(x.float(), w1.float(), None, w2.float(), None),
                               rtol=2e-2, atol=2e-2)
    want = x.float() + oracle.silu_mlp(oracle.rms_norm(x.float(), wn.float()), *f32(w1, b1, w2, b2))
    torch.testing.assert_close(full.cpu().float(), want, rtol=2e-2, atol=2e-2)


def test_silu_mlp_row_index_and_strided_rows(device):
    """Rows listed by an index only (the others untouched, listed rows bit-identical to the dense run) and rows read
    through a stride (one token of every sample of a [B, T, D] stream)."""
    d, f, batch, tokens = 256, 512, 9, 40
    g = torch.Generator().manual_seed(3)
    stream = (0.7 * torch.randn(batch, tokens, d, generator=g)).to(torch.bfloat16)
    _, w1, b1, w2, b2, _ = _draw(1, d, f, seed=5)
    lengths = torch.randint(0, tokens + 1, (batch,), generator=g, dtype=torch.int32)
    lengths[0], lengths[1] = tokens, 0
    to = lambda t: t.to(device)  # noqa: E731
    with torch.no_grad():
        dense = silu_mlp(to(stream), to(w1), to(b1), to(w2), to(b2))
        out = torch.full_like(dense, 5.0)
        silu_mlp(to(stream), to(w1), to(b1), to(w2), to(b2), token_rows=valid_rows(to(lengths), tokens), out=out)
        one_token = silu_mlp(to(stream)[:, 7, :], to(w1), to(b1), to(w2), to(b2))
    valid = torch.arange(tokens)[None, :] < lengths[:, None]
    assert torch.equal(out.cpu()[valid], dense.cpu()[valid])
    assert (out.cpu()[~valid] == 5.0).all()
    assert torch.equal(one_token.cpu(), dense.cpu()[:, 7, :])


def test_feed_forward_modules(device):
    """``FeedForward`` / ``MixedFeedForward`` (parameter names of the reference's modules) against the oracle: the fused
    route, fp32 tokens, the fused norm + residual, the token-specific layers at the end of the stream (the last one
    falls beyond the sequence and is skipped), and a gradient through the unfused route."""
    torch.manual_seed(11)
    d, mult, batch, tokens, ns = 128, 4, 6, 20, 3
    module = MixedFeedForward(d, mult, ns, 0.0).to(torch.bfloat16).eval()
    assert set(dict(module.shared.named_parameters())) == {"net.0.weight", "net.0.bias", "net.3.weight", "net.3.bias"}
    x = (0.8 * torch.randn(batch, tokens, d)).to(torch.bfloat16)
    weights = lambda ffn: tuple(p.detach().float() for p in (ffn.net[0].weight, ffn.net[0].bias, ffn.net[3].weight, ffn.net[3].bias))  # noqa: E731
    seq_token_count = tokens - 2
    shared_w, specific_w = weights(module.shared), [weights(f) for f in module.ns_specific]
    want = oracle.mixed_feed_forward(x.float(), seq_token_count, shared_w, specific_w)
    module = module.to(device)
    with torch.no_grad():
        got = module(x.to(device), seq_token_count)
        got32 = module(x.to(device).float(), seq_token_count)
        wn = (1 + 0.1 * torch.randn(d)).to(torch.bfloat16)
        fused = module.shared(x.to(device), residual=x.to(device), norm_weight=wn.to(device))
    torch.testing.assert_close(got.cpu().float(), want, rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(got32.cpu(), want, rtol=2e-2, atol=2e-2)
    assert got32.dtype == torch.float32
    want_fused = x.float() + oracle.silu_mlp(oracle.rms_norm(x.float(), wn.float()), *shared_w)
    torch.testing.assert_close(fused.cpu().float(), want_fused, rtol=2e-2, atol=2e-2)
    xg = x.to(device).requires_grad_(True)
    module(xg, seq_token_count).float().sum().backward()
    reference = x.float().clone().requires_grad_(True)
    oracle.mixed_feed_forward(reference, seq_token_count, shared_w, specific_w).sum().backward()
    scale = reference.grad.abs().max().item()
    assert (xg.grad.cpu().float() - reference.grad).abs().max().item() <= 3e-2 * scale


def test_silu_mlp_errors(device):
    x, w1, b1, w2, b2, _ = _draw(8, 128, 64, seed=1)
    to = lambda t: t.to(device)  # noqa: E731
    with pytest.raises(ValueError, match="fc1_weight"):
        silu_mlp(to(x), to(w1), to(b1), to(w1), to(b2))
    with pytest.raises(RuntimeError, match="CUDA"):
        silu_mlp(x, w1, b1, w2, b2)
    with pytest.raises(RuntimeError, match="token_rows"):
        silu_mlp(to(x).requires_grad_(True), to(w1), to(b1), to(w2), to(b2), out=torch.empty(8, 128, device=device, dtype=torch.bfloat16))
