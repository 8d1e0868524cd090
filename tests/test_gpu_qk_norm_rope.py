"""GPU parity: the one-pass query / key RMSNorm + rotary embedding (through the C ABI) against the CPU oracle, and the
attention layers that use it."""

from __future__ import annotations

import pytest
import torch
import torch.nn.functional as F

from oracle import reference as oracle
from taac_2026_amd.api import BFTSAttention, UnifiedSelfAttention, qk_norm_rope, valid_rows

pytestmark = pytest.mark.gpu

# fp32 1e-5 and bf16 2e-2 are the benchmark configuration's tolerances for the norms; fp16 5e-3 is the reference's GPU
# test tolerance (tests/gpu/infrastructure/accelerators/test_tilelang_ops_cuda.py:205). The rotary table is rounded to
# the storage dtype on both sides.
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 5e-3}


def _draw(batch, tokens, d_model, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    q = (1.5 * torch.randn(batch, tokens, d_model, generator=g)).to(dtype)
    k = (0.7 * torch.randn(batch, tokens, d_model, generator=g)).to(dtype)
    wq = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(dtype)
    wk = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(dtype)
    return q, k, wq, wk


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(2, 7, 256, 8), (3, 5, 64, 2), (1, 33, 1024, 8), (2, 9, 32, 4), (1, 3, 2048, 16),
                                   (5, 130, 128, 4), (1, 6, 1536, 12)])
@pytest.mark.parametrize("mode", ["norm", "rope", "norm+rope"])
def test_qk_norm_rope_matches_oracle(device, dtype, shape, mode):
    batch, tokens, d_model, heads = shape
    q, k, wq, wk = _draw(batch, tokens, d_model, dtype, seed=d_model + tokens)
    weights = (wq, wk) if "norm" in mode else (None, None)
    base = 10000.0 if "rope" in mode else None
    expected_q, expected_k = oracle.qk_norm_rope(q, k, *weights, num_heads=heads, eps=1e-6, rope_base=base, fp32=True)
    with torch.no_grad():
        got_q, got_k = qk_norm_rope(q.to(device), k.to(device), *(None if w is None else w.to(device) for w in weights),
                                    num_heads=heads, eps=1e-6, rope_base=base)
    assert got_q.shape == q.shape and got_q.dtype == dtype and got_q.is_contiguous()
    torch.testing.assert_close(got_q.cpu().float(), expected_q.float(), rtol=TOL[dtype], atol=TOL[dtype])
    torch.testing.assert_close(got_k.cpu().float(), expected_k.float(), rtol=TOL[dtype], atol=TOL[dtype])
    if dtype == torch.bfloat16:
        # the reference's own evaluation order (every intermediate rounded to bf16) stays within twice the tolerance
        ref_q, ref_k = oracle.qk_norm_rope(q, k, *weights, num_heads=heads, eps=1e-6, rope_base=base)
        torch.testing.assert_close(got_q.cpu().float(), ref_q.float(), rtol=4e-2, atol=4e-2)
        torch.testing.assert_close(got_k.cpu().float(), ref_k.float(), rtol=4e-2, atol=4e-2)


def test_qk_norm_rope_in_place_on_a_packed_projection(device):
    """q and k are the chunk views of a [B, T, 3D] projection: the pass runs in place with the packed row stride, equals
    the out-of-place result bit for bit and leaves the value columns alone."""
    batch, tokens, d_model, heads = 3, 50, 256, 8
    g = torch.Generator().manual_seed(11)
    packed = torch.randn(batch, tokens, 3 * d_model, generator=g).to(torch.bfloat16)
    wq = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
    wk = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
    q, k, v = packed.chunk(3, dim=-1)
    expected_q, expected_k = oracle.qk_norm_rope(q, k, wq, wk, num_heads=heads, rope_base=10000.0, fp32=True)
    with torch.no_grad():
        dev = packed.to(device)
        dq, dk, dv = dev.chunk(3, dim=-1)
        fresh_q, fresh_k = qk_norm_rope(dq, dk, wq.to(device), wk.to(device), num_heads=heads, rope_base=10000.0)
        out_q, out_k = qk_norm_rope(dq, dk, wq.to(device), wk.to(device), num_heads=heads, rope_base=10000.0, inplace=True)
    assert out_q.data_ptr() == dq.data_ptr() and out_k.data_ptr() == dk.data_ptr()
    assert torch.equal(dq, fresh_q) and torch.equal(dk, fresh_k)
    assert torch.equal(dv.cpu(), v)
    torch.testing.assert_close(dq.cpu().float(), expected_q.float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(dk.cpu().float(), expected_k.float(), rtol=2e-2, atol=2e-2)


def test_qk_norm_rope_skips_padded_rows(device):
    """With a row index only the valid tokens are read and written: NaNs at the padded positions change nothing, the
    valid rows equal the run over all rows bit for bit (positions included: the rotary angle follows the token's place
    in its sample, not its place in the index), padded rows come back zero (new tensors) or untouched (in place)."""
    batch, tokens, d_model, heads = 6, 40, 128, 4
    q, k, wq, wk = _draw(batch, tokens, d_model, torch.bfloat16, seed=3)
    lengths = torch.tensor([40, 1, 17, 0, 33, 8], dtype=torch.int32)
    valid = torch.arange(tokens)[None, :] < lengths[:, None]
    with torch.no_grad():
        full_q, full_k = qk_norm_rope(q.to(device), k.to(device), wq.to(device), wk.to(device), num_heads=heads,
                                      rope_base=100.0)
        index = valid_rows(lengths.to(device), tokens)
        qn = torch.where(valid[..., None], q, torch.full_like(q, float("nan"))).to(device)
        kn = torch.where(valid[..., None], k, torch.full_like(k, float("nan"))).to(device)
        got_q, got_k = qk_norm_rope(qn, kn, wq.to(device), wk.to(device), num_heads=heads, rope_base=100.0,
                                    token_rows=index)
        before = qn.clone()
        qk_norm_rope(qn, kn, wq.to(device), wk.to(device), num_heads=heads, rope_base=100.0, token_rows=index, inplace=True)
    mask = valid.to(device)
    assert torch.equal(got_q[mask], full_q[mask]) and torch.equal(got_k[mask], full_k[mask])
    assert torch.count_nonzero(got_q[~mask]) == 0 and torch.count_nonzero(got_k[~mask]) == 0
    assert torch.equal(qn[mask], full_q[mask])
    assert torch.isnan(qn[~mask]).all() and torch.isnan(before[~mask]).all()


def test_qk_norm_rope_argument_errors(device):
    q, k, wq, wk = _draw(2, 4, 64, torch.bfloat16, seed=1)
    q, k, wq, wk = q.to(device), k.to(device), wq.to(device), wk.to(device)
    with pytest.raises(ValueError, match="same shape"):
        qk_norm_rope(q, k[:, :3], wq, wk, num_heads=2)
    with pytest.raises(ValueError, match="divisible"):
        qk_norm_rope(q, k, wq, wk, num_heads=3)
    with pytest.raises(ValueError, match="both norm weights or neither"):
        qk_norm_rope(q, k, wq, None, num_heads=2)
    with pytest.raises(ValueError, match="norm weights, a rope_base, or both"):
        qk_norm_rope(q, k, None, None, num_heads=2)
    with pytest.raises(ValueError, match="1D and match"):
        qk_norm_rope(q, k, wq[:32], wk[:32], num_heads=2)
    with pytest.raises(RuntimeError, match="multiples of 8"):  # head_dim 4: a 16-byte vector would straddle heads
        qk_norm_rope(q, k, wq, wk, num_heads=16, rope_base=10000.0)
    with pytest.raises(RuntimeError, match="CUDA"):
        qk_norm_rope(q.cpu(), k.cpu(), wq.cpu(), wk.cpu(), num_heads=2)


@pytest.mark.parametrize("layer", ["symbiosis", "tokenformer", "tokenformer_no_rope"])
def test_attention_layers_with_normalised_queries_and_keys(device, layer):
    """``UnifiedSelfAttention`` (experiments/symbiosis/backbone.py:24-48) and ``BFTSAttention``
    (experiments/tokenformer/model.py:139-163) against the oracle's composition of the same steps."""
    batch, tokens, d_model, heads = 4, 48, 256, 8
    g = torch.Generator().manual_seed(21)
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)
    lengths = torch.tensor([48, 5, 31, 16], dtype=torch.int32)
    if layer == "symbiosis":
        module = UnifiedSelfAttention(d_model, heads, 0.0)
        base = None
    else:
        base = 10000.0 if layer == "tokenformer" else None
        module = BFTSAttention(d_model, heads, 0.0, use_rope=base is not None, rope_base=10000.0)
    with torch.no_grad():
        module.query_norm.weight.copy_(1.0 + 0.1 * torch.randn(d_model, generator=g))
        module.key_norm.weight.copy_(1.0 + 0.1 * torch.randn(d_model, generator=g))
        module.qkv.bias.copy_(0.05 * torch.randn(3 * d_model, generator=g))
    module = module.eval()
    bf = lambda t: t.detach().to(torch.bfloat16)
    q, k, v = F.linear(x, bf(module.qkv.weight), bf(module.qkv.bias)).chunk(3, dim=-1)
    q, k = oracle.qk_norm_rope(q, k, bf(module.query_norm.weight), bf(module.key_norm.weight), num_heads=heads,
                               eps=module.query_norm.eps, rope_base=base)
    attended = oracle.scaled_dot_product_attention(q, k, v, num_heads=heads, key_lengths=lengths, zero_padded_queries=True)
    expected = F.linear(attended, bf(module.out.weight), bf(module.out.bias))
    with torch.no_grad():
        got = module.to(device)(x.to(device), key_lengths=lengths.to(device), zero_padded_queries=True)
    torch.testing.assert_close(got.cpu().float(), expected.float(), rtol=2e-2, atol=2e-2)
    if base is not None:  # the rotation matters: without it the result is measurably different
        plain = UnifiedSelfAttention(d_model, heads, 0.0).eval()
        plain.load_state_dict(module.state_dict())
        with torch.no_grad():
            other = plain.to(device)(x.to(device), key_lengths=lengths.to(device), zero_padded_queries=True)
        assert (other.float() - got.float()).abs().max().item() > 5e-2


@pytest.mark.parametrize("d_model,heads", [(256, 8), (128, 4)])
@pytest.mark.parametrize("mode", ["norm", "rope", "norm+rope"])
@pytest.mark.parametrize("workgroups", [None, 3])
def test_qkv_projection_prepares_queries_and_keys_in_its_epilogue(device, test_hooks, d_model, heads, mode, workgroups):
    """The packed projection with the query / key preparation in its epilogue: q and k columns come out as
    rotate(projection * weight), the value columns as the plain projection, and the returned per-token factors are
    rsqrt(mean(projection^2) + eps); factor * columns equals the oracle's RMSNorm + rotary embedding. Run with one
    tile per workgroup and with a capped grid (several tiles and the chunk-split last round per workgroup)."""
    from taac_2026_amd.api import qkv_projection

    if workgroups is not None:
        test_hooks(max_workgroups=workgroups)
    batch, tokens = 5, 333
    g = torch.Generator().manual_seed(d_model + len(mode))
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)
    nw = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
    w = (torch.randn(3 * d_model, d_model, generator=g) * d_model ** -0.5).to(torch.bfloat16)
    b = (0.1 * torch.randn(3 * d_model, generator=g)).to(torch.bfloat16)
    wq = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
    wk = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
    weights = (wq, wk) if "norm" in mode else (None, None)
    base = 10000.0 if "rope" in mode else None
    projection = F.linear(oracle.rms_norm_fp32(x, nw).float(), w.float(), b.float()).to(torch.bfloat16)
    q, k, v = projection.chunk(3, dim=-1)
    # Expected queries and keys: the same formulas evaluated in fp32 from the bf16 inputs, without intermediate roundings.
    # The kernel folds the norm weight into the layer's weights and applies the per-token factor to its accumulators, so
    # its single 16-bit rounding sits elsewhere than that of a normalise-then-project evaluation: either is within the
    # tolerance of the unrounded value, but they may differ from each other by one bf16 step of the largest entries.
    exact = F.linear(oracle.rms_norm_fp32(x.float(), nw.float()), w.float(), b.float())
    expected_q, expected_k = oracle.qk_norm_rope(exact[..., :d_model], exact[..., d_model:2 * d_model],
                                                 *(None if t is None else t.float() for t in weights), num_heads=heads,
                                                 eps=1e-6, rope_base=base, fp32=True)
    with torch.no_grad():
        qkv, sq, sk, col = qkv_projection(x.to(device), w.to(device), b.to(device), num_heads=heads,
                                          norm_weight=nw.to(device),
                                          query_weight=None if weights[0] is None else wq.to(device),
                                          key_weight=None if weights[1] is None else wk.to(device), rope_base=base)
    got_q, got_k, got_v = qkv.cpu().chunk(3, dim=-1)
    torch.testing.assert_close(got_v.float(), v.float(), rtol=2e-2, atol=2e-2)
    if "norm" in mode:
        assert sq.shape == (batch, tokens) and sq.dtype == torch.float32
        # the statistic is taken from the rounded projection the kernel itself produced
        rstd = lambda t: torch.rsqrt(t.float().pow(2).mean(-1) + 1e-6)
        torch.testing.assert_close(sq.cpu(), rstd(q), rtol=5e-3, atol=0)
        torch.testing.assert_close(sk.cpu(), rstd(k), rtol=5e-3, atol=0)
        got_q = got_q.float() * sq.cpu()[..., None]
        got_k = got_k.float() * sk.cpu()[..., None]
        if base is None:
            # without a rotation the columns are the plain projection and both weights ride on the query as their
            # product: q * (wq * wk) and k give the same scores as (q * wq) and (k * wk)
            torch.testing.assert_close(col.cpu(), wq.float() * wk.float(), rtol=0, atol=0)
            torch.testing.assert_close(qkv.cpu()[..., :2 * d_model].float(), projection[..., :2 * d_model].float(),
                                       rtol=2e-2, atol=2e-2)
            got_q = got_q * col.cpu() / wk.float()
            got_k = got_k * wk.float()
        else:
            assert col is None
    else:
        assert sq is None and sk is None and col is None
    torch.testing.assert_close(got_q.float(), expected_q.float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(got_k.float(), expected_k.float(), rtol=2e-2, atol=2e-2)


def test_qkv_projection_skips_padded_rows(device):
    from taac_2026_amd.api import qkv_projection

    batch, tokens, d_model, heads = 4, 70, 256, 8
    g = torch.Generator().manual_seed(8)
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)
    w = (torch.randn(3 * d_model, d_model, generator=g) * d_model ** -0.5).to(torch.bfloat16)
    wq = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
    lengths = torch.tensor([70, 3, 0, 41], dtype=torch.int32)
    valid = torch.arange(tokens)[None, :] < lengths[:, None]
    with torch.no_grad():
        full, fq, fk, _ = qkv_projection(x.to(device), w.to(device), None, num_heads=heads, query_weight=wq.to(device),
                                      key_weight=wq.to(device), rope_base=500.0)
        xn = torch.where(valid[..., None], x, torch.full_like(x, float("nan"))).to(device)
        got, sq, sk, _ = qkv_projection(xn, w.to(device), None, num_heads=heads, query_weight=wq.to(device),
                                     key_weight=wq.to(device), rope_base=500.0,
                                     token_rows=valid_rows(lengths.to(device), tokens))
    mask = valid.to(device)
    assert torch.equal(got[mask], full[mask]) and torch.equal(sq[mask], fq[mask]) and torch.equal(sk[mask], fk[mask])
    assert torch.count_nonzero(got[~mask]) == 0 and torch.isfinite(sq).all() and torch.isfinite(sk).all()


def test_golden_vectors(device):
    """The committed pure-Python float64 evaluations (tests/golden/qk_rope_embedding_small.json) against the float32
    kernel; an odd head width (its last feature is not rotated) is reported by the host layer, not served."""
    import json
    from pathlib import Path

    golden = json.loads((Path(__file__).resolve().parent / "golden" / "qk_rope_embedding_small.json").read_text())
    served = 0
    for case in golden["qk"]:
        q, k = torch.tensor(case["query"]), torch.tensor(case["key"])
        weights = [None if case[name] is None else torch.tensor(case[name]).to(device) for name in ("query_weight", "key_weight")]
        head_dim = q.shape[-1] // case["num_heads"]
        call = lambda: qk_norm_rope(q.to(device), k.to(device), *weights, num_heads=case["num_heads"], eps=case["eps"],
                                    rope_base=case["rope_base"])
        if case["rope_base"] is not None and head_dim % 4 != 0:
            with pytest.raises((RuntimeError, ValueError), match="multiples of|must be even"):
                call()
            continue
        with torch.no_grad():
            got_q, got_k = call()
        torch.testing.assert_close(got_q.cpu().double(), torch.tensor(case["query_out"], dtype=torch.float64), rtol=2e-5, atol=2e-6)
        torch.testing.assert_close(got_k.cpu().double(), torch.tensor(case["key_out"], dtype=torch.float64), rtol=2e-5, atol=2e-6)
        served += 1
    assert served == 3


@pytest.mark.parametrize("mode", ["norm", "rope", "norm_rope"])
def test_qk_norm_rope_takes_a_gradient(device, mode):
    """Under autograd the preparation runs as differentiable steps (norm kernels with their backward, the rotation with
    the opposite angles as its backward): outputs equal to the one-pass route, gradients of query, key and the norm
    weights against float64 autograd of the oracle's expression at the reference's gradient tolerance."""
    batch, tokens, d_model, heads = 3, 50, 128, 4
    g = torch.Generator().manual_seed(21)
    q = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)
    k = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)
    wq = (1 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
    wk = (1 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
    gq = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)
    gk = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)
    with_norm, rope_base = mode != "rope", (None if mode == "norm" else 10000.0)
    dev = [t.to(device).requires_grad_(True) for t in (q, k, wq, wk)]
    out_q, out_k = qk_norm_rope(dev[0], dev[1], dev[2] if with_norm else None, dev[3] if with_norm else None,
                                num_heads=heads, rope_base=rope_base)
    torch.autograd.backward([out_q, out_k], [gq.to(device), gk.to(device)])
    with torch.no_grad():
        one_q, one_k = qk_norm_rope(dev[0].detach(), dev[1].detach(), dev[2].detach() if with_norm else None,
                                    dev[3].detach() if with_norm else None, num_heads=heads, rope_base=rope_base)
    torch.testing.assert_close(out_q.detach().float(), one_q.float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(out_k.detach().float(), one_k.float(), rtol=2e-2, atol=2e-2)
    ref = [t.double().requires_grad_(True) for t in (q, k, wq, wk)]
    want_q, want_k = oracle.qk_norm_rope(ref[0], ref[1], ref[2] if with_norm else None, ref[3] if with_norm else None,
                                         num_heads=heads, rope_base=rope_base)
    torch.autograd.backward([want_q, want_k], [gq.double(), gk.double()])
    for index, (got, expected) in enumerate(zip(dev, ref)):
        if index >= 2 and not with_norm:
            assert got.grad is None
            continue
        scale = expected.grad.abs().max().item()
        error = (got.grad.cpu().double() - expected.grad).abs().max().item()
        assert error <= 3e-2 * scale, (index, error, scale)
