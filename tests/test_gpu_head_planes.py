"""GPU tests of the per-head plane layout of q | k | v and of the attention output: the two entry points that write / read
it (``taac_norm_linear_heads_fwd``, ``taac_attn_out_ffn_heads_fwd``) against the row-major entry points, bit for bit,
the block built from them against the oracle, and the backbone's default route against its row-major route."""

from __future__ import annotations

import pytest
import torch

from oracle import reference as oracle
from taac_2026_amd import workloads
from taac_2026_amd.api import (
    PCVRBackbone,
    attention_out_ffn,
    attention_out_ffn_heads,
    flash_attention,
    norm_linear,
    norm_linear_heads,
    valid_rows,
)

pytestmark = pytest.mark.gpu


def _layer(out_features, in_features, g, scale):
    weight = (scale * torch.randn(out_features, in_features, generator=g)).to(torch.bfloat16)
    bias = (0.05 * torch.randn(out_features, generator=g)).to(torch.bfloat16)
    return weight, bias


def _planes_to_rows(planes):
    """[P, M, d] planes -> [M, P * d] rows."""
    return planes.permute(1, 0, 2).reshape(planes.shape[1], -1)


def _rows_to_planes(rows, head_dim):
    return rows.view(rows.shape[0], -1, head_dim).permute(1, 0, 2).contiguous()


@pytest.mark.parametrize("d_model,head_dim", [(256, 32), (256, 64), (128, 32), (128, 64)])
@pytest.mark.parametrize("sparse", [False, True])
def test_projection_into_planes_equals_the_row_major_projection(device, d_model, head_dim, sparse):
    g = torch.Generator().manual_seed(d_model + head_dim)
    batch, tokens = 5, 77                       # 385 rows: a ragged last tile
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    norm_weight = (1 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16).to(device)
    weight, bias = (t.to(device) for t in _layer(3 * d_model, d_model, g, d_model ** -0.5))
    lengths = torch.tensor([77, 1, 40, 0, 63], dtype=torch.int32, device=device)
    token_rows = valid_rows(lengths, tokens) if sparse else None
    for nw, b in ((norm_weight, bias), (None, None), (norm_weight, None)):
        rows = norm_linear(x, weight, b, norm_weight=nw, token_rows=token_rows)
        planes = norm_linear_heads(x, weight, b, head_dim=head_dim, norm_weight=nw, token_rows=token_rows)
        assert planes.shape == (3 * d_model // head_dim, batch * tokens, head_dim)
        assert torch.equal(_planes_to_rows(planes), rows.view(batch * tokens, -1))
    # a caller's buffer: rows the index leaves out keep what the buffer held
    if sparse:
        held = torch.full((3 * d_model // head_dim, batch * tokens, head_dim), 7.0, dtype=torch.bfloat16, device=device)
        norm_linear_heads(x, weight, bias, head_dim=head_dim, norm_weight=norm_weight, token_rows=token_rows, out=held)
        valid = (torch.arange(tokens, device=device)[None, :] < lengths[:, None]).reshape(-1)
        planes = norm_linear_heads(x, weight, bias, head_dim=head_dim, norm_weight=norm_weight, token_rows=token_rows)
        assert torch.equal(held[:, valid], planes[:, valid]) and (held[:, ~valid] == 7.0).all()
        assert not planes[:, ~valid].any()


@pytest.mark.parametrize("d_model,head_dim,hidden", [(256, 32, 1024), (256, 64, 512), (128, 32, 256), (128, 64, 96)])
@pytest.mark.parametrize("sparse", [False, True])
def test_block_tail_from_planes_equals_the_row_major_block_tail(device, d_model, head_dim, hidden, sparse):
    g = torch.Generator().manual_seed(3 * d_model + head_dim)
    batch, tokens = 4, 83
    attn = torch.randn(batch * tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    residual = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    norm_weight = (1 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16).to(device)
    w_out, b_out = (t.to(device) for t in _layer(d_model, d_model, g, d_model ** -0.5))
    w_up, b_up = (t.to(device) for t in _layer(2 * hidden, d_model, g, d_model ** -0.5))
    w_down, b_down = (t.to(device) for t in _layer(d_model, hidden, g, hidden ** -0.5))
    lengths = torch.tensor([83, 2, 0, 51], dtype=torch.int32, device=device)
    token_rows = valid_rows(lengths, tokens) if sparse else None
    for nw, biases in ((norm_weight, True), (None, False)):
        bo, bu, bd = (b_out, b_up, b_down) if biases else (None, None, None)
        expected = attention_out_ffn(attn.view(batch, tokens, d_model), w_out, bo, residual, w_up, bu, w_down, bd,
                                     norm_weight=nw, token_rows=token_rows)
        got = attention_out_ffn_heads(_rows_to_planes(attn, head_dim), w_out, bo, residual, w_up, bu, w_down, bd,
                                      norm_weight=nw, token_rows=token_rows)
        assert got.shape == residual.shape and torch.equal(got, expected)
    # in place on the residual, as the backbone runs it
    target = residual.clone()
    attention_out_ffn_heads(_rows_to_planes(attn, head_dim), w_out, b_out, target, w_up, b_up, w_down, b_down,
                            norm_weight=norm_weight, token_rows=token_rows, out=target)
    reference = attention_out_ffn(attn.view(batch, tokens, d_model), w_out, b_out, residual, w_up, b_up, w_down, b_down,
                                  norm_weight=norm_weight, token_rows=token_rows, out=residual.clone())
    assert torch.equal(target, reference)


@pytest.mark.parametrize("d_model,heads", [(256, 8), (128, 2)])
def test_one_block_in_planes_matches_the_oracle(device, d_model, heads):
    """Projection -> attention -> block tail with q | k | v and the attention output kept as planes, against the oracle's
    block on the same inputs (valid rows; padded rows pass through)."""
    inputs = workloads.backbone_inputs(batch=4, n_feature_tokens=8, n_sequence_tokens=150, d_model=d_model,
                                       num_heads=heads, d_ff=2 * d_model, n_blocks=1, min_sequence_len=5, seed=21)
    weights = {k: v.to(device) for k, v in inputs.blocks[0].items()}
    x = inputs.emb.to(device)
    batch, tokens, _ = x.shape
    head_dim = d_model // heads
    lengths = inputs.key_lengths.to(device)
    token_rows = valid_rows(lengths, tokens)
    planes = norm_linear_heads(x, weights["qkv.weight"], weights.get("qkv.bias"), head_dim=head_dim,
                               norm_weight=weights["attn_norm.weight"], token_rows=token_rows)
    q, k, v = (planes.view(3, heads, batch, tokens, head_dim)[i].transpose(0, 1) for i in range(3))
    attn = flash_attention(q, k, v, key_lengths=lengths, zero_padded_queries=True)   # keeps q's layout: planes again
    attn = attn.transpose(0, 1)
    assert attn.is_contiguous()
    out = attention_out_ffn_heads(attn.reshape(heads, batch * tokens, head_dim), weights["out.weight"],
                                  weights.get("out.bias"), x, weights["up.weight"], weights.get("up.bias"),
                                  weights["down.weight"], weights.get("down.bias"), norm_weight=weights["ffn_norm.weight"],
                                  token_rows=token_rows, out=x.clone())
    expected = oracle.block(inputs.emb.float(), inputs.key_lengths, {k: v.float() for k, v in inputs.blocks[0].items()},
                            num_heads=heads)
    valid = torch.arange(tokens)[None, :] < inputs.key_lengths[:, None]
    torch.testing.assert_close(out.cpu().float()[valid], expected[valid], rtol=2e-2, atol=2e-2)
    assert torch.equal(out.cpu()[~valid], inputs.emb[~valid])


@pytest.mark.parametrize("d_model,heads,d_ff", [(256, 8, 1024), (256, 4, 512), (128, 4, 256), (128, 2, 512)])
@pytest.mark.parametrize("dense_tokens", [False, True])
@pytest.mark.parametrize("qk_norm,rope_base", [(False, None), (True, None), (True, 10000.0), (False, 10000.0)])
def test_backbone_plane_route_equals_its_row_major_route(device, d_model, heads, d_ff, dense_tokens, qk_norm, rope_base):
    """Also with the query / key norms and the rotary embedding of the reference's attention layers, whose projection
    epilogue (statistic, weight, rotation) then stores into the planes."""
    inputs = workloads.backbone_inputs(batch=7, n_feature_tokens=16, n_sequence_tokens=240, d_model=d_model,
                                       num_heads=heads, d_ff=d_ff, n_blocks=3, min_sequence_len=3, seed=d_model + heads,
                                       qk_norm=qk_norm)
    g = torch.Generator().manual_seed(9)
    for weights in inputs.blocks:
        weights["qkv.bias"] = (0.05 * torch.randn(3 * d_model, generator=g)).to(torch.bfloat16)
        if qk_norm:
            weights["query_norm.weight"] = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
            weights["key_norm.weight"] = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
    model = PCVRBackbone(d_model=d_model, num_heads=heads, d_ff=d_ff, n_blocks=3, qk_norm=qk_norm, rope_base=rope_base)
    workloads.load_backbone_state(model, inputs)
    model = model.to(device=device, dtype=torch.bfloat16).eval()
    emb, lengths = inputs.emb.to(device), inputs.key_lengths.to(device)
    with torch.no_grad():
        p, hidden = model(emb, lengths, return_hidden=True, dense_tokens=dense_tokens)
        p_rows, hidden_rows = model(emb, lengths, return_hidden=True, dense_tokens=dense_tokens, row_major_qkv=True)
    assert torch.equal(p, p_rows)
    valid = torch.arange(emb.shape[1], device=device)[None, :] < lengths[:, None]
    assert torch.equal(hidden[valid], hidden_rows[valid])
    if not dense_tokens:
        assert torch.equal(hidden, hidden_rows)


@pytest.mark.parametrize("d_model,heads,d_ff", [(256, 8, 1024), (128, 2, 256), (128, 8, 256)])  # head widths 32, 64, 16 (rows)
@pytest.mark.parametrize("dense_tokens", [False, True])
def test_readout_riding_on_the_last_block_equals_the_readout_kernel(device, d_model, heads, d_ff, dense_tokens):
    """The last block's kernel leaves every token's dot product with the head weight behind and the readout adds those;
    the stand-alone readout kernel (``taac_masked_mean_head``: mean of the rows, then the dot product) on the returned
    hidden state gives the same probabilities up to fp32 summation order. Lengths 0 and T included."""
    from taac_2026_amd import _native

    inputs = workloads.backbone_inputs(batch=9, n_feature_tokens=8, n_sequence_tokens=192, d_model=d_model,
                                       num_heads=heads, d_ff=d_ff, n_blocks=2, min_sequence_len=1, seed=77)
    inputs.key_lengths[0] = 0
    inputs.key_lengths[1] = inputs.emb.shape[1]
    g = torch.Generator().manual_seed(4)
    inputs.head_weight.copy_((0.5 * torch.randn(inputs.head_weight.shape, generator=g)).to(torch.bfloat16))
    inputs.head_bias.fill_(0.25)
    model = PCVRBackbone(d_model=d_model, num_heads=heads, d_ff=d_ff, n_blocks=2)
    workloads.load_backbone_state(model, inputs)
    model = model.to(device=device, dtype=torch.bfloat16).eval()
    emb, lengths = inputs.emb.to(device), inputs.key_lengths.to(device)
    with torch.no_grad():
        p, hidden = model(emb, lengths, return_hidden=True, dense_tokens=dense_tokens)
        p_only = model(emb, lengths, dense_tokens=dense_tokens)
    assert torch.equal(p, p_only)
    batch, tokens, _ = emb.shape
    library = _native.load_library()
    expected = torch.empty(batch, dtype=torch.float32, device=device)
    w_head = inputs.head_weight.to(device).reshape(-1).contiguous()
    b_head = inputs.head_bias.to(device).reshape(-1).contiguous()
    _native.check(library.taac_masked_mean_head(hidden.contiguous().data_ptr(), lengths.data_ptr(), w_head.data_ptr(),
                                                b_head.data_ptr(), expected.data_ptr(), batch, tokens, d_model,
                                                _native.current_stream(device)), "masked_mean_head")
    torch.testing.assert_close(p, expected, rtol=0, atol=2e-6)
    assert abs(p[0].item() - torch.sigmoid(torch.tensor(0.25)).item()) < 1e-6    # no valid token: sigmoid(bias)
    want = oracle.backbone(inputs.emb[1:], inputs.key_lengths[1:], inputs.blocks, inputs.head_weight, inputs.head_bias,
                           num_heads=heads)
    torch.testing.assert_close(p.cpu()[1:], want, rtol=0, atol=2e-2)
