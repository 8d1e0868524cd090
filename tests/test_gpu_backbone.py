"""GPU parity: the 4-block backbone forward (one taac_backbone_fwd call) against the CPU oracle."""

from __future__ import annotations

import math

import pytest
import torch

from oracle import reference as oracle
from taac_2026_amd import workloads
from taac_2026_amd.api import PCVRBackbone, UnifiedInteractionBlock

pytestmark = pytest.mark.gpu


def _run(inputs, device, return_hidden=True, rope_base=None, **routes):
    model = PCVRBackbone(d_model=inputs.emb.shape[-1], num_heads=inputs.num_heads, d_ff=inputs.d_ff,
                         n_blocks=len(inputs.blocks), qk_norm="query_norm.weight" in inputs.blocks[0], rope_base=rope_base)
    workloads.load_backbone_state(model, inputs)
    model = model.to(device=device, dtype=torch.bfloat16).eval()
    with torch.no_grad():
        return model(inputs.emb.to(device), inputs.key_lengths.to(device), return_hidden=return_hidden, **routes)


@pytest.mark.parametrize("batch,n_feature,n_sequence", [(6, 32, 96), (3, 32, 480), (5, 8, 57)])
def test_backbone_matches_oracle(device, batch, n_feature, n_sequence):
    inputs = workloads.backbone_inputs(batch=batch, n_feature_tokens=n_feature, n_sequence_tokens=n_sequence,
                                       min_sequence_len=min(32, n_sequence), seed=batch)
    # The reference's formulas evaluated two ways on the same bf16 inputs and weights: in bf16 end to end (what its
    # torch backend does under autocast) and in fp32 (no intermediate rounding). Probabilities are held to 2e-2
    # against both. The final hidden state has passed through 4 x 7 bf16 rounding points at magnitudes up to ~4.5
    # (bf16 spacing 0.03), so no bf16 pipeline - the reference's own included - stays inside rtol = atol = 2e-2 on
    # every element; it is held to: at most 0.1 % of the elements outside rtol = atol = 2e-2 of the fp32 evaluation,
    # no element further than three bf16 spacings of the largest activation (or than the reference's bf16 evaluation
    # strays), and a mean error no larger than that of
    # the reference's bf16 evaluation.
    expected_p, expected_h = oracle.backbone(inputs.emb, inputs.key_lengths, inputs.blocks, inputs.head_weight,
                                             inputs.head_bias, num_heads=inputs.num_heads, return_hidden=True)
    blocks32 = [{k: v.float() for k, v in w.items()} for w in inputs.blocks]
    exact_p, exact_h = oracle.backbone(inputs.emb.float(), inputs.key_lengths, blocks32, inputs.head_weight.float(),
                                       inputs.head_bias.float(), num_heads=inputs.num_heads, return_hidden=True)
    p, hidden = _run(inputs, device)
    assert p.shape == (batch,) and p.dtype == torch.float32
    torch.testing.assert_close(p.cpu(), expected_p, rtol=0, atol=2e-2)
    torch.testing.assert_close(p.cpu(), exact_p, rtol=0, atol=2e-2)
    tokens = inputs.emb.shape[1]
    valid = torch.arange(tokens)[None, :] < inputs.key_lengths[:, None]
    exact = exact_h[valid]
    ours_err = (hidden.cpu().float()[valid] - exact).abs()
    bf16_err = (expected_h.float()[valid] - exact).abs()
    outside = (ours_err > 2e-2 + 2e-2 * exact.abs()).float().mean().item()
    spacing = 2.0 ** (math.floor(math.log2(exact.abs().max().item())) - 7)
    assert outside <= 1e-3, outside
    assert ours_err.max().item() <= max(3 * spacing, bf16_err.max().item()), (ours_err.max().item(), spacing)
    assert ours_err.mean().item() <= bf16_err.mean().item(), (ours_err.mean().item(), bf16_err.mean().item())
    assert torch.isfinite(hidden).all()


@pytest.mark.parametrize("qk_norm,rope_base", [(True, None), (True, 10000.0), (False, 10000.0)])
@pytest.mark.parametrize("d_model,heads,d_ff", [(256, 8, 512), (128, 4, 256), (64, 2, 96)])
def test_backbone_with_normalised_and_rotated_queries_and_keys(device, qk_norm, rope_base, d_model, heads, d_ff):
    """The block as the reference's layers run it: RMSNorm(d_model) of the query and the key
    (experiments/symbiosis/backbone.py:33-36) and TokenFormer's rotary embedding (experiments/tokenformer/model.py:
    153-154). Widths 128 / 256 take the path without a pass over q and k (projection epilogue + attention row
    factors), width 64 the in-place pass; with and without the valid-row index."""
    inputs = workloads.backbone_inputs(batch=5, n_feature_tokens=8, n_sequence_tokens=120, d_model=d_model,
                                       num_heads=heads, d_ff=d_ff, n_blocks=2, min_sequence_len=9, seed=11,
                                       qk_norm=qk_norm)
    g = torch.Generator().manual_seed(5)
    for weights in inputs.blocks:
        weights["qkv.bias"] = (0.05 * torch.randn(3 * d_model, generator=g)).to(torch.bfloat16)
        if qk_norm:
            weights["query_norm.weight"] = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
            weights["key_norm.weight"] = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
    expected_p, expected_h = oracle.backbone(inputs.emb, inputs.key_lengths, inputs.blocks, inputs.head_weight,
                                             inputs.head_bias, num_heads=heads, return_hidden=True, rope_base=rope_base)
    blocks32 = [{k: v.float() for k, v in w.items()} for w in inputs.blocks]
    exact_p, exact_h = oracle.backbone(inputs.emb.float(), inputs.key_lengths, blocks32, inputs.head_weight.float(),
                                       inputs.head_bias.float(), num_heads=heads, return_hidden=True, rope_base=rope_base)
    valid = torch.arange(inputs.emb.shape[1])[None, :] < inputs.key_lengths[:, None]
    results = [_run(inputs, device, rope_base=rope_base), _run(inputs, device, rope_base=rope_base, dense_tokens=True)]
    for p, hidden in results:
        torch.testing.assert_close(p.cpu(), expected_p, rtol=0, atol=2e-2)
        torch.testing.assert_close(p.cpu(), exact_p, rtol=0, atol=2e-2)
        ours_err = (hidden.cpu().float()[valid] - exact_h[valid]).abs()
        bf16_err = (expected_h.float()[valid] - exact_h[valid]).abs()
        assert (ours_err > 2e-2 + 2e-2 * exact_h[valid].abs()).float().mean().item() <= 1e-3
        assert ours_err.mean().item() <= 1.25 * bf16_err.mean().item() + 1e-4
    if d_model != 64:
        assert torch.equal(results[0][1][valid.to(device)], results[1][1][valid.to(device)])
    # the preparation is not a no-op: the plain recipe gives measurably different hidden states
    plain = [{k: v for k, v in w.items() if not k.startswith(("query_norm", "key_norm"))} for w in inputs.blocks]
    _, plain_h = oracle.backbone(inputs.emb, inputs.key_lengths, plain, inputs.head_weight, inputs.head_bias,
                                 num_heads=heads, return_hidden=True)
    assert (plain_h.float()[valid] - expected_h.float()[valid]).abs().max().item() > 5e-2


def test_backbone_skips_padded_positions(device):
    """The fused forward walks the valid tokens only: garbage (NaN) at the padded positions of the embeddings changes
    nothing, the valid rows of the hidden state are bit-identical to the run over all B*T positions
    (``dense_tokens=True``) and to the route with the out projection and the feed-forward half as two kernels, and the
    padded rows of the returned hidden state are zeros."""
    inputs = workloads.backbone_inputs(batch=7, n_feature_tokens=32, n_sequence_tokens=224, min_sequence_len=16, seed=3)
    tokens = inputs.emb.shape[1]
    valid = torch.arange(tokens)[None, :] < inputs.key_lengths[:, None]
    p_ref, h_ref = _run(inputs, device)
    poisoned = workloads.BackboneInputs(inputs.emb.clone(), inputs.key_lengths, inputs.blocks, inputs.head_weight,
                                        inputs.head_bias, inputs.num_heads, inputs.d_ff)
    poisoned.emb[~valid] = float("nan")
    p_poisoned, h_poisoned = _run(poisoned, device)
    assert torch.equal(p_poisoned, p_ref) and torch.equal(h_poisoned, h_ref)
    assert (h_ref.cpu()[~valid] == 0).all()
    p_dense, h_dense = _run(inputs, device, dense_tokens=True)
    assert torch.equal(p_dense, p_ref)
    assert torch.equal(h_dense.cpu()[valid], h_ref.cpu()[valid])
    # two kernels round the feed-forward update before the residual add, one kernel rounds their sum once
    p_split, h_split = _run(inputs, device, split_out_ffn=True)
    torch.testing.assert_close(p_split, p_ref, rtol=0, atol=2e-3)
    # (differences of one bf16 step per block, carried through four blocks)
    torch.testing.assert_close(h_split.cpu().float()[valid], h_ref.cpu().float()[valid], rtol=2 ** -5, atol=2 ** -4)


def test_backbone_config4_full_size(device):
    """Config 4 at full size (B=1024, T=512): 64 samples spread over the batch against the oracle; all outputs finite;
    batch rows independent (a sample gives the same probability alone and inside the batch)."""
    inputs = workloads.backbone_inputs()
    p, hidden = _run(inputs, device)
    assert torch.isfinite(p).all() and torch.isfinite(hidden).all()
    assert ((p > 0) & (p < 1)).all()
    pick = torch.unique(torch.linspace(0, 1023, 64).round().long())
    sub = workloads.BackboneInputs(inputs.emb[pick], inputs.key_lengths[pick], inputs.blocks, inputs.head_weight,
                                   inputs.head_bias, inputs.num_heads, inputs.d_ff)
    expected = oracle.backbone(sub.emb, sub.key_lengths, sub.blocks, sub.head_weight, sub.head_bias,
                               num_heads=sub.num_heads)
    torch.testing.assert_close(p.cpu()[pick], expected, rtol=0, atol=2e-2)
    p_sub = _run(sub, device, return_hidden=False)
    torch.testing.assert_close(p_sub.cpu(), p.cpu()[pick], rtol=0, atol=1e-6)


def test_interaction_block_module(device):
    """UnifiedInteractionBlock (QK-norm, padding-masked residual updates) against the same recipe on the CPU."""
    torch.manual_seed(1)
    d_model, heads, tokens, batch = 128, 4, 40, 3
    block = UnifiedInteractionBlock(d_model, heads, 4, 0.0).to(torch.bfloat16).eval()
    x = (0.5 * torch.randn(batch, tokens, d_model)).to(torch.bfloat16)
    lengths = torch.tensor([40, 17, 1])
    padding = oracle.make_padding_mask(lengths, tokens)
    mask = (~padding)[:, None, None, :].expand(batch, heads, tokens, tokens)
    sd = {k: v.detach() for k, v in block.state_dict().items()}

    import torch.nn.functional as F
    h = oracle.rms_norm(x, sd["attn_norm.weight"])
    q, k, v = F.linear(h, sd["attention.qkv.weight"], sd["attention.qkv.bias"]).chunk(3, -1)
    q = oracle.rms_norm(q, sd["attention.query_norm.weight"])
    k = oracle.rms_norm(k, sd["attention.key_norm.weight"])
    a = oracle.scaled_dot_product_attention(q, k, v, num_heads=heads, key_lengths=lengths)
    keep = (~padding).unsqueeze(-1).to(x.dtype)
    attn_tokens = x + F.linear(a, sd["attention.out.weight"], sd["attention.out.bias"]) * keep
    ffn = oracle.swiglu_ffn(oracle.rms_norm(attn_tokens, sd["ffn_norm.weight"]), sd["ffn.up.weight"], sd["ffn.up.bias"],
                            sd["ffn.down.weight"], sd["ffn.down.bias"])
    expected = attn_tokens + ffn * keep

    block = block.to(device)
    with torch.no_grad():
        got, got_attn = block(x.to(device), padding.to(device), mask.to(device))
    torch.testing.assert_close(got_attn.cpu().float(), attn_tokens.float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(got.cpu().float(), expected.float(), rtol=2e-2, atol=2e-2)


def _symbiosis_block_case(d_model, heads, tokens, batch, seed):
    from taac_2026_amd.api import MetadataAttentionMask

    g = torch.Generator().manual_seed(seed)
    block = UnifiedInteractionBlock(d_model, heads, 4, 0.0).to(torch.bfloat16).eval()
    with torch.no_grad():
        for name, parameter in block.named_parameters():
            if name.endswith("norm.weight"):
                parameter.add_((0.1 * torch.randn(parameter.shape, generator=g)).to(parameter.dtype))
            elif name.endswith("bias"):
                parameter.add_((0.05 * torch.randn(parameter.shape, generator=g)).to(parameter.dtype))
    x = (0.5 * torch.randn(batch, tokens, d_model, generator=g)).to(torch.bfloat16)
    padding = torch.rand(batch, tokens, generator=g) < 0.35   # padding anywhere, not a prefix
    padding[0] = False
    padding[1, 1:] = True                                      # a single valid token
    padding[:, 0] = False                                      # every sample keeps its first token
    roles = torch.randint(0, 8, (tokens,), generator=g)
    state = {k.replace("attention.", "").replace("ffn.", ""): v.detach() for k, v in block.state_dict().items()}
    return block, x, padding, roles, state, MetadataAttentionMask(enabled=True)


@pytest.mark.parametrize("d_model,heads,tokens,batch", [(128, 4, 70, 5), (256, 8, 150, 4)])
def test_interaction_block_fused_routes_under_role_masks_and_scattered_padding(device, d_model, heads, tokens, batch):
    """The reference block as the model runs it: role-based attention mask, padding anywhere in the sequence, updates
    masked at padded rows. Both fused routes against the oracle's statement of the block; padded rows pass through bit
    for bit and are never read (NaN there changes nothing). With the model's own mask object the attention runs over
    every sample's valid tokens moved to the front; a dense mask (or token_layout="positions") keeps the positions."""
    block, x, padding, roles, state, mask_module = _symbiosis_block_case(d_model, heads, tokens, batch, seed=d_model + tokens)
    dense_mask = oracle.metadata_attention_mask(padding, roles)
    want, want_attn = oracle.interaction_block(x.float(), padding, dense_mask, {k: v.float() for k, v in state.items()},
                                               num_heads=heads)
    valid = ~padding
    block = block.to(device)
    with torch.no_grad():
        mask = mask_module(padding.to(device), roles.to(device))
        two, two_attn = block(x.to(device), padding.to(device), mask)
        one, none = block(x.to(device), padding.to(device), mask, return_attention_tokens=False)
        from_dense, _ = block(x.to(device), padding.to(device), dense_mask.to(device))
        block.token_layout = "positions"
        by_position, by_position_attn = block(x.to(device), padding.to(device), mask)
        block.token_layout = "front"
        poisoned = x.clone()
        poisoned[padding] = float("nan")
        stream = poisoned.to(device)
        in_place, _ = block(stream, padding.to(device), mask, return_attention_tokens=False, inplace=True)
    assert none is None and in_place.data_ptr() == stream.data_ptr()
    torch.testing.assert_close(two_attn.cpu().float()[valid], want_attn[valid], rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(two.cpu().float()[valid], want[valid], rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(one.cpu().float()[valid], want[valid], rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(one.cpu().float(), two.cpu().float(), rtol=2 ** -6, atol=2 ** -6)
    assert torch.equal(from_dense.cpu(), by_position.cpu())
    torch.testing.assert_close(by_position_attn.cpu().float()[valid], want_attn[valid], rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(by_position.cpu().float(), two.cpu().float(), rtol=2 ** -6, atol=2 ** -6)
    for result in (two, one, two_attn):
        assert torch.equal(result.cpu()[padding], x[padding])          # x + update * 0
    assert torch.equal(in_place.cpu()[valid], one.cpu()[valid])
    assert torch.isnan(in_place.cpu()[padding].float()).all()


def test_interaction_block_projects_padded_tokens_when_the_mask_does_not_hide_them(device):
    """Without a mask (or under a dense mask that does not exclude the padded keys) the reference block attends to the
    projections of the padded tokens as well (experiments/symbiosis/backbone.py:58-63): the fused route must then
    project every row instead of reading rows it never wrote. Checked against the oracle's statement of the block, with
    the allocator's memory poisoned beforehand so that an unwritten row cannot pass by luck."""
    block, x, padding, roles, state, _ = _symbiosis_block_case(128, 4, 70, 5, seed=33)
    state32 = {k: v.float() for k, v in state.items()}
    batch, tokens, _ = x.shape
    structure = torch.rand(tokens, tokens, generator=torch.Generator().manual_seed(1)) < 0.6
    structure |= torch.eye(tokens, dtype=torch.bool)           # every query sees itself: no empty rows
    structure = structure[None, None].expand(batch, 1, tokens, tokens)   # shared by the batch, padded keys visible
    valid = ~padding
    block = block.to(device)
    for mask in (None, structure):
        want, want_attn = oracle.interaction_block(x.float(), padding, mask, state32, num_heads=4)
        # fill the caching allocator's free blocks of the size the projection will ask for with NaN
        poison = torch.full((batch * tokens, 3 * 128), float("nan"), dtype=torch.bfloat16, device=device)
        del poison
        with torch.no_grad():
            got, got_attn = block(x.to(device), padding.to(device), None if mask is None else mask.to(device))
            one, _ = block(x.to(device), padding.to(device), None if mask is None else mask.to(device),
                           return_attention_tokens=False)
        assert torch.isfinite(got.float()).all()
        torch.testing.assert_close(got_attn.cpu().float()[valid], want_attn[valid], rtol=2e-2, atol=2e-2)
        torch.testing.assert_close(got.cpu().float()[valid], want[valid], rtol=2e-2, atol=2e-2)
        torch.testing.assert_close(one.cpu().float()[valid], want[valid], rtol=2e-2, atol=2e-2)
        assert torch.equal(got.cpu()[padding], x[padding])
    # the padded tokens matter in these cases: hiding them changes the result
    hidden_keys, _ = oracle.interaction_block(x.float(), padding, valid[:, None, None, :].expand(batch, 1, tokens, tokens),
                                              state32, num_heads=4)
    no_mask, _ = oracle.interaction_block(x.float(), padding, None, state32, num_heads=4)
    assert (hidden_keys[valid] - no_mask[valid]).abs().max().item() > 5e-2


def test_one_block_at_the_headline_widths_holds_elementwise_tolerance(device):
    """A single block at the headline widths (d_model 256, 8 heads, d_ff 1024, 512 tokens, key-length route through the
    backbone entry point): every valid element of the hidden state within rtol = atol = 2e-2 of the fp32 evaluation of
    the reference's formulas. (The looser statistical bound of the 4-block tests is accumulation over 28 rounding
    points, not a property of a block.)"""
    inputs = workloads.backbone_inputs(batch=6, n_blocks=1, seed=11)
    assert inputs.emb.shape[1:] == (512, 256) and inputs.d_ff == 1024 and inputs.num_heads == 8
    blocks32 = [{k: v.float() for k, v in w.items()} for w in inputs.blocks]
    exact_p, exact_h = oracle.backbone(inputs.emb.float(), inputs.key_lengths, blocks32, inputs.head_weight.float(),
                                       inputs.head_bias.float(), num_heads=inputs.num_heads, return_hidden=True)
    valid = torch.arange(512)[None, :] < inputs.key_lengths[:, None]
    for routes in ({}, {"dense_tokens": True}, {"split_out_ffn": True}):
        p, hidden = _run(inputs, device, **routes)
        torch.testing.assert_close(hidden.cpu().float()[valid], exact_h[valid], rtol=2e-2, atol=2e-2)
        torch.testing.assert_close(p.cpu(), exact_p, rtol=0, atol=2e-2)


def test_interaction_block_routes_agree(device):
    """fp32 tokens take the module-by-module route (norms, attention layer and feed-forward as separate calls with the
    padding multiply in torch), bf16 tokens the fused one; both state the same block."""
    block, x, padding, roles, _, mask_module = _symbiosis_block_case(128, 4, 48, 3, seed=9)
    block = block.to(device)
    with torch.no_grad():
        mask = mask_module(padding.to(device), roles.to(device))
        fused, fused_attn = block(x.to(device), padding.to(device), mask)
        plain, plain_attn = block(x.to(device).float(), padding.to(device), mask)
    valid = ~padding
    torch.testing.assert_close(plain_attn.cpu()[valid], fused_attn.cpu().float()[valid], rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(plain.cpu()[valid], fused.cpu().float()[valid], rtol=2e-2, atol=2e-2)


def test_block_stack_shares_the_indices_of_its_mask(device):
    """run_interaction_blocks = the blocks called one after the other on fresh tensors, bit for bit; the indices and the
    gathered mask are built once (by the first block) and rebuilt when the padding mask is written to."""
    from taac_2026_amd.api import run_interaction_blocks

    block, x, padding, roles, _, mask_module = _symbiosis_block_case(128, 4, 70, 5, seed=21)
    other, *_ = _symbiosis_block_case(128, 4, 70, 5, seed=22)
    blocks = [block.to(device), other.to(device), block]
    dev_x, dev_pad = x.to(device), padding.to(device)
    with torch.no_grad():
        mask = mask_module(dev_pad, roles.to(device))
        expected = dev_x
        for module in blocks:
            expected, _ = module(expected, dev_pad, mask_module(dev_pad, roles.to(device)), return_attention_tokens=False)
        before = dev_x.clone()
        got = run_interaction_blocks(blocks, dev_x, dev_pad, mask)
        assert torch.equal(dev_x, before) and got.data_ptr() != dev_x.data_ptr()
        assert torch.equal(got, expected)
        entry = mask.cache["front"]
        assert run_interaction_blocks(blocks, dev_x, dev_pad, mask) is not None and mask.cache["front"] is entry
        dev_pad[3, 5] = ~dev_pad[3, 5]     # an in-place write: the cached indices no longer describe the mask
        run_interaction_blocks(blocks[:1], dev_x, dev_pad, mask)
        assert mask.cache["front"] is not entry


def test_valid_rows_from_a_padding_mask(device):
    from taac_2026_amd.api import valid_rows

    g = torch.Generator().manual_seed(2)
    for batch, tokens in ((7, 100), (3, 32), (5, 513), (1, 1)):
        padding = torch.rand(batch, tokens, generator=g) < 0.4
        if batch > 1:
            padding[1] = True
        rows, count = valid_rows(None, tokens, padding_mask=padding.to(device))
        expected = (~padding).flatten().nonzero().flatten()
        assert int(count.item()) == expected.numel()
        assert torch.equal(rows[:expected.numel()].cpu().long(), expected)
        offsets = rows[batch * tokens:batch * tokens + batch + 1].cpu().long()
        assert torch.equal(offsets, torch.cat([torch.zeros(1, dtype=torch.long), (~padding).sum(1).cumsum(0)]))
    lengths = torch.tensor([5, 0, 9], dtype=torch.int32)
    by_len = valid_rows(lengths.to(device), 9)
    by_mask = valid_rows(None, 9, padding_mask=(torch.arange(9)[None, :] >= lengths[:, None]).to(device))
    assert int(by_len[1].item()) == int(by_mask[1].item()) == 14 and torch.equal(by_len[0][:14], by_mask[0][:14])
    with pytest.raises(ValueError, match="key_lengths or padding_mask"):
        valid_rows(None, 9)
