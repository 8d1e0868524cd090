"""CPU tests of the host side: argument validation, error taxonomy, mask planning, module surface. No kernel runs."""

from __future__ import annotations

import json
from pathlib import Path

import pytest
import torch

from taac_2026_amd import accelerators, api
from taac_2026_amd.accelerators import attention as attention_ops
from taac_2026_amd.accelerators.tensor_validation import require_cuda_tensors, require_same_dtype
from taac_2026_amd.modeling import normalization as norm_modeling
from taac_2026_amd.modeling import sequence as sequence_modeling

MASKS = json.loads((Path(__file__).resolve().parent / "golden" / "mask_vectors.json").read_text())


def test_validation_helpers_error_taxonomy():
    with pytest.raises(RuntimeError, match="sample_op requires CUDA tensors"):
        require_cuda_tensors("sample_op", torch.empty(1))
    with pytest.raises(ValueError, match="sample_op requires tensors to share the same dtype"):
        require_same_dtype("sample_op", torch.empty(1, dtype=torch.float32), torch.empty(1, dtype=torch.float16))
    assert require_cuda_tensors("sample_op", None) is None


def test_rms_norm_argument_errors():
    x = torch.randn(4, 8)
    with pytest.raises(ValueError, match="at least 2 dimensions"):
        api.rms_norm(torch.randn(8), torch.ones(8))
    with pytest.raises(ValueError, match="weight must be a 1D tensor"):
        api.rms_norm(x, torch.ones(1, 8))
    with pytest.raises(ValueError, match="last dimension 8 does not match weight size 4"):
        api.rms_norm(x, torch.ones(4))
    with pytest.raises(ValueError, match="unsupported rms_norm backend: nope"):
        api.rms_norm(x, torch.ones(8), backend="nope")
    # there is no CPU path: a CPU tensor is refused, never silently computed elsewhere
    for backend in ("hip", "torch", "triton", "tilelang"):
        with pytest.raises(RuntimeError, match="requires CUDA tensors"):
            api.rms_norm(x, torch.ones(8), backend=backend)


def test_layer_norm_argument_errors():
    x = torch.randn(4, 8)
    with pytest.raises(ValueError, match="bias must be a 1D tensor"):
        api.layer_norm(x, torch.ones(8), torch.ones(1, 8))
    with pytest.raises(ValueError, match="does not match bias shape"):
        api.layer_norm(x, torch.ones(8), torch.ones(4))
    with pytest.raises(ValueError, match="unsupported layer_norm backend"):
        api.layer_norm(x, torch.ones(8), torch.ones(8), backend="tilelang")
    with pytest.raises(RuntimeError, match="requires CUDA tensors"):
        api.layer_norm(x, torch.ones(8), torch.ones(8))


def test_flash_attention_argument_errors():
    q = torch.randn(2, 3, 5, 8)
    with pytest.raises(ValueError, match=r"shape \(batch, heads, seq_len, head_dim\)"):
        api.flash_attention(q[0], q[0], q[0])
    with pytest.raises(ValueError, match="matching batch dimensions"):
        api.flash_attention(q, q[:1], q)
    with pytest.raises(ValueError, match="matching head counts"):
        api.flash_attention(q, q[:, :2], q[:, :2])
    with pytest.raises(ValueError, match="matching key and value sequence lengths"):
        api.flash_attention(q, q, q[:, :, :4])
    with pytest.raises(ValueError, match="matching head dimensions"):
        api.flash_attention(q, q[..., :4], q[..., :4])
    with pytest.raises(ValueError, match="share the same dtype"):
        api.flash_attention(q, q.half(), q)
    with pytest.raises(ValueError, match="unsupported flash attention backend"):
        api.flash_attention(q, q, q, backend="triton")
    with pytest.raises(RuntimeError, match=r"dropout_p to be in \[0, 1\)"):
        api.flash_attention(q, q, q, dropout_p=1.0, training=True)
    with pytest.raises(RuntimeError, match="only supports dropout during training"):
        api.flash_attention(q, q, q, dropout_p=0.1, training=False)
    with pytest.raises(RuntimeError, match="requires CUDA tensors"):
        api.flash_attention(q, q, q)


def test_mask_planner_known_answers():
    case = MASKS["plan_prefix_key_mask"]
    q, k = torch.randn(*case["q_shape"]), torch.randn(*case["k_shape"])
    key_valid = torch.tensor(case["key_valid"])
    mask = key_valid[:, None, None, :].expand(2, 3, 4, 6)
    for form in (mask, key_valid, key_valid[:, None, None, :]):
        plan = attention_ops.plan_flash_attention_mask(q, k, form, is_causal=False)
        assert torch.equal(plan.key_lengths, torch.tensor(case["expected_key_lengths"], dtype=torch.int32))
        assert plan.query_self_mask is None and plan.is_causal is False
    assert accelerators._plan_tilelang_flash_attention_mask is attention_ops.plan_flash_attention_mask

    case = MASKS["plan_causal_valid_mask"]
    q, k = torch.randn(*case["q_shape"]), torch.randn(*case["k_shape"])
    padding = torch.tensor(case["padding_mask"])
    plan = attention_ops.plan_flash_attention_mask(q, k, api.causal_valid_attention_mask(padding, 3), is_causal=False)
    assert torch.equal(plan.key_lengths, torch.tensor(case["expected_key_lengths"], dtype=torch.int32))
    assert plan.query_self_mask.tolist() == case["expected_query_self_mask"]
    assert plan.is_causal is True

    plan = attention_ops.plan_flash_attention_mask(q, k, None, is_causal=True)
    assert plan.key_lengths.tolist() == [5, 5] and plan.key_lengths.dtype == torch.int32 and plan.is_causal is True


def test_mask_planner_rejections():
    case = MASKS["plan_rejects_non_prefix"]
    q, k = torch.randn(*case["q_shape"]), torch.randn(*case["k_shape"])
    mask = torch.tensor(case["key_row"])[None, None, None, :].expand(2, 3, 5, 5)
    with pytest.raises(RuntimeError, match=case["error_fragment"]):
        attention_ops.plan_flash_attention_mask(q, k, mask, is_causal=False)
    with pytest.raises(RuntimeError, match="structured bool attention masks"):
        attention_ops.plan_flash_attention_mask(q, k, torch.zeros(2, 3, 5, 5), is_causal=False)
    with pytest.raises(RuntimeError, match="4D bool masks matching"):
        attention_ops.plan_flash_attention_mask(q, k, torch.ones(2, 1, 5, 5, dtype=torch.bool), is_causal=False)
    per_head = torch.ones(2, 3, 5, 5, dtype=torch.bool).clone()
    per_head[:, 1, :, 4] = False
    with pytest.raises(RuntimeError, match="shared across heads"):
        attention_ops.plan_flash_attention_mask(q, k, per_head, is_causal=False)
    arbitrary = torch.ones(2, 3, 5, 5, dtype=torch.bool).clone()
    arbitrary[:, :, 2, 1] = False
    with pytest.raises(RuntimeError, match="prefix key masks or causal_valid_attention_mask-style"):
        attention_ops.plan_flash_attention_mask(q, k, arbitrary, is_causal=False)
    k7 = torch.randn(2, 3, 7, 8)
    ragged = torch.ones(2, 3, 5, 7, dtype=torch.bool).clone()
    ragged[:, :, 0, 6] = False
    with pytest.raises(RuntimeError, match="query and key lengths match"):
        attention_ops.plan_flash_attention_mask(q, k7, ragged, is_causal=False)


def test_sequence_helpers_known_answers():
    case = MASKS["make_padding_mask"]
    assert api.make_padding_mask(torch.tensor(case["lengths"]), case["max_len"]).tolist() == case["expected"]
    case = MASKS["safe_key_padding_mask"]
    assert api.safe_key_padding_mask(torch.tensor(case["mask"])).tolist() == case["expected"]
    assert api.safe_key_padding_mask(torch.zeros(0, 3, dtype=torch.bool)).shape == (0, 3)
    tokens = torch.arange(24, dtype=torch.float32).view(2, 3, 4)
    padding = torch.tensor([[False, True, True], [True, True, True]])
    pooled = api.masked_mean(tokens, padding)
    assert pooled[0].tolist() == tokens[0, 0].tolist() and pooled[1].tolist() == [0.0] * 4
    assert api.masked_mean(tokens[:, :0], None).shape == (2, 4)


def test_runtime_configuration_and_modules():
    with pytest.raises(ValueError, match="unsupported rms_norm backend: nope"):
        api.configure_rms_norm_runtime(backend="nope", block_rows=1)
    with pytest.raises(ValueError, match="rms_norm block_rows must be positive"):
        api.configure_rms_norm_runtime(backend="torch", block_rows=0)
    api.configure_rms_norm_runtime(backend="triton", block_rows=4)
    norm = api.RMSNorm(6)
    api.configure_rms_norm_runtime(backend="hip", block_rows=1)
    assert (norm.backend, norm.block_rows) == ("triton", 4)  # captured at construction
    assert norm_modeling.rms_norm_runtime_state() == ("hip", 1)
    assert norm.weight.tolist() == [1.0] * 6
    ln = api.LayerNorm(6)
    assert ln.weight.tolist() == [1.0] * 6 and ln.bias.tolist() == [0.0] * 6 and ln.eps == 1e-5
    with pytest.raises(ValueError, match="unsupported layer_norm backend"):
        api.LayerNorm(6, backend="tilelang")
    with pytest.raises(ValueError, match="unsupported flash attention backend"):
        api.configure_flash_attention_runtime(backend="nope")
    api.configure_flash_attention_runtime(backend="tilelang")
    assert sequence_modeling.flash_attention_runtime_state() == "tilelang"
    api.configure_flash_attention_runtime(backend="hip")


def test_block_modules_keep_reference_parameter_names():
    block = api.UnifiedInteractionBlock(32, 4, 4, 0.0)
    names = set(dict(block.named_parameters()))
    assert {"attn_norm.weight", "attention.qkv.weight", "attention.qkv.bias", "attention.query_norm.weight",
            "attention.key_norm.weight", "attention.out.weight", "ffn_norm.weight", "ffn.up.weight", "ffn.up.bias",
            "ffn.down.weight", "ffn.down.bias"} <= names
    assert block.ffn.up.weight.shape == (256, 32) and block.ffn.down.weight.shape == (32, 128)
    model = api.PCVRBackbone(d_model=32, num_heads=4, d_ff=64, n_blocks=2)
    assert float(model.blocks[0].qkv.bias.abs().sum()) == 0.0
    with pytest.raises(RuntimeError, match="requires CUDA tensors"):
        model(torch.zeros(1, 4, 32, dtype=torch.bfloat16), torch.tensor([4], dtype=torch.int32))
    with pytest.raises(ValueError, match="divisible"):
        api.PCVRBackbone(d_model=30, num_heads=4)


def test_dense_layer_argument_errors():
    x = torch.zeros(4, 8, dtype=torch.bfloat16)
    w = torch.zeros(16, 8, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="requires CUDA tensors"):
        api.linear(x, w)
    with pytest.raises(RuntimeError, match="requires CUDA tensors"):
        api.swiglu_linear(x, w)
    with pytest.raises(RuntimeError, match="requires CUDA tensors"):
        api.amax(x)


def test_structural_masks_match_the_per_element_rules():
    """The (T, T) structural parts of the two model-level masks (vectorised torch expressions) against the oracle's
    per-element restatement, for every layer, both sequence modes and ragged padding."""
    from oracle import reference as oracle
    from taac_2026_amd.modeling.masks import bfts_structural_mask, metadata_structural_mask
    from taac_2026_amd.modeling.sequence import safe_key_padding_mask

    g = torch.Generator().manual_seed(0)
    tokens, layers = 37, 5
    roles = torch.tensor([0] * 3 + [4] + [1] * 24 + [4] + [2] * 4 + [5] * 3 + [3])
    padding = torch.rand(3, tokens, generator=g) < 0.3
    padding[2] = True
    eye = torch.eye(tokens, dtype=torch.bool)
    for layer in range(layers):
        for causal in (True, False):
            structural = bfts_structural_mask(roles, layer, layers, seq_causal=causal, seq_keep_per_domain=10)
            dense = structural[None] & ~safe_key_padding_mask(padding)[:, None, :]
            dense = torch.where(padding[:, :, None], eye[None], dense)
            expected = oracle.bfts_attention_mask(padding, roles, layer, layers, seq_causal=causal, seq_keep_per_domain=10)
            assert torch.equal(dense[:, None], expected), (layer, causal)
    roles = torch.randint(0, 8, (29,), generator=g)
    padding = torch.rand(2, 29, generator=g) < 0.25
    dense = metadata_structural_mask(roles)[None] & ~safe_key_padding_mask(padding)[:, None, :]
    assert torch.equal(dense[:, None], oracle.metadata_attention_mask(padding, roles))


def test_hash_compress_ids_against_the_rule_stated_per_element():
    from taac_2026_amd.api import hash_compress_ids

    values = torch.tensor([[0, 1, 2, 7, 8, 9, -3, 15, 16, 17, 10**12]])
    got = hash_compress_ids(values, 8)
    expected = [[0 if v <= 0 else (v - 1) % 8 + 1 for v in values[0].tolist()]]
    assert got.tolist() == expected and got.dtype == values.dtype
    assert got.max().item() <= 8 and (got[values > 0] >= 1).all()
    assert hash_compress_ids(values, 0).tolist() == [[0] * values.shape[1]]
    assert hash_compress_ids(values.to(torch.int32)[:, :10], 3).dtype == torch.int32
