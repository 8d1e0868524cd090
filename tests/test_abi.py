"""The C-ABI library loads without a GPU, exports every symbol include/taac_hip.h declares, and rejects bad arguments
on the host before anything is launched."""

from __future__ import annotations

import ctypes
import re
from pathlib import Path

import pytest

from taac_2026_amd import _native

HEADER = Path(__file__).resolve().parents[1] / "include" / "taac_hip.h"


def _declared_symbols() -> set[str]:
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return set(re.findall(r"\b(taac_[a-z0-9_]+)\s*\(", text))


def test_header_and_binding_agree():
    declared = _declared_symbols()
    assert declared == set(_native.SIGNATURES), declared ^ set(_native.SIGNATURES)


def test_library_exports_every_declared_symbol():
    library = _native.load_library()
    for name in _declared_symbols():
        assert hasattr(library, name), name
    assert library.taac_abi_version() == _native.ABI_VERSION
    header_version = int(re.search(r"#define TAAC_ABI_VERSION (\d+)", HEADER.read_text()).group(1))
    assert header_version == _native.ABI_VERSION


def test_host_side_argument_validation_without_gpu():
    library = _native.load_library()
    fake = ctypes.c_void_p(256)
    # cols <= 0 -> invalid value
    assert library.taac_rmsnorm_fwd(fake, fake, fake, 4, 0, 1e-6, _native.TAAC_BF16, None) == _native.TAAC_ERR_INVALID_VALUE
    assert b"cols" in library.taac_last_error()
    # unknown dtype
    assert library.taac_layernorm_fwd(fake, fake, fake, fake, 4, 8, 1e-5, 9, None) == _native.TAAC_ERR_INVALID_VALUE
    # zero rows is a successful no-op
    assert library.taac_rmsnorm_fwd(fake, fake, fake, 0, 8, 1e-6, _native.TAAC_BF16, None) == _native.TAAC_OK
    strides = _native.Int64x4(64, 8, 8, 1)
    # head_dim 12 is outside the kernel's envelope -> unsupported
    status = library.taac_flash_attn_fwd(fake, fake, fake, None, fake, 1, 1, 4, 4, 12, strides, strides, strides, strides,
                                         0, 0, _native.TAAC_BF16, None)
    assert status == _native.TAAC_ERR_UNSUPPORTED and b"head_dim" in library.taac_last_error()
    # fp32 attention operands are not accepted by the kernel entry point
    status = library.taac_flash_attn_fwd(fake, fake, fake, None, fake, 1, 1, 4, 4, 16, strides, strides, strides, strides,
                                         0, 0, _native.TAAC_F32, None)
    assert status == _native.TAAC_ERR_INVALID_VALUE
    # zero_padded_queries needs Tq == Tk
    status = library.taac_flash_attn_fwd(fake, fake, fake, None, fake, 1, 1, 4, 8, 16, strides, strides, strides, strides,
                                         0, 1, _native.TAAC_BF16, None)
    assert status == _native.TAAC_ERR_INVALID_VALUE
    # dense layer: K not a multiple of 8; residual epilogue without residual; empty M is a no-op
    assert library.taac_linear_bf16(fake, 16, fake, None, None, fake, 16, 4, 16, 12, _native.EPI_NONE, 1, None) == \
        _native.TAAC_ERR_UNSUPPORTED
    assert library.taac_linear_bf16(fake, 16, fake, None, None, fake, 16, 4, 16, 16, _native.EPI_RESIDUAL, 1, None) == \
        _native.TAAC_ERR_INVALID_VALUE
    assert library.taac_linear_bf16(fake, 16, fake, None, None, fake, 16, 0, 16, 16, _native.EPI_NONE, 1, None) == _native.TAAC_OK
    assert library.taac_linear_bf16(fake, 16, fake, None, None, fake, 16, 4, 16, 16, 7, 1, None) == _native.TAAC_ERR_INVALID_VALUE
    # backbone: workspace too small
    assert library.taac_backbone_workspace_bytes(2, 16, 32, 64, 1) == 2 * (2 * 16 * 32 * 2) + 2 * 16 * 96 * 2 + 2 * 16 * 64 * 2
    assert library.taac_ffn_packed_bytes(256, 1024) == 3 * 256 * 1024 * 2 and library.taac_ffn_packed_bytes(96, 64) == -1
    assert library.taac_linear_packed_bytes(768, 256) == 768 * 256 * 2 and library.taac_linear_packed_bytes(72, 256) == -1
    weights = (_native.BlockWeights * 1)()
    status = library.taac_backbone_fwd(fake, fake, weights, 1, fake, None, 2, 16, 32, 4, 64, 1e-6, None, 0, fake, 16, None, fake, None)
    assert status == _native.TAAC_ERR_INVALID_VALUE and b"workspace" in library.taac_last_error()
    status = library.taac_backbone_fwd(fake, fake, weights, 1, fake, None, 2, 16, 32, 5, 64, 1e-6, None, 0, fake, 1 << 20, None, fake, None)
    assert status == _native.TAAC_ERR_UNSUPPORTED
    # unknown flag bits of the backbone and of the attention mask argument are rejected, not ignored
    status = library.taac_backbone_fwd(fake, fake, weights, 1, fake, None, 2, 16, 32, 4, 64, 1e-6, None, 64, fake, 1 << 20, None, fake, None)
    assert status == _native.TAAC_ERR_INVALID_VALUE and b"flag" in library.taac_last_error()
    status = library.taac_flash_attn_fwd(fake, fake, fake, None, fake, 1, 1, 4, 4, 16, strides, strides, strides, strides,
                                         4, 0, _native.TAAC_BF16, None)
    assert status == _native.TAAC_ERR_INVALID_VALUE and b"is_causal" in library.taac_last_error()


def test_host_side_validation_of_the_widened_entry_points_without_gpu():
    library = _native.load_library()
    fake = ctypes.c_void_p(256)
    bf16, f32 = _native.TAAC_BF16, _native.TAAC_F32
    invalid, unsupported, ok = _native.TAAC_ERR_INVALID_VALUE, _native.TAAC_ERR_UNSUPPORTED, _native.TAAC_OK

    # query / key normalisation + rotation
    def qk(**kw):
        a = dict(q=fake, k=fake, ld_in=64, q_out=fake, k_out=fake, ld_out=64, rows=8, tps=4, d_model=64, heads=4,
                 qw=fake, kw=fake, eps=1e-6, cos_sin=None, row_index=None, n_rows=None, dtype=bf16)
        a.update(kw)
        return library.taac_qk_norm_rope_fwd(a["q"], a["k"], a["ld_in"], a["q_out"], a["k_out"], a["ld_out"], a["rows"],
                                             a["tps"], a["d_model"], a["heads"], a["qw"], a["kw"], a["eps"],
                                             a["cos_sin"], a["row_index"], a["n_rows"], a["dtype"], None)

    assert qk(heads=5) == invalid and b"divisible" in library.taac_last_error()
    assert qk(kw=None) == invalid and b"come together" in library.taac_last_error()
    assert qk(qw=None, kw=None) == invalid and b"neither" in library.taac_last_error()
    assert qk(ld_in=32) == invalid and b"row stride" in library.taac_last_error()
    assert qk(row_index=fake) == invalid
    assert qk(rows=0) == ok
    assert qk(dtype=9) == invalid

    # embedding bag
    def bag(**kw):
        a = dict(weight=fake, n=16, e=8, values=fake, i64=0, bags=4, size=2, out=fake, count=None, dtype=f32)
        a.update(kw)
        return library.taac_embedding_bag_mean_fwd(a["weight"], a["n"], a["e"], a["values"], a["i64"], a["bags"],
                                                   a["size"], a["out"], a["count"], a["dtype"], None)

    assert bag(n=0) == invalid
    assert bag(values=None) == invalid and b"null" in library.taac_last_error()
    assert bag(bags=0) == ok
    assert bag(dtype=9) == invalid

    def bag_bwd(**kw):
        a = dict(values=fake, i64=0, bags=4, size=2, grad_out=fake, grad_weight=fake, n=16, e=8, workspace=None, dtype=f32)
        a.update(kw)
        return library.taac_embedding_bag_mean_bwd(a["values"], a["i64"], a["bags"], a["size"], a["grad_out"],
                                                   a["grad_weight"], a["n"], a["e"], a["workspace"], a["dtype"], None)

    assert bag_bwd(e=0) == invalid
    assert bag_bwd(grad_weight=None) == invalid and b"null" in library.taac_last_error()
    assert bag_bwd(dtype=bf16) == invalid and b"workspace" in library.taac_last_error()
    assert bag_bwd(dtype=9) == invalid

    # normalisation backward: workspace size, too-small workspace, width outside the envelope
    floats = library.taac_norm_bwd_workspace_floats(1000, 256, 0)
    assert floats > 0 and library.taac_norm_bwd_workspace_floats(1000, 256, 1) == 2 * floats
    assert library.taac_rmsnorm_bwd(fake, fake, fake, fake, fake, fake, 255, 1000, 256, 1e-6, bf16, None) == invalid
    assert b"workspace" in library.taac_last_error()
    # a width that is not a whole number of 16-byte vectors takes the generic kernel, which needs its workspace too
    assert library.taac_rmsnorm_bwd(fake, fake, fake, fake, fake, fake, 8 * 260 - 1, 8, 260, 1e-6, bf16, None) == invalid
    assert b"workspace" in library.taac_last_error()
    # the variant with the built-in scratch array rejects widths beyond the array before it touches the device
    assert library.taac_rmsnorm_bwd_static(fake, fake, fake, fake, fake, 8, 2056, 1e-6, bf16, None) == unsupported
    assert b"2048" in library.taac_last_error()
    assert library.taac_rmsnorm_bwd_static(fake, fake, fake, fake, fake, -1, 256, 1e-6, bf16, None) == invalid
    assert library.taac_layernorm_bwd(fake, fake, fake, None, fake, fake, fake, 1 << 30, 8, 256, 1e-5, bf16, None) == invalid

    # out projection + feed-forward half in one kernel: both weight sets packed, the block input required
    def tail(**kw):
        a = dict(packed_out=fake, residual=fake, packed_ffn=fake, d=256, f=64, m=8, rows=None, attn_rows=None)
        a.update(kw)
        return library.taac_attn_out_ffn_fwd(fake, a["d"], None, a["packed_out"], a["residual"], a["d"], None, 1e-6, None,
                                             None, a["packed_ffn"], fake, a["d"], a["m"], a["d"], a["f"], a["rows"], a["rows"],
                                             a["attn_rows"], a.get("folded", 0), None)

    assert tail(folded=1) == invalid and b"norm_folded needs" in library.taac_last_error()
    assert tail(packed_out=None) == invalid and b"packed" in library.taac_last_error()
    assert tail(packed_ffn=None) == invalid
    assert tail(residual=None) == invalid and b"block input" in library.taac_last_error()
    assert tail(d=192) == unsupported
    assert tail(f=48) == unsupported
    assert tail(m=0) == ok
    assert tail(attn_rows=fake) == invalid and b"x_rows needs rows" in library.taac_last_error()
    status = library.taac_norm_linear_fwd(fake, 256, None, 1e-6, fake, None, None, None, 0, fake, 64, 8, 64, 256, None, None,
                                          fake, 0, None)
    assert status == invalid and b"x_rows needs rows" in library.taac_last_error()
    status = library.taac_norm_linear_fwd(fake, 256, fake, 1e-6, fake, None, None, None, 0, fake, 64, 8, 64, 256, None, None,
                                          None, 1, None)
    assert status == invalid and b"norm_folded needs" in library.taac_last_error()

    # the same two layers on per-head planes: packed weights only, head_dim 32 or 64, model width 128 / 256
    def plane_projection(**kw):
        a = dict(packed=fake, head_dim=32, m=8, n=768, k=256)
        a.update(kw)
        return library.taac_norm_linear_heads_fwd(fake, a["k"], None, 1e-6, None, a["packed"], fake, a["head_dim"], a["m"],
                                                  a["n"], a["k"], None, None, 0, None)

    assert plane_projection(packed=None) == invalid and b"packed" in library.taac_last_error()
    assert plane_projection(head_dim=16) == unsupported and b"head_dim" in library.taac_last_error()
    assert plane_projection(k=192) == unsupported
    assert plane_projection(m=0) == ok

    def plane_tail(**kw):
        a = dict(packed_out=fake, residual=fake, packed_ffn=fake, head_dim=64, d=256, f=64, m=8)
        a.update(kw)
        return library.taac_attn_out_ffn_heads_fwd(fake, a["head_dim"], None, a["packed_out"], a["residual"], a["d"], None,
                                                   1e-6, None, None, a["packed_ffn"], fake, a["d"], a["m"], a["d"], a["f"],
                                                   None, None, 0, None)

    assert plane_tail(packed_out=None) == invalid and b"packed" in library.taac_last_error()
    assert plane_tail(head_dim=48) == unsupported and b"head_dim" in library.taac_last_error()
    assert plane_tail(residual=None) == invalid and b"block input" in library.taac_last_error()
    assert plane_tail(d=192) == unsupported
    assert plane_tail(m=0) == ok

    # the flags of norm_folded: the activation's constants come with a packed gated blob at a supported shape, a linear
    # layer knows the norm flag only
    def folded_ffn(flags, **kw):
        a = dict(packed=fake, norm=fake, d=256, f=64, m=0)
        a.update(kw)
        return library.taac_swiglu_ffn_fwd(fake, a["d"], a["norm"], 1e-6, fake, None, fake, None, a["packed"], None, a["d"], fake,
                                           a["d"], a["m"], a["d"], a["f"], 1, None, None, flags, None)

    both = _native.FOLDED_NORM | _native.FOLDED_ACTIVATION
    assert folded_ffn(both) == ok and folded_ffn(_native.FOLDED_ACTIVATION, norm=None) == ok
    assert folded_ffn(4) == invalid and b"TAAC_FOLDED" in library.taac_last_error()
    assert folded_ffn(_native.FOLDED_ACTIVATION, packed=None) == invalid and b"taac_ffn_pack_weights_folded" in library.taac_last_error()
    assert folded_ffn(both, f=36864) == invalid  # no room for three weight buffers: such a blob cannot exist
    assert library.taac_ffn_activation_fold_supported(256, 1024) == 1 and library.taac_ffn_activation_fold_supported(128, 512) == 1
    assert library.taac_ffn_activation_fold_supported(256, 36864) == 0 and library.taac_ffn_activation_fold_supported(64, 128) == 0
    assert library.taac_ffn_pack_weights_folded(fake, fake, None, fake, 256, 36864, 1, 1, None) == unsupported
    assert library.taac_ffn_pack_weights_folded(fake, None, None, fake, 256, 64, 1, 1, None) == invalid
    assert library.taac_attn_out_gate_ffn_fwd(fake, 256, None, fake, fake, 256, fake, 256, None, 1e-6, None, None, fake, fake, 256,
                                              0, 256, 64, None, None, None, _native.FOLDED_ACTIVATION, None) == invalid
    assert library.taac_norm_linear_fwd(fake, 256, fake, 1e-6, None, None, fake, None, 256, fake, 256, 0, 256, 256, None, None,
                                        None, 2, None) == invalid

    # readout: indices inside the sequence, one kind of validity, a complete classifier, something to write
    def readout(**kw):
        a = dict(lengths=None, bits=None, t=16, d=64, cls=0, cand=3, fc1=fake, fc2=fake, hidden=32, actions=1, emb=None,
                 logits=fake, b=2)
        a.update(kw)
        return library.taac_candidate_readout_fwd(fake, a["lengths"], a["bits"], a["b"], a["t"], a["d"], a["cls"], a["cand"],
                                                  None, None, 1e-6, a["fc1"], None, a["hidden"], a["fc2"], None,
                                                  a["actions"], a["emb"], a["logits"], 0, None)

    assert readout(cls=16) == invalid and b"outside the sequence" in library.taac_last_error()
    assert readout(cand=16) == invalid
    assert readout(lengths=fake, bits=fake) == invalid and b"not both" in library.taac_last_error()
    assert readout(d=12) == unsupported and readout(d=2048) == unsupported
    assert readout(hidden=2048) == unsupported
    assert readout(fc2=None) == invalid and readout(logits=None) == invalid
    assert readout(fc1=None, emb=None) == invalid and b"nothing to compute" in library.taac_last_error()
    assert readout(b=0) == ok

    # attention with structured masks, the training forward and the backward
    strides = _native.Int64x4(2048, 16, 128, 1)

    def masked(**kw):
        a = dict(lengths=None, struct=fake, stride=0, any=fake, valid=None, self=None, tq=64, tk=64, d=16, zero=0, dtype=bf16)
        a.update(kw)
        return library.taac_flash_attn_masked_fwd(fake, fake, fake, a["lengths"], a["struct"], a["stride"], a["any"], a["valid"],
                                                  a["self"], None, None, None, fake, 1, 8, a["tq"], a["tk"], a["d"],
                                                  strides, strides, strides, strides, a["zero"], a["dtype"], None)

    assert masked(struct=None) == invalid and b"struct_bits" in library.taac_last_error()
    assert masked(any=None) == invalid and b"block_any" in library.taac_last_error()
    assert masked(stride=64) == invalid and b"struct_sample_stride" in library.taac_last_error()
    assert masked(stride=-1) == invalid
    # the row index of the front layout and the mask gathered into it
    assert library.taac_front_rows(None, fake, 2, 8, fake, fake, None) == invalid and b"null" in library.taac_last_error()
    assert library.taac_front_rows(fake, fake, 0, 8, fake, fake, None) == ok
    assert library.taac_front_rows(fake, fake, -1, 8, fake, fake, None) == invalid
    assert library.taac_mask_front_bits(fake, 8192, fake, 2, fake, None) == unsupported
    assert library.taac_mask_front_bits(None, 8, fake, 2, fake, None) == invalid
    assert library.taac_mask_front_bits(fake, 8, fake, 0, fake, None) == ok
    assert masked(tk=4096 + 64) == unsupported and b"at most" in library.taac_last_error()
    assert masked(self=fake, tk=128) == invalid and b"self rows" in library.taac_last_error()
    assert masked(d=12) == unsupported
    assert library.taac_mask_pack_bits(None, 4, 4, fake, None) == invalid
    assert library.taac_mask_pack_bits(fake, 0, 4, fake, None) == ok
    assert library.taac_mask_block_any(fake, 0, 4, fake, None) == invalid

    def per_tile(**kw):
        a = dict(bits=fake, keys=fake, tiles=fake, tq=64, tk=64, d=32, strides=strides)
        a.update(kw)
        return library.taac_flash_attn_sparse_fwd(fake, fake, fake, None, a["bits"], 0, a["keys"], a["tiles"], None, None, None,
                                                  None, None, fake, 1, 8, a["tq"], a["tk"], a["d"], strides, a["strides"],
                                                  a["strides"], strides, 0, bf16, None)

    assert per_tile(keys=None) == invalid and b"compact_keys" in library.taac_last_error()
    assert per_tile(tiles=None) == invalid and per_tile(bits=None) == invalid
    assert per_tile(d=128) == unsupported and b"head_dim" in library.taac_last_error()
    assert per_tile(tk=4096) == unsupported and b"2048" in library.taac_last_error()
    assert per_tile(strides=_native.Int64x4(1 << 40, 1 << 30, 1 << 23, 1)) == unsupported and b"32-bit" in library.taac_last_error()
    assert library.taac_mask_compact(fake, 1, 0, 64, 0, fake, fake, fake, None) == invalid
    assert library.taac_mask_compact(None, 1, 64, 64, 0, fake, fake, fake, None) == invalid
    assert library.taac_mask_compact(fake, 1, 64, 4096, 0, fake, fake, fake, None) == unsupported
    assert library.taac_mask_compact(fake, 2, 64, 64, 16, fake, fake, fake, None) == invalid and b"stride" in library.taac_last_error()
    status = library.taac_flash_attn_train_fwd(fake, fake, fake, None, fake, None, 1, 8, 64, 64, 16, strides, strides,
                                               strides, strides, 0, 0, bf16, None)
    assert status == invalid and b"lse" in library.taac_last_error()

    def backward(**kw):
        a = dict(lse=fake, delta=fake, tq=64, tk=64, d=16, zero=0, dtype=bf16)
        a.update(kw)
        return library.taac_flash_attn_bwd(fake, fake, fake, fake, fake, a["lse"], None, fake, fake, fake, a["delta"],
                                           1, 8, a["tq"], a["tk"], a["d"], strides, strides, strides, strides, strides,
                                           strides, strides, strides, 0, a["zero"], a["dtype"], None)

    assert backward(d=72) == unsupported and b"head_dim" in library.taac_last_error()
    assert backward(dtype=f32) == invalid
    assert backward(lse=None) == invalid and b"null" in library.taac_last_error()
    assert backward(tk=0) == unsupported
    assert backward(tq=64, tk=128, zero=1) == invalid

    # training under structured masks: the structured forward with the log-sum-exp, the bit-form and byte-form backward
    def masked_train(**kw):
        a = dict(bits=fake, stride=0, block_any=fake, self=None, keep=None, scale=1.0, lse=fake, tq=64, tk=64)
        a.update(kw)
        return library.taac_flash_attn_masked_train_fwd(fake, fake, fake, None, a["bits"], a["stride"], a["block_any"], None,
                                                        a["self"], a["keep"], a["scale"], fake, a["lse"], 1, 8, a["tq"],
                                                        a["tk"], 16, strides, strides, strides, strides, 0, bf16, None)

    assert masked_train(bits=None) == invalid and b"struct_bits" in library.taac_last_error()
    assert masked_train(lse=None) == invalid and b"lse" in library.taac_last_error()
    assert masked_train(block_any=None) == invalid and b"block_any" in library.taac_last_error()
    assert masked_train(keep=fake, scale=0.5) == invalid and b"dropout_scale" in library.taac_last_error()
    assert masked_train(keep=fake, scale=1.25, self=fake) == unsupported and b"self-only" in library.taac_last_error()

    def bits_backward(**kw):
        a = dict(bits=fake, stride=0, keep=None, scale=1.0, d=16, lse=fake)
        a.update(kw)
        return library.taac_flash_attn_bits_bwd(fake, fake, fake, fake, fake, a["lse"], None, a["bits"], a["stride"], None,
                                                a["keep"], a["scale"], fake, fake, fake, fake, 1, 8, 64, 64, a["d"], strides,
                                                strides, strides, strides, strides, strides, strides, strides, 0, bf16, None)

    assert bits_backward(bits=None) == invalid and b"struct_bits" in library.taac_last_error()
    assert bits_backward(stride=-4) == invalid and b"stride" in library.taac_last_error()
    assert bits_backward(d=72) == unsupported and b"head_dim" in library.taac_last_error()
    assert bits_backward(keep=fake, scale=0.5) == invalid and b"dropout_scale" in library.taac_last_error()
    assert bits_backward(lse=None) == invalid
    status = library.taac_flash_attn_mask_bwd(fake, fake, fake, fake, fake, fake, None, None, 0, 0, None, fake, fake, fake, fake,
                                              1, 8, 64, 64, 16, strides, strides, strides, strides, strides, strides, strides,
                                              strides, 0, bf16, None)
    assert status == invalid and b"visibility" in library.taac_last_error()
    status = library.taac_flash_attn_mask_bwd(fake, fake, fake, fake, fake, fake, None, fake, -1, 0, None, fake, fake, fake, fake,
                                              1, 8, 64, 64, 16, strides, strides, strides, strides, strides, strides, strides,
                                              strides, 0, bf16, None)
    assert status == invalid and b"stride" in library.taac_last_error()
    # the gradient merge for scattered padding
    assert library.taac_rows_merge_bits(fake, fake, None, fake, None, fake, fake, 2, 8, 12, None) == unsupported
    assert library.taac_rows_merge_bits(fake, fake, None, None, None, fake, fake, 2, 8, 16, None) == invalid
    assert library.taac_rows_merge_bits(fake, fake, None, fake, None, fake, fake, 0, 8, 16, None) == ok
    assert library.taac_rows_merge_bits(fake, fake, None, fake, None, fake, fake, -1, 8, 16, None) == invalid


def test_status_mapping_to_python_exceptions():
    library = _native.load_library()
    fake = ctypes.c_void_p(256)
    status = library.taac_rmsnorm_fwd(fake, fake, fake, 4, 0, 1e-6, _native.TAAC_BF16, None)
    with pytest.raises(ValueError, match="rms_norm"):
        _native.check(status, "rms_norm")
    strides = _native.Int64x4(64, 8, 8, 1)
    status = library.taac_flash_attn_fwd(fake, fake, fake, None, fake, 1, 1, 4, 4, 12, strides, strides, strides, strides,
                                         0, 0, _native.TAAC_BF16, None)
    with pytest.raises(RuntimeError, match="head_dim"):
        _native.check(status, "flash_attention")
    _native.check(_native.TAAC_OK, "anything")
