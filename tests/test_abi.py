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
    status = library.taac_backbone_fwd(fake, fake, weights, 1, fake, None, 2, 16, 32, 4, 64, 1e-6, None, fake, 16, None, fake, None)
    assert status == _native.TAAC_ERR_INVALID_VALUE and b"workspace" in library.taac_last_error()
    status = library.taac_backbone_fwd(fake, fake, weights, 1, fake, None, 2, 16, 32, 5, 64, 1e-6, None, fake, 1 << 20, None, fake, None)
    assert status == _native.TAAC_ERR_UNSUPPORTED


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
