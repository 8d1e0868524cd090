"""ctypes binding of libtaac_hip.so (declared in include/taac_hip.h).

The library is the only compute backend of this package: if it cannot be loaded every operator raises
``RuntimeError`` - there is no eager / CPU fallback.
"""

from __future__ import annotations

import ctypes
import threading
from pathlib import Path

import torch

LIBRARY_PATH = Path(__file__).resolve().parent / "libtaac_hip.so"

TAAC_OK = 0
TAAC_ERR_INVALID_VALUE = -1
TAAC_ERR_UNSUPPORTED = -2
TAAC_ERR_LAUNCH = -3

TAAC_F32, TAAC_BF16, TAAC_F16 = 0, 1, 2
EPI_NONE, EPI_RESIDUAL, EPI_SWIGLU = 0, 1, 2
ATTN_CAUSAL, ATTN_REGISTER_STAGING = 1, 2
BACKBONE_DENSE_TOKENS, BACKBONE_SPLIT_OUT_FFN, BACKBONE_FP8, BACKBONE_ROW_MAJOR_QKV = 1, 2, 4, 8
FOLDED_NORM, FOLDED_ACTIVATION = 1, 2

ABI_VERSION = 9

_DTYPE_CODES = {torch.float32: TAAC_F32, torch.bfloat16: TAAC_BF16, torch.float16: TAAC_F16}

c_void_p = ctypes.c_void_p
c_int = ctypes.c_int
c_int32 = ctypes.c_int32
c_int64 = ctypes.c_int64
c_float = ctypes.c_float
Int64x4 = c_int64 * 4


class BlockWeights(ctypes.Structure):
    """Mirror of ``taac_block_weights``."""

    _fields_ = [
        ("attn_norm_weight", c_void_p),
        ("qkv_weight", c_void_p),
        ("qkv_bias", c_void_p),
        ("out_weight", c_void_p),
        ("out_bias", c_void_p),
        ("ffn_norm_weight", c_void_p),
        ("up_weight", c_void_p),
        ("up_bias", c_void_p),
        ("down_weight", c_void_p),
        ("down_bias", c_void_p),
        ("query_norm_weight", c_void_p),
        ("key_norm_weight", c_void_p),
    ]


# name -> (restype, argtypes); every symbol include/taac_hip.h declares.
SIGNATURES: dict[str, tuple[object, list[object]]] = {
    "taac_abi_version": (c_int, []),
    "taac_last_error": (ctypes.c_char_p, []),
    "taac_test_hooks": (None, [c_int32, c_int32]),
    "taac_rmsnorm_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_float, c_int, c_void_p]),
    "taac_layernorm_fwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_float, c_int, c_void_p],
    ),
    "taac_norm_bwd_workspace_floats": (c_int64, [c_int64, c_int32, c_int]),
    "taac_rmsnorm_bwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32, c_float, c_int, c_void_p],
    ),
    "taac_layernorm_bwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32, c_float, c_int,
         c_void_p],
    ),
    "taac_rmsnorm_bwd_static": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_float, c_int, c_void_p],
    ),
    "taac_flash_attn_fwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32]
        + [ctypes.POINTER(c_int64)] * 4
        + [c_int, c_int, c_int, c_void_p],
    ),
    "taac_flash_attn_scaled_fwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32,
         c_int32]
        + [ctypes.POINTER(c_int64)] * 4
        + [c_int, c_int, c_int, c_void_p],
    ),
    "taac_flash_attn_amax_fwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32,
         c_int32, c_int32]
        + [ctypes.POINTER(c_int64)] * 4
        + [c_int, c_int, c_int, c_void_p],
    ),
    "taac_flash_attn_masked_fwd": (
        c_int,
        [c_void_p] * 5 + [c_int64] + [c_void_p] * 7 + [c_int32, c_int32, c_int32, c_int32, c_int32]
        + [ctypes.POINTER(c_int64)] * 4
        + [c_int, c_int, c_void_p],
    ),
    "taac_flash_attn_sparse_fwd": (
        c_int,
        [c_void_p] * 5 + [c_int64] + [c_void_p] * 8 + [c_int32, c_int32, c_int32, c_int32, c_int32]
        + [ctypes.POINTER(c_int64)] * 4
        + [c_int, c_int, c_void_p],
    ),
    "taac_mask_compact": (c_int, [c_void_p, c_int32, c_int32, c_int32, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "taac_mask_pack_bits": (c_int, [c_void_p, c_int64, c_int32, c_void_p, c_void_p]),
    "taac_mask_block_any": (c_int, [c_void_p, c_int32, c_int32, c_void_p, c_void_p]),
    "taac_flash_attn_train_fwd": (
        c_int,
        [c_void_p] * 6 + [c_int32, c_int32, c_int32, c_int32, c_int32]
        + [ctypes.POINTER(c_int64)] * 4
        + [c_int, c_int, c_int, c_void_p],
    ),
    "taac_flash_attn_bwd": (
        c_int,
        [c_void_p] * 11 + [c_int32, c_int32, c_int32, c_int32, c_int32]
        + [ctypes.POINTER(c_int64)] * 8
        + [c_int, c_int, c_int, c_void_p],
    ),
    "taac_linear_wgrad_workspace_floats": (c_int64, [c_int64, c_int32, c_int32]),
    "taac_linear_wgrad": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32, c_int32, c_int, c_void_p],
    ),
    "taac_swiglu_bwd": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int32, c_int, c_void_p],
    ),
    "taac_rows_gather": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int32, c_void_p]),
    "taac_rows_merge": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_void_p]),
    "taac_rows_merge_bits": (c_int, [c_void_p] * 7 + [c_int32, c_int32, c_int32, c_void_p]),
    "taac_swiglu_ffn_bwd_packed_bytes": (c_int64, [c_int32, c_int32]),
    "taac_swiglu_ffn_bwd_pack_weights": (c_int, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_void_p]),
    "taac_swiglu_ffn_bwd_hidden": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int32,
         c_int32, c_int, c_void_p],
    ),
    "taac_flash_attn_masked_train_fwd": (
        c_int,
        [c_void_p] * 5 + [c_int64] + [c_void_p] * 4 + [c_float] + [c_void_p] * 2 + [c_int32] * 5
        + [ctypes.POINTER(c_int64)] * 4 + [c_int, c_int, c_void_p],
    ),
    "taac_flash_attn_mask_bwd": (
        c_int,
        [c_void_p] * 8 + [c_int64, c_int64] + [c_void_p] * 5 + [c_int32] * 5 + [ctypes.POINTER(c_int64)] * 8
        + [c_int, c_int, c_void_p],
    ),
    "taac_flash_attn_bits_bwd": (
        c_int,
        [c_void_p] * 8 + [c_int64] + [c_void_p] * 2 + [c_float] + [c_void_p] * 4 + [c_int32] * 5
        + [ctypes.POINTER(c_int64)] * 8 + [c_int, c_int, c_void_p],
    ),
    "taac_flash_attn_train_dropout_fwd": (
        c_int,
        [c_void_p] * 5 + [c_float] + [c_void_p] * 2 + [c_int32, c_int32, c_int32, c_int32, c_int32]
        + [ctypes.POINTER(c_int64)] * 4
        + [c_int, c_int, c_int, c_void_p],
    ),
    "taac_flash_attn_dropout_bwd": (
        c_int,
        [c_void_p] * 8 + [c_float] + [c_void_p] * 4 + [c_int32, c_int32, c_int32, c_int32, c_int32]
        + [ctypes.POINTER(c_int64)] * 8
        + [c_int, c_int, c_int, c_void_p],
    ),
    "taac_linear_bf16": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32, c_int32, c_int, c_int,
         c_void_p],
    ),
    "taac_linear_f16": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32, c_int32, c_int, c_int,
         c_void_p],
    ),
    "taac_swiglu_ffn_fwd": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
         c_void_p, c_int64, c_int64, c_int32, c_int32, c_int, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "taac_attn_out_ffn_fwd": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_float, c_void_p, c_void_p, c_void_p,
         c_void_p, c_int64, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "taac_norm_linear_heads_fwd": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_int32, c_void_p,
         c_void_p, c_int, c_void_p],
    ),
    "taac_attn_out_ffn_heads_fwd": (
        c_int,
        [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_float, c_void_p, c_void_p, c_void_p,
         c_void_p, c_int64, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "taac_silu_mlp_packed_bytes": (c_int64, [c_int32, c_int32]),
    "taac_silu_mlp_pack_weights": (c_int, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_void_p]),
    "taac_silu_mlp_fwd": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64,
         c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p],
    ),
    "taac_attn_out_gate_ffn_fwd": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_float, c_void_p,
         c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "taac_norm_linear_fwd": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64,
         c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "taac_front_rows": (c_int, [c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_void_p, c_void_p]),
    "taac_mask_front_bits": (c_int, [c_void_p, c_int32, c_void_p, c_int32, c_void_p, c_void_p]),
    "taac_valid_rows": (c_int, [c_void_p, c_int32, c_int32, c_void_p, c_void_p, c_void_p]),
    "taac_valid_rows_from_bits": (c_int, [c_void_p, c_int32, c_int32, c_void_p, c_void_p, c_void_p]),
    "taac_norm_linear_qk_fwd": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32,
         c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "taac_row_rstd": (c_int, [c_void_p, c_int64, c_int32, c_float, c_void_p, c_void_p, c_void_p, c_void_p]),
    "taac_qk_norm_rope_fwd": (
        c_int,
        [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int32, c_int32, c_int32, c_void_p,
         c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "taac_ffn_packed_bytes": (c_int64, [c_int32, c_int32]),
    "taac_ffn_pack_weights": (c_int, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int, c_void_p]),
    "taac_ffn_pack_weights_norm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int, c_void_p]),
    "taac_ffn_activation_fold_supported": (c_int, [c_int32, c_int32]),
    "taac_ffn_pack_weights_folded": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int, c_int, c_void_p]),
    "taac_linear_packed_bytes": (c_int64, [c_int32, c_int32]),
    "taac_linear_pack_weights": (c_int, [c_void_p, c_void_p, c_int32, c_int32, c_void_p]),
    "taac_linear_pack_weights_norm": (c_int, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_void_p]),
    "taac_amax": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p]),
    "taac_quantize_fp8": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p]),
    "taac_linear_fp8": (
        c_int,
        [c_void_p, c_int, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
         c_int32, c_int32, c_int, c_int, c_void_p],
    ),
    "taac_embedding_bag_mean_fwd": (
        c_int,
        [c_void_p, c_int64, c_int32, c_void_p, c_int, c_int64, c_int32, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "taac_embedding_bag_mean_bwd": (
        c_int,
        [c_void_p, c_int, c_int64, c_int32, c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_int, c_void_p],
    ),
    "taac_candidate_readout_fwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_float,
         c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "taac_masked_mean_head": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_void_p],
    ),
    "taac_backbone_workspace_bytes": (c_int64, [c_int32, c_int32, c_int32, c_int32, c_int32]),
    "taac_backbone_fp8_scales_offset": (c_int64, [c_int32, c_int32, c_int32, c_int32, c_int32]),
    "taac_norm_linear_fp8_fwd": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64,
         c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p],
    ),
    "taac_ffn_fp8_packed_bytes": (c_int64, [c_int32, c_int32]),
    "taac_ffn_fp8_pack_weights": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int, c_void_p]),
    "taac_swiglu_ffn_fp8_fwd": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int32, c_int32, c_int, c_void_p, c_void_p, c_void_p, c_float,
         c_void_p, c_void_p],
    ),
    "taac_backbone_fwd": (
        c_int,
        [c_void_p, c_void_p, ctypes.POINTER(BlockWeights), c_int32, c_void_p, c_void_p, c_int32, c_int32, c_int32,
         c_int32, c_int32, c_float, c_void_p, c_int, c_void_p, c_int64, c_void_p, c_void_p, c_void_p],
    ),
}

_lock = threading.Lock()
_library: ctypes.CDLL | None = None


def library_available() -> bool:
    return LIBRARY_PATH.exists()


def load_library() -> ctypes.CDLL:
    """Load libtaac_hip.so once and attach the prototypes. Raises RuntimeError when it is missing."""
    global _library
    if _library is not None:
        return _library
    with _lock:
        if _library is not None:
            return _library
        if not LIBRARY_PATH.exists():
            raise RuntimeError(
                f"libtaac_hip.so not found at {LIBRARY_PATH}: build it with `python -m taac_2026_amd.build`; "
                "this package has no fallback backend"
            )
        try:
            library = ctypes.CDLL(str(LIBRARY_PATH))
        except OSError as error:
            raise RuntimeError(f"failed to load {LIBRARY_PATH}: {error}") from error
        for name, (restype, argtypes) in SIGNATURES.items():
            function = getattr(library, name)
            function.restype = restype
            function.argtypes = argtypes
        version = library.taac_abi_version()
        if version != ABI_VERSION:
            raise RuntimeError(f"libtaac_hip.so ABI version {version} does not match the binding ({ABI_VERSION})")
        _library = library
        return library


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODES[dtype]
    except KeyError:
        raise RuntimeError(f"libtaac_hip does not support dtype {dtype}") from None


def check(status: int, operator_name: str) -> None:
    """Map a taac_status to the reference's error taxonomy: ValueError for bad arguments, RuntimeError otherwise."""
    if status == TAAC_OK:
        return
    message = load_library().taac_last_error().decode("utf-8", "replace")
    if status == TAAC_ERR_INVALID_VALUE:
        raise ValueError(f"{operator_name}: {message}")
    raise RuntimeError(f"{operator_name}: {message}")


def ptr(tensor: torch.Tensor | None) -> int | None:
    return None if tensor is None else tensor.data_ptr()


def current_stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


__all__ = [
    "ABI_VERSION",
    "BlockWeights",
    "EPI_NONE",
    "EPI_RESIDUAL",
    "EPI_SWIGLU",
    "Int64x4",
    "LIBRARY_PATH",
    "SIGNATURES",
    "check",
    "current_stream",
    "dtype_code",
    "library_available",
    "load_library",
    "ptr",
]
