"""RMSNorm / LayerNorm operator boundary backed by the gfx950 row kernels.

Signatures, argument checks and error texts mirror the reference operators
(src/taac2026/infrastructure/accelerators/normalization/rms_norm.py:76-86,377-401 and layer_norm.py:69-88,261-280).
There is exactly one compute path - ``taac_rmsnorm_fwd`` / ``taac_layernorm_fwd`` of libtaac_hip.so - so the
``backend`` keyword is validated against the names the reference accepts (plus ``"hip"``) and otherwise ignored, and
``block_rows`` (a Triton/TileLang launch hint) is accepted for call-site compatibility only.
"""

from __future__ import annotations

import torch

from taac_2026_amd import _native
from taac_2026_amd.accelerators.tensor_validation import require_cuda_tensors

RMS_NORM_BACKENDS = ("hip", "torch", "tilelang", "triton")
LAYER_NORM_BACKENDS = ("hip", "torch", "triton")


def _normalize_rms_norm_inputs(x: torch.Tensor, weight: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Size]:
    if x.ndim < 2:
        raise ValueError("rms_norm expects input with at least 2 dimensions")
    if weight.ndim != 1:
        raise ValueError("rms_norm weight must be a 1D tensor")
    if x.shape[-1] != weight.shape[0]:
        raise ValueError(f"last dimension {x.shape[-1]} does not match weight size {weight.shape[0]}")
    rows = x.reshape(-1, x.shape[-1]).contiguous()
    return rows, weight.to(device=rows.device, dtype=rows.dtype).contiguous(), x.shape


def _normalize_layer_norm_inputs(
    x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Size]:
    if x.ndim < 2:
        raise ValueError("layer_norm expects input with at least 2 dimensions")
    if weight.ndim != 1:
        raise ValueError("layer_norm weight must be a 1D tensor")
    if bias.ndim != 1:
        raise ValueError("layer_norm bias must be a 1D tensor")
    if x.shape[-1] != weight.shape[0]:
        raise ValueError(f"last dimension {x.shape[-1]} does not match weight size {weight.shape[0]}")
    if weight.shape != bias.shape:
        raise ValueError(f"layer_norm weight shape {tuple(weight.shape)} does not match bias shape {tuple(bias.shape)}")
    rows = x.reshape(-1, x.shape[-1]).contiguous()
    return (
        rows,
        weight.to(device=rows.device, dtype=rows.dtype).contiguous(),
        bias.to(device=rows.device, dtype=rows.dtype).contiguous(),
        x.shape,
    )


def _resolve_rms_norm_backend(x: torch.Tensor, backend: str) -> str:
    if backend not in RMS_NORM_BACKENDS:
        raise ValueError(f"unsupported rms_norm backend: {backend}")
    require_cuda_tensors("hip rms_norm", x)
    return "hip"


def _resolve_layer_norm_backend(x: torch.Tensor, backend: str) -> str:
    if backend not in LAYER_NORM_BACKENDS:
        raise ValueError(f"unsupported layer_norm backend: {backend}")
    require_cuda_tensors("hip layer_norm", x)
    return "hip"


def resolved_rms_norm_backend(x: torch.Tensor, backend: str = "hip", *, eps: float = 1e-6, block_rows=None) -> str:
    del eps, block_rows
    return _resolve_rms_norm_backend(x, backend)


def resolved_layer_norm_backend(x: torch.Tensor, backend: str = "hip", *, eps: float = 1e-5, block_rows=None) -> str:
    del eps, block_rows
    return _resolve_layer_norm_backend(x, backend)


def hip_rms_norm_kernel(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``(rows[R, D] contiguous, weight[D] in x's dtype, eps) -> Tensor[R, D]``.

    Same contract as a kernel handed to the reference's ``register_rms_norm_kernel`` (rms_norm.py:31,66-68).
    """
    library = _native.load_library()
    require_cuda_tensors("hip rms_norm", x, weight)
    out = torch.empty_like(x)
    status = library.taac_rmsnorm_fwd(
        x.data_ptr(), weight.data_ptr(), out.data_ptr(), x.shape[0], x.shape[1], float(eps),
        _native.dtype_code(x.dtype), _native.current_stream(x.device),
    )
    _native.check(status, "rms_norm")
    return out


def hip_layer_norm_kernel(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float) -> torch.Tensor:
    """``(rows, weight, bias, eps) -> Tensor``; contract of ``register_layer_norm_kernel`` (layer_norm.py:24,60-62)."""
    library = _native.load_library()
    require_cuda_tensors("hip layer_norm", x, weight, bias)
    out = torch.empty_like(x)
    status = library.taac_layernorm_fwd(
        x.data_ptr(), weight.data_ptr(), bias.data_ptr(), out.data_ptr(), x.shape[0], x.shape[1], float(eps),
        _native.dtype_code(x.dtype), _native.current_stream(x.device),
    )
    _native.check(status, "layer_norm")
    return out


def _backward_workspace(rows: torch.Tensor, layer_norm_parts: bool) -> torch.Tensor:
    library = _native.load_library()
    count = int(library.taac_norm_bwd_workspace_floats(rows.shape[0], rows.shape[1], int(layer_norm_parts)))
    return torch.empty(count, dtype=torch.float32, device=rows.device)


def hip_rms_norm_backward_kernel(x: torch.Tensor, weight: torch.Tensor, grad_out: torch.Tensor, eps: float
                                 ) -> tuple[torch.Tensor, torch.Tensor]:
    """``(rows [R, D], weight [D], grad_out [R, D], eps) -> (grad_rows [R, D], grad_weight [D])`` in x's dtype."""
    library = _native.load_library()
    require_cuda_tensors("hip rms_norm backward", x, weight, grad_out)
    grad_x, grad_w = torch.empty_like(x), torch.empty_like(weight)
    workspace = _backward_workspace(x, False)
    status = library.taac_rmsnorm_bwd(
        x.data_ptr(), weight.data_ptr(), grad_out.data_ptr(), grad_x.data_ptr(), grad_w.data_ptr(), workspace.data_ptr(),
        workspace.numel(), x.shape[0], x.shape[1], float(eps), _native.dtype_code(x.dtype), _native.current_stream(x.device),
    )
    _native.check(status, "rms_norm backward")
    return grad_x, grad_w


def hip_rms_norm_backward_static_kernel(x: torch.Tensor, weight: torch.Tensor, grad_out: torch.Tensor, eps: float,
                                        grad_x: torch.Tensor, grad_w: torch.Tensor) -> None:
    """:func:`hip_rms_norm_backward_kernel` for callers that cannot allocate device memory (graph capture, serving loops):
    writes into the given ``grad_x [R, D]`` / ``grad_w [D]`` and keeps the partial sums in the library's built-in device
    array (``taac_rmsnorm_bwd_static``; at most 2048 columns; calls that overlap on one GPU must be serialised)."""
    library = _native.load_library()
    require_cuda_tensors("hip rms_norm backward", x, weight, grad_out, grad_x, grad_w)
    if grad_x.shape != x.shape or grad_w.shape != weight.shape or grad_x.dtype != x.dtype or grad_w.dtype != x.dtype:
        raise ValueError("rms_norm backward: grad_x / grad_w must have the shape and dtype of x / weight")
    if not (x.is_contiguous() and grad_out.is_contiguous() and grad_x.is_contiguous() and grad_w.is_contiguous()):
        raise ValueError("rms_norm backward: tensors must be contiguous")
    status = library.taac_rmsnorm_bwd_static(
        x.data_ptr(), weight.data_ptr(), grad_out.data_ptr(), grad_x.data_ptr(), grad_w.data_ptr(), x.shape[0], x.shape[1],
        float(eps), _native.dtype_code(x.dtype), _native.current_stream(x.device),
    )
    _native.check(status, "rms_norm backward")


def hip_layer_norm_backward_kernel(x: torch.Tensor, weight: torch.Tensor, grad_out: torch.Tensor, eps: float
                                   ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``-> (grad_rows, grad_weight, grad_bias)`` in x's dtype."""
    library = _native.load_library()
    require_cuda_tensors("hip layer_norm backward", x, weight, grad_out)
    grad_x, grad_w, grad_b = torch.empty_like(x), torch.empty_like(weight), torch.empty_like(weight)
    workspace = _backward_workspace(x, True)
    status = library.taac_layernorm_bwd(
        x.data_ptr(), weight.data_ptr(), grad_out.data_ptr(), grad_x.data_ptr(), grad_w.data_ptr(), grad_b.data_ptr(),
        workspace.data_ptr(), workspace.numel(), x.shape[0], x.shape[1], float(eps), _native.dtype_code(x.dtype),
        _native.current_stream(x.device),
    )
    _native.check(status, "layer_norm backward")
    return grad_x, grad_w, grad_b


class _HipRMSNormFunction(torch.autograd.Function):
    """Forward and backward on the HIP kernels (the role of _TritonRMSNormFunction, rms_norm.py:318-340); the backward
    recomputes the row statistic from the saved input, so the forward is the inference kernel."""

    @staticmethod
    def forward(ctx, rows: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
        ctx.save_for_backward(rows, weight)
        ctx.eps = float(eps)
        return hip_rms_norm_kernel(rows, weight, eps)

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        rows, weight = ctx.saved_tensors
        grad_rows, grad_weight = hip_rms_norm_backward_kernel(rows, weight, grad_out.contiguous(), ctx.eps)
        return grad_rows, grad_weight, None


class _HipLayerNormFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rows: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float) -> torch.Tensor:
        ctx.save_for_backward(rows, weight)
        ctx.eps = float(eps)
        return hip_layer_norm_kernel(rows, weight, bias, eps)

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        rows, weight = ctx.saved_tensors
        grad_rows, grad_weight, grad_bias = hip_layer_norm_backward_kernel(rows, weight, grad_out.contiguous(), ctx.eps)
        return grad_rows, grad_weight, grad_bias, None


def _needs_grad(*tensors: torch.Tensor) -> bool:
    return torch.is_grad_enabled() and any(t.requires_grad for t in tensors)


def rms_norm(
    x: torch.Tensor,
    weight: torch.Tensor,
    eps: float = 1e-6,
    *,
    backend: str = "hip",
    block_rows: int | None = None,
) -> torch.Tensor:
    """``x * rsqrt(mean(x^2, -1) + eps) * weight`` over the last dimension, fp32 accumulation. Differentiable: with
    autograd enabled and an input that requires grad, the backward runs on the HIP kernel too (rms_norm.py:345-360)."""
    del block_rows
    rows, normalized_weight, original_shape = _normalize_rms_norm_inputs(x, weight)
    _resolve_rms_norm_backend(rows, backend)
    if _needs_grad(x, weight):
        return _HipRMSNormFunction.apply(rows, normalized_weight, eps).reshape(original_shape)
    return hip_rms_norm_kernel(rows, normalized_weight, eps).reshape(original_shape)


def layer_norm(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor,
    eps: float = 1e-5,
    *,
    backend: str = "hip",
    block_rows: int | None = None,
) -> torch.Tensor:
    """``F.layer_norm(x, (D,), weight, bias, eps)`` over the last dimension, fp32 statistics. Differentiable like
    :func:`rms_norm` (layer_norm.py:170-258)."""
    del block_rows
    rows, normalized_weight, normalized_bias, original_shape = _normalize_layer_norm_inputs(x, weight, bias)
    _resolve_layer_norm_backend(rows, backend)
    if _needs_grad(x, weight, bias):
        return _HipLayerNormFunction.apply(rows, normalized_weight, normalized_bias, eps).reshape(original_shape)
    return hip_layer_norm_kernel(rows, normalized_weight, normalized_bias, eps).reshape(original_shape)


__all__ = [
    "LAYER_NORM_BACKENDS",
    "RMS_NORM_BACKENDS",
    "hip_layer_norm_backward_kernel",
    "hip_layer_norm_kernel",
    "hip_rms_norm_backward_kernel",
    "hip_rms_norm_backward_static_kernel",
    "hip_rms_norm_kernel",
    "layer_norm",
    "resolved_layer_norm_backend",
    "resolved_rms_norm_backend",
    "rms_norm",
]
