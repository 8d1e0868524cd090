"""Tensor checks shared by the HIP operators.

Error types and message texts follow the reference's helpers
(src/taac2026/infrastructure/accelerators/tensor_validation.py:14-38): device problems are ``RuntimeError``,
dtype disagreements are ``ValueError``.
"""

from __future__ import annotations

from collections.abc import Iterable

import torch


def concrete_tensors(tensors: Iterable[torch.Tensor | None]) -> tuple[torch.Tensor, ...]:
    return tuple(t for t in tensors if t is not None)


def require_same_device(operator_name: str, *tensors: torch.Tensor | None) -> torch.device | None:
    present = concrete_tensors(tensors)
    if not present:
        return None
    first = present[0].device
    if any(t.device != first for t in present[1:]):
        raise RuntimeError(f"{operator_name} requires all tensors to live on the same device")
    return first


def require_cuda_tensors(operator_name: str, *tensors: torch.Tensor | None) -> torch.device | None:
    device = require_same_device(operator_name, *tensors)
    if device is not None and device.type != "cuda":
        raise RuntimeError(f"{operator_name} requires CUDA tensors")
    return device


def require_same_dtype(operator_name: str, *tensors: torch.Tensor | None) -> torch.dtype | None:
    present = concrete_tensors(tensors)
    if not present:
        return None
    first = present[0].dtype
    if any(t.dtype != first for t in present[1:]):
        raise ValueError(f"{operator_name} requires tensors to share the same dtype")
    return first


def require_inference(operator_name: str, *tensors: torch.Tensor | None) -> None:
    """The HIP kernels are forward-only: refuse to silently drop a gradient."""
    if torch.is_grad_enabled() and any(t.requires_grad for t in concrete_tensors(tensors)):
        raise RuntimeError(
            f"{operator_name} is forward-only: call it under torch.no_grad() or torch.inference_mode()"
        )


__all__ = [
    "concrete_tensors",
    "require_cuda_tensors",
    "require_inference",
    "require_same_device",
    "require_same_dtype",
]
