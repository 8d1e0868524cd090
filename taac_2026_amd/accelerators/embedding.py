"""Embedding-bag operator boundary backed by the gfx950 gather kernel.

Mirrors ``embedding_bag_mean`` (src/taac2026/infrastructure/accelerators/embedding/embedding_bag.py:86-100, 439-467):
``F.embedding_bag(values, weight, mode="mean", padding_idx=0)`` for a (bags, bag_size) id matrix.
"""

from __future__ import annotations

import torch

from taac_2026_amd import _native
from taac_2026_amd.accelerators.tensor_validation import require_cuda_tensors, require_same_device

EMBEDDING_BAG_MEAN_BACKENDS = ("hip", "torch", "tilelang", "triton", "cuembed")


def _normalize_embedding_bag_mean_inputs(
    embedding_weight: torch.Tensor, values: torch.Tensor
) -> tuple[torch.Tensor, torch.Tensor, torch.Size]:
    """embedding_bag.py:86-100."""
    if embedding_weight.ndim != 2:
        raise ValueError("embedding_bag_mean weight must be a 2D tensor")
    if values.ndim != 2:
        raise ValueError("embedding_bag_mean values must be a 2D tensor")
    require_same_device("embedding_bag_mean", embedding_weight, values)
    return embedding_weight.contiguous(), values.contiguous(), values.shape


def _resolve_embedding_bag_mean_backend(embedding_weight: torch.Tensor, values: torch.Tensor, backend: str) -> str:
    if backend not in EMBEDDING_BAG_MEAN_BACKENDS:
        raise ValueError(f"unsupported embedding_bag_mean backend: {backend}")
    require_cuda_tensors("hip embedding_bag_mean", embedding_weight, values)
    if embedding_weight.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise RuntimeError(f"hip embedding_bag_mean does not support dtype {embedding_weight.dtype}")
    if values.dtype not in (torch.int32, torch.int64):
        raise RuntimeError(f"hip embedding_bag_mean requires int32 or int64 values, got {values.dtype}")
    return "hip"


def resolved_embedding_bag_mean_backend(embedding_weight: torch.Tensor, values: torch.Tensor, backend: str = "hip", *,
                                        block_rows: int | None = None, block_cols: int | None = None) -> str:
    del block_rows, block_cols
    weight, ids, _ = _normalize_embedding_bag_mean_inputs(embedding_weight, values)
    return _resolve_embedding_bag_mean_backend(weight, ids, backend)


def hip_embedding_bag_mean_kernel(embedding_weight: torch.Tensor, values: torch.Tensor, *,
                                  check_indices: bool = False) -> torch.Tensor:
    """``(weight (N, E), values (B, L) int32 / int64) -> (B, E)`` in weight's dtype: the contract of a kernel handed to
    the reference's ``register_embedding_bag_mean_kernel`` (embedding_bag.py:39,77-79). ``check_indices`` reads back the
    count of ids outside ``[0, N)`` (a host synchronisation) and raises ``IndexError`` like the torch backend; without
    it such ids are skipped like padding."""
    library = _native.load_library()
    require_cuda_tensors("hip embedding_bag_mean", embedding_weight, values)
    out = torch.empty(values.shape[0], embedding_weight.shape[1], dtype=embedding_weight.dtype, device=embedding_weight.device)
    counter = torch.zeros(1, dtype=torch.int32, device=values.device) if check_indices else None
    status = library.taac_embedding_bag_mean_fwd(
        embedding_weight.data_ptr(), embedding_weight.shape[0], embedding_weight.shape[1], values.data_ptr(),
        int(values.dtype == torch.int64), values.shape[0], values.shape[1], out.data_ptr(), _native.ptr(counter),
        _native.dtype_code(embedding_weight.dtype), _native.current_stream(embedding_weight.device),
    )
    _native.check(status, "embedding_bag_mean")
    if counter is not None and int(counter.item()) != 0:
        raise IndexError(f"embedding_bag_mean: {int(counter.item())} ids are outside [0, {embedding_weight.shape[0]})")
    return out


def hip_embedding_bag_mean_backward_kernel(values: torch.Tensor, grad_out: torch.Tensor, num_embeddings: int) -> torch.Tensor:
    """``(values (B, L), grad_out (B, E)) -> grad_weight (N, E)`` in grad_out's dtype: the backward kernels of the
    reference (embedding/kernels/triton.py:91-150, tilelang.py:95-140). fp32 sums; a 16-bit gradient is rounded once."""
    library = _native.load_library()
    require_cuda_tensors("hip embedding_bag_mean backward", values, grad_out)
    grad_out = grad_out.contiguous()
    emb_dim = grad_out.shape[1]
    grad_weight = torch.empty(num_embeddings, emb_dim, dtype=grad_out.dtype, device=grad_out.device)
    workspace = None
    if grad_out.dtype != torch.float32:
        workspace = torch.empty(num_embeddings, emb_dim, dtype=torch.float32, device=grad_out.device)
    status = library.taac_embedding_bag_mean_bwd(
        values.data_ptr(), int(values.dtype == torch.int64), values.shape[0], values.shape[1], grad_out.data_ptr(),
        grad_weight.data_ptr(), num_embeddings, emb_dim, _native.ptr(workspace), _native.dtype_code(grad_out.dtype),
        _native.current_stream(grad_out.device),
    )
    _native.check(status, "embedding_bag_mean backward")
    return grad_weight


class _HipEmbeddingBagMeanFunction(torch.autograd.Function):
    """embedding_bag.py:327-353: the ids are saved, the table's gradient comes from the backward kernel."""

    @staticmethod
    def forward(ctx, embedding_weight: torch.Tensor, values: torch.Tensor, check_indices: bool) -> torch.Tensor:
        out = hip_embedding_bag_mean_kernel(embedding_weight, values, check_indices=check_indices)
        ctx.save_for_backward(values)
        ctx.num_embeddings = embedding_weight.shape[0]
        ctx.weight_dtype = embedding_weight.dtype
        return out

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        if not ctx.needs_input_grad[0]:
            return None, None, None
        (values,) = ctx.saved_tensors
        grad_weight = hip_embedding_bag_mean_backward_kernel(values, grad_out.to(ctx.weight_dtype), ctx.num_embeddings)
        return grad_weight, None, None


def embedding_bag_mean(embedding_weight: torch.Tensor, values: torch.Tensor, *, backend: str = "hip",
                       block_rows: int | None = None, block_cols: int | None = None,
                       check_indices: bool = False) -> torch.Tensor:
    """Mean of the table rows named by each bag's non-zero ids (id 0 = padding; an all-padding bag gives zeros).
    ``block_rows`` / ``block_cols`` are TileLang / Triton launch hints, accepted and ignored."""
    del block_rows, block_cols
    weight, ids, _ = _normalize_embedding_bag_mean_inputs(embedding_weight, values)
    _resolve_embedding_bag_mean_backend(weight, ids, backend)
    if torch.is_grad_enabled() and weight.requires_grad:
        return _HipEmbeddingBagMeanFunction.apply(weight, ids, check_indices)
    return hip_embedding_bag_mean_kernel(weight, ids, check_indices=check_indices)


__all__ = [
    "EMBEDDING_BAG_MEAN_BACKENDS",
    "embedding_bag_mean",
    "hip_embedding_bag_mean_backward_kernel",
    "hip_embedding_bag_mean_kernel",
    "resolved_embedding_bag_mean_backend",
]
