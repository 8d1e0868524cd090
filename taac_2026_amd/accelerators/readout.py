"""Readout of the token backbone backed by one gfx950 kernel.

Mirrors what ``PCVRSymbiosis`` does after its blocks (experiments/symbiosis/model.py:215-222, 291, 309, 316-317):
``final_norm`` over the tokens, ``CandidateClsPooler`` (experiments/symbiosis/pooling.py:16-32: cls token | candidate
token | masked mean, then ``RMSNorm(3 * d_model)``) and the classifier ``Linear -> SiLU -> Linear``.
"""

from __future__ import annotations

import torch

from taac_2026_amd import _native
from taac_2026_amd.accelerators.tensor_validation import require_cuda_tensors


def _candidate_readout_training(tokens, cls_index, candidate_index, key_lengths, padding_mask, token_norm_weight,
                                pool_norm_weight, eps, classifier, sigmoid, return_embedding):
    """The readout for tensors that take a gradient: the same expression from differentiable pieces - the HIP RMSNorm
    (forward and backward kernels) over the tokens and over the pooled vector, torch for the masked mean and for the
    classifier's two small products (``CandidateClsPooler.forward``, experiments/symbiosis/pooling.py:24-32, and the
    classifier of experiments/symbiosis/model.py:215-222, as the reference evaluates them under autograd)."""
    from taac_2026_amd.accelerators.normalization import rms_norm

    batch, token_count, _ = tokens.shape
    x = tokens if token_norm_weight is None else rms_norm(tokens, token_norm_weight, eps)
    if padding_mask is not None:
        keep = ~padding_mask
    elif key_lengths is not None:
        keep = torch.arange(token_count, device=tokens.device)[None, :] < key_lengths[:, None]
    else:
        keep = torch.ones(batch, token_count, dtype=torch.bool, device=tokens.device)
    weights = keep.to(torch.float32)
    counts = weights.sum(dim=1, keepdim=True).clamp_min(1.0)
    mean = torch.einsum("btd,bt->bd", x.float(), weights / counts).to(x.dtype)      # masked mean, fp32 accumulation
    cls_summary = x[:, cls_index, :]
    candidate_summary = x[:, candidate_index, :] if candidate_index is not None else torch.zeros_like(cls_summary)
    pooled = torch.cat([cls_summary, candidate_summary, mean], dim=-1)
    if pool_norm_weight is not None:
        pooled = rms_norm(pooled, pool_norm_weight, eps)
    if classifier is None:
        return pooled
    fc1_weight, fc1_bias, fc2_weight, fc2_bias = classifier
    hidden = torch.nn.functional.silu(torch.nn.functional.linear(pooled, fc1_weight, fc1_bias))
    logits = torch.nn.functional.linear(hidden, fc2_weight, fc2_bias).float()
    if sigmoid:
        logits = torch.sigmoid(logits)
    return (logits, pooled) if return_embedding else logits


def candidate_readout(
    tokens: torch.Tensor,
    *,
    cls_index: int,
    candidate_index: int | None = None,
    key_lengths: torch.Tensor | None = None,
    padding_mask: torch.Tensor | None = None,
    token_norm_weight: torch.Tensor | None = None,
    pool_norm_weight: torch.Tensor | None = None,
    eps: float = 1e-6,
    fc1_weight: torch.Tensor | None = None,
    fc1_bias: torch.Tensor | None = None,
    fc2_weight: torch.Tensor | None = None,
    fc2_bias: torch.Tensor | None = None,
    sigmoid: bool = False,
    return_embedding: bool = False,
):
    """``tokens`` (B, T, D) bf16 -> pooled embedding (B, 3D) bf16 and / or classifier output (B, actions) float32.

    Valid tokens of the mean: ``t < key_lengths[b]``, or ``~padding_mask[b, t]`` (True = padding, any pattern), or all.
    ``token_norm_weight`` fuses the per-token RMSNorm in front (``final_norm``), ``pool_norm_weight`` the pooler's
    ``RMSNorm(3D)``. Without ``fc1_weight`` only the embedding is computed. Returns the logits (probabilities with
    ``sigmoid=True``), the embedding, or ``(logits, embedding)`` with ``return_embedding=True``, like
    ``PCVRSymbiosis.forward`` / ``predict``. Tensors that require a gradient take a differentiable route (the HIP norm
    kernels with their backward, torch for the mean and the classifier) instead of the one-kernel inference route.
    """
    name = "hip candidate_readout"
    weights = (token_norm_weight, pool_norm_weight, fc1_weight, fc1_bias, fc2_weight, fc2_bias)
    require_cuda_tensors(name, tokens, key_lengths, padding_mask, *weights)
    if tokens.ndim != 3:
        raise ValueError(f"{name} expects tokens of shape (batch, tokens, d_model)")
    for t in (tokens, *weights):
        if t is not None and t.dtype != torch.bfloat16:
            raise RuntimeError(f"{name} expects bfloat16 tensors, got {t.dtype}")
    if key_lengths is not None and padding_mask is not None:
        raise ValueError(f"{name}: give key_lengths or padding_mask, not both")
    batch, token_count, d_model = tokens.shape
    if not 0 <= int(cls_index) < token_count or (candidate_index is not None and not 0 <= int(candidate_index) < token_count):
        raise ValueError(f"{name}: token index outside the sequence")
    if token_norm_weight is not None and token_norm_weight.shape != (d_model,):
        raise ValueError(f"{name}: token_norm_weight must have shape ({d_model},)")
    if pool_norm_weight is not None and pool_norm_weight.shape != (3 * d_model,):
        raise ValueError(f"{name}: pool_norm_weight must have shape ({3 * d_model},)")
    classifier = fc1_weight is not None
    hidden = actions = 0
    if classifier:
        if fc2_weight is None or fc1_weight.ndim != 2 or fc1_weight.shape[1] != 3 * d_model:
            raise ValueError(f"{name}: the classifier needs fc1_weight (hidden, {3 * d_model}) and fc2_weight (actions, hidden)")
        hidden = fc1_weight.shape[0]
        if fc2_weight.ndim != 2 or fc2_weight.shape[1] != hidden:
            raise ValueError(f"{name}: fc2_weight must have shape (actions, {hidden})")
        actions = fc2_weight.shape[0]
        if (fc1_bias is not None and fc1_bias.shape != (hidden,)) or (fc2_bias is not None and fc2_bias.shape != (actions,)):
            raise ValueError(f"{name}: bias shapes must match the layers")
    elif fc2_weight is not None:
        raise ValueError(f"{name}: fc2_weight without fc1_weight")
    tokens = tokens.contiguous()
    lengths = None if key_lengths is None else key_lengths.to(torch.int32).contiguous()
    if lengths is not None and lengths.shape != (batch,):
        raise ValueError(f"{name}: key_lengths must have shape ({batch},)")
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (tokens, *weights)):
        if padding_mask is not None and (padding_mask.dtype is not torch.bool or padding_mask.shape != (batch, token_count)):
            raise ValueError(f"{name}: padding_mask must be a bool tensor of shape ({batch}, {token_count})")
        return _candidate_readout_training(
            tokens, int(cls_index), None if candidate_index is None else int(candidate_index), lengths, padding_mask,
            token_norm_weight, pool_norm_weight, float(eps),
            (fc1_weight, fc1_bias, fc2_weight, fc2_bias) if classifier else None, bool(sigmoid), bool(return_embedding))
    valid_bits = None
    if padding_mask is not None:
        if padding_mask.dtype is not torch.bool or padding_mask.shape != (batch, token_count):
            raise ValueError(f"{name}: padding_mask must be a bool tensor of shape ({batch}, {token_count})")
        from taac_2026_amd.accelerators.attention import _pack_bits

        valid_bits = _pack_bits((~padding_mask).contiguous())
    want_embedding = return_embedding or not classifier
    embedding = torch.empty(batch, 3 * d_model, dtype=torch.bfloat16, device=tokens.device) if want_embedding else None
    logits = torch.empty(batch, actions, dtype=torch.float32, device=tokens.device) if classifier else None
    contiguous = [None if w is None else w.contiguous() for w in weights]
    library = _native.load_library()
    status = library.taac_candidate_readout_fwd(
        tokens.data_ptr(), _native.ptr(lengths), _native.ptr(valid_bits), batch, token_count, d_model, int(cls_index),
        -1 if candidate_index is None else int(candidate_index), _native.ptr(contiguous[0]), _native.ptr(contiguous[1]),
        float(eps), _native.ptr(contiguous[2]), _native.ptr(contiguous[3]), hidden, _native.ptr(contiguous[4]),
        _native.ptr(contiguous[5]), actions, _native.ptr(embedding), _native.ptr(logits), int(bool(sigmoid)),
        _native.current_stream(tokens.device),
    )
    _native.check(status, "candidate_readout")
    if not classifier:
        return embedding
    return (logits, embedding) if return_embedding else logits


__all__ = ["candidate_readout"]
