"""Dense-layer operators of the backbone block on gfx950 MFMA (bf16 and FP8 e4m3 operands).

These replace the ``nn.Linear`` + elementwise sequences of the reference's block
(experiments/symbiosis/backbone.py:11-68): ``linear`` covers QKV / output / down projections with an optional
fused residual add, ``swiglu_linear`` is the up projection with ``silu(gate) * value`` fused into its epilogue, and
the ``*_fp8`` functions are the per-tensor-scaled e4m3 variants (scale = amax / 448, fp32 accumulation, bf16 out).
Weights use the torch ``nn.Linear`` layout ``[out_features, in_features]``.
"""

from __future__ import annotations

import weakref

import torch

from taac_2026_amd import _native
from taac_2026_amd.accelerators.tensor_validation import require_cuda_tensors, require_inference

FP8_MAX = 448.0


def _as_rows(x: torch.Tensor) -> tuple[torch.Tensor, torch.Size]:
    if x.ndim < 2:
        raise ValueError("linear expects input with at least 2 dimensions")
    rows = x.reshape(-1, x.shape[-1])
    if rows.stride(-1) != 1 or rows.stride(0) % 8 != 0 or rows.data_ptr() % 16 != 0:
        rows = rows.contiguous()
    return rows, x.shape


def _check_16(operator_name: str, *tensors: torch.Tensor | None) -> torch.dtype:
    """All tensors bfloat16, or all float16 (the tiled dense kernel exists for both): returns the common dtype."""
    dtypes = {t.dtype for t in tensors if t is not None}
    if len(dtypes) != 1 or not dtypes <= {torch.bfloat16, torch.float16}:
        raise RuntimeError(f"{operator_name} expects tensors of one 16-bit dtype (bfloat16 or float16), got {sorted(map(str, dtypes))}")
    return next(iter(dtypes))


def _is_f16(*tensors: torch.Tensor | None) -> bool:
    return any(t is not None and t.dtype == torch.float16 for t in tensors)


def _f16_inference_only(operator_name: str, *tensors: torch.Tensor | None) -> None:
    if _needs_grad(*tensors):
        raise RuntimeError(f"{operator_name}: the float16 dense layers are forward-only; train in bfloat16 or call "
                           "them under torch.no_grad()")


def _check_bf16(operator_name: str, *tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and t.dtype != torch.bfloat16:
            raise RuntimeError(f"{operator_name} expects bfloat16 tensors, got {t.dtype}")


def _check_weight(operator_name: str, rows: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None) -> None:
    if weight.ndim != 2:
        raise ValueError(f"{operator_name} weight must be a 2D tensor [out_features, in_features]")
    if rows.shape[-1] != weight.shape[1]:
        raise ValueError(f"last dimension {rows.shape[-1]} does not match weight in_features {weight.shape[1]}")
    if bias is not None and (bias.ndim != 1 or bias.shape[0] != weight.shape[0]):
        raise ValueError(f"{operator_name} bias must have shape ({weight.shape[0]},)")


def _needs_grad(*tensors: torch.Tensor | None) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def linear_wgrad(grad_out: torch.Tensor, inputs: torch.Tensor, *, with_bias: bool = True,
                 dtype: torch.dtype = torch.bfloat16) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Weight and bias gradient of ``y = inputs @ w.T + b``: ``(grad_out.T @ inputs, grad_out.sum(0))`` over the flattened
    rows, fp32 accumulation with a fixed summation order (``taac_linear_wgrad``). Returns tensors of ``dtype``."""
    name = "hip linear_wgrad"
    require_cuda_tensors(name, grad_out, inputs)
    _check_bf16(name, grad_out, inputs)
    dy, _ = _as_rows(grad_out)
    a, _ = _as_rows(inputs)
    if dy.shape[0] != a.shape[0]:
        raise ValueError("linear_wgrad: grad_out and inputs must have the same number of rows")
    if dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("linear_wgrad returns bfloat16 or float32 gradients")
    rows, out_features, in_features = dy.shape[0], dy.shape[1], a.shape[1]
    grad_w = torch.empty(out_features, in_features, dtype=dtype, device=dy.device)
    grad_b = torch.empty(out_features, dtype=dtype, device=dy.device) if with_bias else None
    library = _native.load_library()
    count = int(library.taac_linear_wgrad_workspace_floats(rows, out_features, in_features))
    workspace = torch.empty(max(count, 1), dtype=torch.float32, device=dy.device)
    status = library.taac_linear_wgrad(
        dy.data_ptr(), dy.stride(0), a.data_ptr(), a.stride(0), grad_w.data_ptr(), _native.ptr(grad_b), workspace.data_ptr(),
        workspace.numel(), rows, out_features, in_features, _native.dtype_code(dtype), _native.current_stream(dy.device),
    )
    _native.check(status, "linear_wgrad")
    return grad_w, grad_b


def swiglu_backward(pre_activation: torch.Tensor, grad_hidden: torch.Tensor | None, *, gate_first: bool = True,
                    want_hidden: bool = True) -> tuple[torch.Tensor | None, torch.Tensor | None]:
    """From the up projection ``[.., 2F]`` (gate | value): the gated hidden state ``silu(gate) * value`` and, with
    ``grad_hidden``, the gradient of the up projection ``[.., 2F]`` (``taac_swiglu_bwd``). Returns (hidden, grad)."""
    name = "hip swiglu_backward"
    require_cuda_tensors(name, pre_activation, grad_hidden)
    _check_bf16(name, pre_activation, grad_hidden)
    gu, shape = _as_rows(pre_activation)
    hidden_size = gu.shape[1] // 2
    dh = None
    if grad_hidden is not None:
        dh, _ = _as_rows(grad_hidden)
    hidden = torch.empty(gu.shape[0], hidden_size, dtype=gu.dtype, device=gu.device) if want_hidden else None
    grad = torch.empty_like(gu, memory_format=torch.contiguous_format) if dh is not None else None
    library = _native.load_library()
    status = library.taac_swiglu_bwd(
        gu.data_ptr(), gu.stride(0), _native.ptr(dh), dh.stride(0) if dh is not None else hidden_size, _native.ptr(grad),
        2 * hidden_size, _native.ptr(hidden), hidden_size, gu.shape[0], hidden_size, int(bool(gate_first)),
        _native.current_stream(gu.device),
    )
    _native.check(status, "swiglu_backward")
    return (None if hidden is None else hidden.reshape(*shape[:-1], hidden_size),
            None if grad is None else grad.reshape(*shape[:-1], 2 * hidden_size))


def swiglu_ffn_backward_supported(d_model: int, hidden_size: int) -> bool:
    """Whether ``swiglu_ffn_backward_hidden`` covers these widths (its weight steps must fit the LDS, which bounds F)."""
    return int(_native.load_library().taac_swiglu_ffn_bwd_packed_bytes(int(d_model), int(hidden_size))) >= 0


def swiglu_ffn_backward_hidden(h: torch.Tensor, grad_out: torch.Tensor, up_weight: torch.Tensor,
                               up_bias: torch.Tensor | None, down_weight: torch.Tensor, *,
                               gate_first: bool = True) -> tuple[torch.Tensor, torch.Tensor] | None:
    """The activation part of the feed-forward backward as one kernel (``taac_swiglu_ffn_bwd_hidden``): from the input
    ``h [.., D]`` of the up projection and the gradient ``grad_out [.., D]`` of the feed-forward output, the hidden state
    ``[.., F]`` and the gradient ``[.., 2F]`` of the up projection; the up projection itself and ``grad_out @ down_weight``
    stay in registers. Returns ``None`` for shapes the kernel is not built for (width 128 / 256, F a multiple of 32)."""
    name = "hip swiglu_ffn_backward_hidden"
    require_cuda_tensors(name, h, grad_out, up_weight, up_bias, down_weight)
    _check_bf16(name, h, grad_out, up_weight, up_bias, down_weight)
    rows, shape = _as_rows(h)
    dy, _ = _as_rows(grad_out)
    d_model, hidden_size = down_weight.shape
    if rows.shape != dy.shape or rows.shape[1] != d_model or up_weight.shape != (2 * hidden_size, d_model):
        raise ValueError(f"{name}: expected h and grad_out [.., D], up_weight [2F, D], down_weight [D, F]")
    library = _native.load_library()
    nbytes = int(library.taac_swiglu_ffn_bwd_packed_bytes(d_model, hidden_size))
    if nbytes < 0:
        return None

    def pack() -> torch.Tensor:
        blob = torch.empty(nbytes, dtype=torch.uint8, device=rows.device)
        status = library.taac_swiglu_ffn_bwd_pack_weights(
            up_weight.detach().contiguous().data_ptr(), down_weight.detach().contiguous().data_ptr(), blob.data_ptr(),
            d_model, hidden_size, _native.current_stream(rows.device))
        _native.check(status, "swiglu_ffn_backward_hidden (pack)")
        return blob

    packed = _packed_cache.get((up_weight, down_weight), pack, variant=2)
    hidden = torch.empty(rows.shape[0], hidden_size, dtype=rows.dtype, device=rows.device)
    grad_pre = torch.empty(rows.shape[0], 2 * hidden_size, dtype=rows.dtype, device=rows.device)
    status = library.taac_swiglu_ffn_bwd_hidden(
        rows.data_ptr(), rows.stride(0), dy.data_ptr(), dy.stride(0), packed.data_ptr(), _native.ptr(up_bias),
        hidden.data_ptr(), hidden_size, grad_pre.data_ptr(), 2 * hidden_size, rows.shape[0], d_model, hidden_size,
        int(bool(gate_first)), _native.current_stream(rows.device))
    _native.check(status, "swiglu_ffn_backward_hidden")
    return hidden.reshape(*shape[:-1], hidden_size), grad_pre.reshape(*shape[:-1], 2 * hidden_size)


def _plain_product(rows: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """``F.linear(rows, weight, bias)`` without autograd, by the token-stationary kernel where its shapes allow
    (:func:`norm_linear` without a norm), else by the tiled one."""
    with torch.no_grad():
        if _fused_width(weight.shape[1]) and weight.shape[0] % 64 == 0:
            return norm_linear(rows, weight, bias)
        return linear(rows, weight, bias)


def _input_grad(grad_rows: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``grad_rows @ weight``: a forward-shaped product with the transposed weight."""
    return _plain_product(grad_rows, weight.detach().t().contiguous())


class _NormLinearFunction(torch.autograd.Function):
    """``residual + linear(rmsnorm(x))`` (norm and residual optional) for training: the forward is the inference kernel and
    saves only its inputs; the backward recomputes the normalised rows and runs the input-gradient product, the weight
    gradient and the norm backward as HIP kernels (what torch autograd derives for the reference's nn.Linear layers,
    experiments/symbiosis/backbone.py:24-48)."""

    @staticmethod
    def forward(ctx, x, weight, bias, norm_weight, residual, eps):
        with torch.no_grad():
            out = norm_linear(x, weight, bias, norm_weight=norm_weight, eps=eps, residual=residual)
        ctx.save_for_backward(x, weight, *(() if norm_weight is None else (norm_weight,)))
        ctx.has_norm, ctx.has_bias, ctx.has_residual, ctx.eps = norm_weight is not None, bias is not None, residual is not None, eps
        return out

    @staticmethod
    def backward(ctx, grad_out):
        from taac_2026_amd.accelerators.normalization import hip_rms_norm_backward_kernel, hip_rms_norm_kernel

        x, weight = ctx.saved_tensors[:2]
        norm_weight = ctx.saved_tensors[2] if ctx.has_norm else None
        rows, shape = _as_rows(x)
        rows = rows.contiguous()
        dy, _ = _as_rows(grad_out if grad_out.dtype == torch.bfloat16 else grad_out.to(torch.bfloat16))
        dy = dy.contiguous()
        with torch.no_grad():
            h = hip_rms_norm_kernel(rows, norm_weight, ctx.eps) if ctx.has_norm else rows
            grad_w, grad_b = linear_wgrad(dy, h, with_bias=ctx.has_bias)
            grad_h = _input_grad(dy, weight)
            grad_norm = None
            if ctx.has_norm:
                grad_rows, grad_norm = hip_rms_norm_backward_kernel(rows, norm_weight, grad_h.contiguous(), ctx.eps)
            else:
                grad_rows = grad_h
        return (grad_rows.reshape(shape), grad_w, grad_b, grad_norm, grad_out if ctx.has_residual else None, None)


class _SwigluFfnFunction(torch.autograd.Function):
    """``residual + down(silu(gate) * value)``, ``gate, value = up(rmsnorm(x))``, for training: the forward is the fused
    inference kernel and saves only its inputs; the backward recomputes the up projection and the hidden state
    (experiments/symbiosis/backbone.py:11-21)."""

    @staticmethod
    def forward(ctx, x, up_weight, up_bias, down_weight, down_bias, residual, norm_weight, gate_first, eps):
        with torch.no_grad():
            out = swiglu_ffn(x, up_weight, up_bias, down_weight, down_bias, residual=residual, gate_first=gate_first,
                             norm_weight=norm_weight, eps=eps)
        ctx.save_for_backward(x, up_weight, down_weight, *(t for t in (up_bias, norm_weight) if t is not None))
        ctx.flags = (up_bias is not None, down_bias is not None, residual is not None, norm_weight is not None,
                     bool(gate_first), eps)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        from taac_2026_amd.accelerators.normalization import hip_rms_norm_backward_kernel, hip_rms_norm_kernel

        has_up_bias, has_down_bias, has_residual, has_norm, gate_first, eps = ctx.flags
        saved = list(ctx.saved_tensors)
        x, up_weight, down_weight = saved[:3]
        rest = saved[3:]
        up_bias = rest.pop(0) if has_up_bias else None
        norm_weight = rest.pop(0) if has_norm else None
        rows, shape = _as_rows(x)
        rows = rows.contiguous()
        dy, _ = _as_rows(grad_out if grad_out.dtype == torch.bfloat16 else grad_out.to(torch.bfloat16))
        dy = dy.contiguous()
        with torch.no_grad():
            h = hip_rms_norm_kernel(rows, norm_weight, eps) if has_norm else rows
            fused = swiglu_ffn_backward_hidden(h, dy, up_weight, up_bias, down_weight, gate_first=gate_first)
            if fused is not None:
                hidden, grad_pre = fused
            else:
                pre = _plain_product(h, up_weight.detach(), None if up_bias is None else up_bias.detach())   # [M, 2F]
                grad_hidden = _input_grad(dy, down_weight)                                           # [M, F]
                hidden, grad_pre = swiglu_backward(pre, grad_hidden, gate_first=gate_first)
            grad_down_w, grad_down_b = linear_wgrad(dy, hidden, with_bias=has_down_bias)
            grad_up_w, grad_up_b = linear_wgrad(grad_pre, h, with_bias=has_up_bias)
            grad_h = _input_grad(grad_pre, up_weight)
            grad_norm = None
            if has_norm:
                grad_rows, grad_norm = hip_rms_norm_backward_kernel(rows, norm_weight, grad_h.contiguous(), eps)
            else:
                grad_rows = grad_h
        return (grad_rows.reshape(shape), grad_up_w, grad_up_b, grad_down_w, grad_down_b,
                grad_out if has_residual else None, grad_norm, None, None)


class _SwigluDropoutFfnFunction(torch.autograd.Function):
    """``residual + down(keep / (1 - p) * silu(gate) * value)``, ``gate, value = up(x)``: the feed-forward of the reference's
    blocks in training mode (``down(dropout(silu(gate) * value))``, experiments/symbiosis/backbone.py:11-21) under a keep
    mask ``[.., F]`` of the hidden state drawn by the caller. The hidden state reaches memory here (the mask applies to
    it): up projection with the activation in its epilogue, the mask as an element-wise product, down projection; the
    backward recomputes the up projection and runs the activation backward, both weight gradients and both input
    gradients as HIP kernels."""

    @staticmethod
    def forward(ctx, x, up_weight, up_bias, down_weight, down_bias, residual, keep, scale, gate_first):
        with torch.no_grad():
            hidden = swiglu_linear(x, up_weight, up_bias, gate_first=gate_first)
            dropped = hidden * keep.to(hidden.dtype) * scale
            out = _plain_product(dropped, down_weight, down_bias)
            if residual is not None:
                out = out + residual
        ctx.save_for_backward(x, up_weight, down_weight, dropped, keep, *(() if up_bias is None else (up_bias,)))
        ctx.flags = (up_bias is not None, down_bias is not None, residual is not None, bool(gate_first), float(scale))
        return out

    @staticmethod
    def backward(ctx, grad_out):
        has_up_bias, has_down_bias, has_residual, gate_first, scale = ctx.flags
        x, up_weight, down_weight, dropped, keep, *rest = ctx.saved_tensors
        up_bias = rest[0] if has_up_bias else None
        rows, shape = _as_rows(x)
        rows = rows.contiguous()
        dy, _ = _as_rows(grad_out if grad_out.dtype == torch.bfloat16 else grad_out.to(torch.bfloat16))
        dy = dy.contiguous()
        with torch.no_grad():
            dropped_rows, _ = _as_rows(dropped)
            grad_down_w, grad_down_b = linear_wgrad(dy, dropped_rows.contiguous(), with_bias=has_down_bias)
            grad_hidden = _input_grad(dy, down_weight) * (_as_rows(keep)[0].to(dy.dtype) * scale)
            pre = _plain_product(rows, up_weight.detach(), None if up_bias is None else up_bias.detach())
            _, grad_pre = swiglu_backward(pre, grad_hidden.contiguous(), gate_first=gate_first, want_hidden=False)
            grad_up_w, grad_up_b = linear_wgrad(grad_pre, rows, with_bias=has_up_bias)
            grad_rows = _input_grad(grad_pre, up_weight)
        return (grad_rows.reshape(shape), grad_up_w, grad_up_b, grad_down_w, grad_down_b,
                grad_out if has_residual else None, None, None, None)


def swiglu_ffn_dropout(x: torch.Tensor, up_weight: torch.Tensor, up_bias: torch.Tensor | None, down_weight: torch.Tensor,
                       down_bias: torch.Tensor | None, *, dropout_p: float, residual: torch.Tensor | None = None,
                       gate_first: bool = True, keep_mask: torch.Tensor | None = None) -> torch.Tensor:
    """The reference's feed-forward in training mode: ``residual + down(dropout(silu(gate) * value))``. ``keep_mask``
    (bool or uint8 ``[.., F]``, non-zero = keep) fixes the dropped units; without it one is drawn from torch's generator
    (``rand >= p``). Differentiable; bf16 tensors."""
    name = "hip swiglu_ffn_dropout"
    require_cuda_tensors(name, x, up_weight, up_bias, down_weight, down_bias, residual, keep_mask)
    _check_bf16(name, x, up_weight, up_bias, down_weight, down_bias, residual)
    if not 0.0 <= dropout_p < 1.0:
        raise ValueError(f"{name}: dropout_p must be in [0, 1)")
    hidden_shape = (*x.shape[:-1], down_weight.shape[1])
    if keep_mask is None:
        keep_mask = torch.rand(hidden_shape, device=x.device) >= dropout_p
    elif tuple(keep_mask.shape) != hidden_shape:
        raise ValueError(f"{name}: keep_mask must have shape {hidden_shape}")
    return _SwigluDropoutFfnFunction.apply(x, up_weight, up_bias, down_weight, down_bias, residual, keep_mask,
                                           1.0 / (1.0 - dropout_p), bool(gate_first))


def linear(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None = None,
    *,
    residual: torch.Tensor | None = None,
) -> torch.Tensor:
    """``F.linear(x, weight, bias)`` (+ ``residual``) on bfloat16 or float16 tensors with fp32 accumulation (float16:
    forward only)."""
    name = "hip linear"
    require_cuda_tensors(name, x, weight, bias, residual)
    if _is_f16(x, weight, bias, residual):
        _f16_inference_only(name, x, weight, bias, residual)
    elif _needs_grad(x, weight, bias, residual):
        return _NormLinearFunction.apply(x, weight, bias, None, residual, 1e-6)
    dtype = _check_16(name, x, weight, bias, residual)
    rows, shape = _as_rows(x)
    _check_weight(name, rows, weight, bias)
    weight = weight.contiguous()
    out_features = weight.shape[0]
    out = torch.empty((rows.shape[0], out_features), dtype=x.dtype, device=x.device)
    res_rows = None
    if residual is not None:
        if residual.shape != (*shape[:-1], out_features):
            raise ValueError("linear residual must have the shape of the output")
        res_rows = residual.reshape(-1, out_features).contiguous()
    library = _native.load_library()
    entry = library.taac_linear_f16 if dtype == torch.float16 else library.taac_linear_bf16
    status = entry(
        rows.data_ptr(), rows.stride(0), weight.data_ptr(), _native.ptr(bias), _native.ptr(res_rows), out.data_ptr(),
        out_features, rows.shape[0], out_features, weight.shape[1],
        _native.EPI_RESIDUAL if res_rows is not None else _native.EPI_NONE, 1, _native.current_stream(x.device),
    )
    _native.check(status, "linear")
    return out.reshape(*shape[:-1], out_features)


def swiglu_linear(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None = None,
    *,
    gate_first: bool = True,
) -> torch.Tensor:
    """``g, u = F.linear(x, weight, bias).chunk(2, -1); silu(g) * u`` (``g * silu(u)`` if not ``gate_first``)."""
    name = "hip swiglu_linear"
    require_cuda_tensors(name, x, weight, bias)
    require_inference(name, x, weight, bias)
    dtype = _check_16(name, x, weight, bias)
    rows, shape = _as_rows(x)
    _check_weight(name, rows, weight, bias)
    if weight.shape[0] % 2 != 0:
        raise ValueError("swiglu_linear weight must have an even number of output features")
    weight = weight.contiguous()
    hidden = weight.shape[0] // 2
    out = torch.empty((rows.shape[0], hidden), dtype=x.dtype, device=x.device)
    library = _native.load_library()
    entry = library.taac_linear_f16 if dtype == torch.float16 else library.taac_linear_bf16
    status = entry(
        rows.data_ptr(), rows.stride(0), weight.data_ptr(), _native.ptr(bias), None, out.data_ptr(), hidden,
        rows.shape[0], weight.shape[0], weight.shape[1], _native.EPI_SWIGLU, int(bool(gate_first)),
        _native.current_stream(x.device),
    )
    _native.check(status, "swiglu_linear")
    return out.reshape(*shape[:-1], hidden)


def _fused_width(d: int) -> bool:
    return d in (128, 256)


class _PackedWeightCache:
    """Fragment-ordered copies of weight tensors for the token-stationary kernels, keyed by tensor identity and
    version counter so that an in-place update of a weight is repacked. Bounded; oldest entries are dropped."""

    def __init__(self, capacity: int = 128) -> None:
        self._entries: dict[tuple, tuple[tuple, torch.Tensor]] = {}
        self._capacity = capacity

    def get(self, tensors: tuple[torch.Tensor, ...], pack, variant: int = 0) -> torch.Tensor:
        key = tuple(id(t) for t in tensors) + (variant,)
        stamp = tuple((weakref.ref(t), t._version, t.data_ptr()) for t in tensors)
        hit = self._entries.get(key)
        if hit is not None:
            old_stamp, packed = hit
            if all(o[0]() is t and o[1] == t._version and o[2] == t.data_ptr() for o, t in zip(old_stamp, tensors)):
                return packed
        packed = pack()
        if len(self._entries) >= self._capacity:
            self._entries.pop(next(iter(self._entries)))
        self._entries[key] = (stamp, packed)
        return packed

    def clear(self) -> None:
        self._entries.clear()


_packed_cache = _PackedWeightCache()


def clear_packed_weight_cache() -> None:
    _packed_cache.clear()


def ffn_activation_fold_supported(d_model: int, hidden_size: int) -> bool:
    """Whether the fused feed-forward kernels take the constants of ``silu(g) * u`` from the packed up projection at
    this shape (``pack_ffn_weights(fold_activation=True)``)."""
    return bool(_native.load_library().taac_ffn_activation_fold_supported(int(d_model), int(hidden_size)))


def pack_ffn_weights(up_weight: torch.Tensor, down_weight: torch.Tensor, *, gate_first: bool = True,
                     norm_weight: torch.Tensor | None = None, fold_activation: bool = False) -> torch.Tensor:
    """Fragment-ordered blob of ``(up_weight [2F, D], down_weight [D, F])`` for ``swiglu_ffn`` (uint8 tensor).

    The blob depends on ``gate_first`` (which half of ``up_weight`` goes through SiLU): pass the same value to
    ``swiglu_ffn``. ``norm_weight`` ``[D]``: the weight of the RMSNorm in front of the up projection, folded into the
    blob (``taac_ffn_pack_weights_norm``; the kernels are then called with ``TAAC_FOLDED_NORM``). ``fold_activation``:
    the up projection also carries the constants of the gate's activation (``taac_ffn_pack_weights_folded``; the
    kernels are then called with ``TAAC_FOLDED_ACTIVATION``)."""
    library = _native.load_library()
    d_model, hidden = down_weight.shape
    nbytes = library.taac_ffn_packed_bytes(d_model, hidden)
    if nbytes < 0:
        raise RuntimeError(f"pack_ffn_weights: unsupported shape D={d_model}, F={hidden}")
    up_weight, down_weight = up_weight.contiguous(), down_weight.contiguous()
    packed = torch.empty(nbytes, dtype=torch.uint8, device=up_weight.device)
    if norm_weight is not None and norm_weight.shape != (d_model,):
        raise ValueError("rms_norm weight must be 1D and match the normalized dimension")
    if fold_activation:
        norm = norm_weight.contiguous() if norm_weight is not None else None
        status = library.taac_ffn_pack_weights_folded(up_weight.data_ptr(), down_weight.data_ptr(), _native.ptr(norm),
                                                      packed.data_ptr(), d_model, hidden, int(bool(gate_first)), 1,
                                                      _native.current_stream(up_weight.device))
    elif norm_weight is not None:
        status = library.taac_ffn_pack_weights_norm(up_weight.data_ptr(), down_weight.data_ptr(),
                                                    norm_weight.contiguous().data_ptr(), packed.data_ptr(), d_model, hidden,
                                                    int(bool(gate_first)), _native.current_stream(up_weight.device))
    else:
        status = library.taac_ffn_pack_weights(up_weight.data_ptr(), down_weight.data_ptr(), packed.data_ptr(), d_model,
                                               hidden, int(bool(gate_first)),
                                               _native.current_stream(up_weight.device))
    _native.check(status, "pack_ffn_weights")
    return packed


def _packed_ffn(up_weight: torch.Tensor, down_weight: torch.Tensor, gate_first: bool, norm_weight: torch.Tensor | None,
                fold_activation: bool = False):
    """Cached feed-forward blob, with the weight of the norm in front of it folded in when there is one (and, with
    ``fold_activation``, the constants of the gate's activation)."""
    variant = int(bool(gate_first)) + (8 if fold_activation else 0)
    if norm_weight is None:
        return _packed_cache.get((up_weight, down_weight),
                                 lambda: pack_ffn_weights(up_weight, down_weight, gate_first=gate_first,
                                                          fold_activation=fold_activation),
                                 variant=variant)
    return _packed_cache.get((up_weight, down_weight, norm_weight),
                             lambda: pack_ffn_weights(up_weight, down_weight, gate_first=gate_first, norm_weight=norm_weight,
                                                      fold_activation=fold_activation),
                             variant=4 + variant)


def _fold_choice(name: str, fold_activation: bool | None, d_model: int, hidden: int) -> bool:
    """``fold_activation`` of the fused feed-forward wrappers: None takes the folded blob wherever the kernels accept it."""
    supported = ffn_activation_fold_supported(d_model, hidden)
    if fold_activation and not supported:
        raise RuntimeError(f"{name}: the kernels do not take the activation's constants from the blob at D={d_model}, F={hidden}")
    return supported if fold_activation is None else bool(fold_activation)


def _folded_flags(norm_weight: torch.Tensor | None, fold_activation: bool) -> int:
    return (_native.FOLDED_NORM if norm_weight is not None else 0) | (_native.FOLDED_ACTIVATION if fold_activation else 0)


def pack_linear_weight(weight: torch.Tensor, norm_weight: torch.Tensor | None = None) -> torch.Tensor:
    """Fragment-ordered blob of ``weight [N, K]`` for ``norm_linear`` (uint8 tensor). ``norm_weight`` ``[K]``: the weight
    of the RMSNorm in front of the layer, folded into the blob (``taac_linear_pack_weights_norm``); the kernel is then
    called with ``norm_folded = 1`` and applies only the norm's per-token factor, to its accumulators."""
    library = _native.load_library()
    out_features, in_features = weight.shape
    nbytes = library.taac_linear_packed_bytes(out_features, in_features)
    if nbytes < 0:
        raise RuntimeError(f"pack_linear_weight: unsupported shape N={out_features}, K={in_features}")
    weight = weight.contiguous()
    packed = torch.empty(nbytes, dtype=torch.uint8, device=weight.device)
    if norm_weight is not None:
        if norm_weight.shape != (in_features,):
            raise ValueError("rms_norm weight must be 1D and match the normalized dimension")
        status = library.taac_linear_pack_weights_norm(weight.data_ptr(), norm_weight.contiguous().data_ptr(),
                                                       packed.data_ptr(), out_features, in_features,
                                                       _native.current_stream(weight.device))
    else:
        status = library.taac_linear_pack_weights(weight.data_ptr(), packed.data_ptr(), out_features, in_features,
                                                  _native.current_stream(weight.device))
    _native.check(status, "pack_linear_weight")
    return packed


def _packed_linear(weight: torch.Tensor, norm_weight: torch.Tensor | None) -> torch.Tensor:
    """Cached blob of a layer, with the weight of the norm in front of it folded in when there is one."""
    if norm_weight is None:
        return _packed_cache.get((weight,), lambda: pack_linear_weight(weight))
    return _packed_cache.get((weight, norm_weight), lambda: pack_linear_weight(weight, norm_weight), variant=3)


def valid_rows(key_lengths: torch.Tensor | None, tokens: int, *,
               padding_mask: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """Row index of the valid tokens of a padded ``[B, tokens, ...]`` batch: token ``t`` of sample ``b`` is valid iff
    ``t < key_lengths[b]``, or - for padding that is not a prefix - iff ``not padding_mask[b, t]`` (bool ``[B, tokens]``,
    True = padding). Returns ``(rows, n_rows)`` with ``rows[:n_rows] = b * tokens + t`` in increasing order, both int32
    on the device (no host synchronisation). ``rows[B * tokens : B * tokens + B + 1]`` holds the per-sample offsets.
    Pass the pair as ``token_rows=`` to :func:`norm_linear` / :func:`swiglu_ffn` / :func:`attention_out_ffn` to skip the
    padded positions."""
    name = "hip valid_rows"
    if (key_lengths is None) == (padding_mask is None):
        raise ValueError(f"{name}: give key_lengths or padding_mask")
    require_cuda_tensors(name, key_lengths, padding_mask)
    library = _native.load_library()
    if padding_mask is not None:
        if padding_mask.dtype is not torch.bool or padding_mask.ndim != 2 or padding_mask.shape[1] != int(tokens):
            raise ValueError(f"{name}: padding_mask must be a bool tensor of shape (batch, {int(tokens)})")
        from taac_2026_amd.accelerators.attention import _pack_bits

        batch = padding_mask.shape[0]
        bits = _pack_bits((~padding_mask).contiguous())
        rows = torch.empty(batch * int(tokens) + batch + 1, dtype=torch.int32, device=padding_mask.device)
        count = torch.empty(1, dtype=torch.int32, device=padding_mask.device)
        status = library.taac_valid_rows_from_bits(bits.data_ptr(), batch, int(tokens), rows.data_ptr(), count.data_ptr(),
                                                   _native.current_stream(padding_mask.device))
        _native.check(status, "valid_rows")
        return rows, count
    lengths = key_lengths.to(torch.int32).contiguous()
    batch = lengths.numel()
    rows = torch.empty(batch * int(tokens) + batch + 1, dtype=torch.int32, device=lengths.device)
    count = torch.empty(1, dtype=torch.int32, device=lengths.device)
    status = library.taac_valid_rows(lengths.data_ptr(), batch, int(tokens), rows.data_ptr(), count.data_ptr(),
                                     _native.current_stream(lengths.device))
    _native.check(status, "valid_rows")
    return rows, count


def front_rows(token_rows: tuple[torch.Tensor, torch.Tensor], batch: int, tokens: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Second index for the layout in which every sample's valid tokens sit at the front of its ``tokens`` rows, in
    their original order: ``(front, lengths)`` with ``front[i] = b * tokens + rank`` for token ``i`` of
    ``token_rows`` and ``lengths[b]`` = the sample's number of valid tokens (int32, on the device). A projection called
    with ``token_rows=(front, count), input_rows=rows`` writes that layout, in which scattered padding has become
    prefix padding (``key_lengths=lengths`` for the attention call); ``token_rows=(rows, count), input_rows=front``
    reads it back."""
    name = "hip front_rows"
    rows, count = token_rows
    require_cuda_tensors(name, rows, count)
    if rows.dtype != torch.int32 or rows.numel() < batch * tokens + batch + 1 or not rows.is_contiguous():
        raise ValueError(f"{name}: token_rows must be the index returned by valid_rows for (batch, tokens)")
    front = torch.empty(max(1, batch * tokens), dtype=torch.int32, device=rows.device)
    lengths = torch.empty(batch, dtype=torch.int32, device=rows.device)
    library = _native.load_library()
    status = library.taac_front_rows(rows.data_ptr(), count.data_ptr(), int(batch), int(tokens), front.data_ptr(),
                                     lengths.data_ptr(), _native.current_stream(rows.device))
    _native.check(status, "front_rows")
    return front, lengths


def _input_rows(name: str, input_rows: torch.Tensor | None, index: torch.Tensor | None, rows: torch.Tensor):
    if input_rows is None:
        return None
    if index is None:
        raise ValueError(f"{name}: input_rows needs token_rows")
    require_cuda_tensors(name, input_rows)
    if input_rows.dtype != torch.int32 or not input_rows.is_contiguous() or input_rows.numel() < rows.shape[0]:
        raise ValueError(f"{name}: input_rows must be a contiguous int32 index that covers the {rows.shape[0]} rows of the input")
    return input_rows


def _output_rows(name: str, out: torch.Tensor | None, shape: tuple[int, int], sparse: bool, like: torch.Tensor):
    if out is None:
        return (torch.zeros if sparse else torch.empty)(shape, dtype=like.dtype, device=like.device)
    require_cuda_tensors(name, like, out)
    if out.dtype != like.dtype or out.numel() != shape[0] * shape[1] or out.shape[-1] != shape[1] or not out.is_contiguous():
        raise ValueError(f"{name}: out must be a contiguous {like.dtype} tensor with {shape[0]} rows of {shape[1]}")
    return out.view(shape)


def _token_rows(name: str, token_rows, rows: torch.Tensor):
    if token_rows is None:
        return None, None
    index, count = token_rows
    require_cuda_tensors(name, index, count)
    if index.dtype != torch.int32 or count.dtype != torch.int32 or count.numel() != 1 or not index.is_contiguous():
        raise ValueError(f"{name}: token_rows must be (int32 row index, int32 scalar count) as returned by valid_rows")
    if index.numel() < rows.shape[0]:
        raise ValueError(f"{name}: the row index must cover the {rows.shape[0]} rows of the input")
    return index, count


def swiglu_ffn(
    x: torch.Tensor,
    up_weight: torch.Tensor,
    up_bias: torch.Tensor | None,
    down_weight: torch.Tensor,
    down_bias: torch.Tensor | None,
    *,
    residual: torch.Tensor | None = None,
    gate_first: bool = True,
    norm_weight: torch.Tensor | None = None,
    eps: float = 1e-6,
    token_rows: tuple[torch.Tensor, torch.Tensor] | None = None,
    out: torch.Tensor | None = None,
    fold_activation: bool | None = None,
) -> torch.Tensor:
    """``residual + down(silu(gate) * value)`` with ``gate, value = up(rmsnorm(x)).chunk(2, -1)``.

    ``fold_activation``: whether the packed up projection carries the constants of the gate's activation (one multiplication less per
    hidden unit in the kernel; each weight is still rounded once); None takes that form wherever the kernels accept it.

    ``norm_weight`` (optional) fuses the pre-FFN RMSNorm; ``residual`` (optional) the residual add. For model widths
    128 / 256 with a hidden size that is a multiple of 32 the whole expression is ONE kernel
    (``taac_swiglu_ffn_fwd``: the projection and the gated hidden state stay in registers); other shapes run
    norm -> up(+SiLU-gate) -> down(+residual) as separate kernels.

    ``token_rows`` (fused shapes only): ``(rows, n_rows)`` from :func:`valid_rows`; only those rows of the flattened
    input are processed, the other rows of the result are zeros. ``out`` (fused shapes only): a contiguous bf16 tensor
    of the result's shape to write into (rows outside ``token_rows`` keep their content); it may be ``residual``.
    """
    name = "hip swiglu_ffn"
    require_cuda_tensors(name, x, up_weight, up_bias, down_weight, down_bias, residual, norm_weight)
    if _is_f16(x, up_weight, down_weight):
        _f16_inference_only(name, x, up_weight, up_bias, down_weight, down_bias, residual, norm_weight)
    elif _needs_grad(x, up_weight, up_bias, down_weight, down_bias, residual, norm_weight):
        if token_rows is not None or out is not None:
            raise RuntimeError("hip swiglu_ffn: token_rows / out belong to the inference route; call it under "
                               "torch.no_grad() or pass dense tensors when a gradient is needed")
        return _SwigluFfnFunction.apply(x, up_weight, up_bias, down_weight, down_bias, residual, norm_weight,
                                        bool(gate_first), float(eps))
    half = _check_16(name, x, up_weight, up_bias, down_weight, down_bias, residual, norm_weight) == torch.float16
    rows, shape = _as_rows(x)
    _check_weight(name, rows, up_weight, up_bias)
    d_model, hidden = rows.shape[1], up_weight.shape[0] // 2
    if up_weight.shape[0] % 2 != 0 or down_weight.shape != (d_model, hidden):
        raise ValueError("swiglu_ffn expects up_weight [2F, D] and down_weight [D, F]")
    if residual is not None and residual.shape != shape:
        raise ValueError("swiglu_ffn residual must have the shape of the input")
    if half or not (_fused_width(d_model) and hidden % 32 == 0):  # float16: the tiled kernels, layer by layer
        if token_rows is not None or out is not None:
            raise RuntimeError("swiglu_ffn: token_rows / out need a fused shape (width 128 / 256, hidden size a multiple of 32)")
        h = rows
        if norm_weight is not None:
            from taac_2026_amd.accelerators.normalization import rms_norm

            h = rms_norm(rows, norm_weight, eps)
        gated = swiglu_linear(h, up_weight, up_bias, gate_first=gate_first)
        res_rows = residual.reshape(-1, d_model) if residual is not None else None
        return linear(gated, down_weight, down_bias, residual=res_rows).reshape(shape)
    fold = _fold_choice(name, fold_activation, d_model, hidden)
    packed = _packed_ffn(up_weight, down_weight, gate_first, norm_weight, fold)
    res_rows = None
    if residual is not None:
        res_rows = residual.reshape(-1, d_model)
        if res_rows.stride(-1) != 1 or res_rows.stride(0) % 8 != 0:
            res_rows = res_rows.contiguous()
    index, count = _token_rows(name, token_rows, rows)
    out = _output_rows(name, out, (rows.shape[0], d_model), index is not None, x)
    library = _native.load_library()
    status = library.taac_swiglu_ffn_fwd(
        rows.data_ptr(), rows.stride(0), _native.ptr(norm_weight), float(eps), None,
        _native.ptr(up_bias), None, _native.ptr(down_bias), packed.data_ptr(), _native.ptr(res_rows),
        res_rows.stride(0) if res_rows is not None else d_model, out.data_ptr(), d_model, rows.shape[0], d_model,
        hidden, int(bool(gate_first)), _native.ptr(index), _native.ptr(count), _folded_flags(norm_weight, fold),
        _native.current_stream(x.device),
    )
    _native.check(status, "swiglu_ffn")
    return out.reshape(shape)


def pack_mlp_weights(fc1_weight: torch.Tensor, fc2_weight: torch.Tensor) -> torch.Tensor:
    """Fragment-ordered blob of ``(fc1_weight [F, D], fc2_weight [D, F])`` for :func:`silu_mlp` (uint8 tensor)."""
    library = _native.load_library()
    d_model, hidden = fc2_weight.shape
    nbytes = library.taac_silu_mlp_packed_bytes(d_model, hidden)
    if nbytes < 0:
        raise RuntimeError(f"pack_mlp_weights: unsupported shape D={d_model}, F={hidden}")
    fc1_weight, fc2_weight = fc1_weight.contiguous(), fc2_weight.contiguous()
    packed = torch.empty(nbytes, dtype=torch.uint8, device=fc1_weight.device)
    status = library.taac_silu_mlp_pack_weights(fc1_weight.data_ptr(), fc2_weight.data_ptr(), packed.data_ptr(), d_model,
                                                hidden, _native.current_stream(fc1_weight.device))
    _native.check(status, "pack_mlp_weights")
    return packed


def silu_mlp(
    x: torch.Tensor,
    fc1_weight: torch.Tensor,
    fc1_bias: torch.Tensor | None,
    fc2_weight: torch.Tensor,
    fc2_bias: torch.Tensor | None,
    *,
    residual: torch.Tensor | None = None,
    norm_weight: torch.Tensor | None = None,
    eps: float = 1e-6,
    token_rows: tuple[torch.Tensor, torch.Tensor] | None = None,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """``residual + fc2(silu(fc1(rmsnorm(x))))`` (norm and residual optional): OneTrans' feed-forward
    (experiments/onetrans/model.py:33-44) in eval mode. For model widths 128 / 256 with a hidden size that is a multiple
    of 32, under ``torch.no_grad()``, the whole expression is ONE kernel (``taac_silu_mlp_fwd``: the hidden state stays in
    registers); other shapes, and tensors that take a gradient, run the two dense layers as kernels of their own with
    the activation between them. ``token_rows`` / ``out`` (fused route only) as in :func:`swiglu_ffn`."""
    name = "hip silu_mlp"
    tensors = (x, fc1_weight, fc1_bias, fc2_weight, fc2_bias, residual, norm_weight)
    require_cuda_tensors(name, *tensors)
    hidden, d_model = fc1_weight.shape
    if fc2_weight.shape != (d_model, hidden) or x.shape[-1] != d_model:
        raise ValueError("silu_mlp expects fc1_weight [F, D], fc2_weight [D, F] and input rows of D features")
    if residual is not None and residual.shape != x.shape:
        raise ValueError("silu_mlp residual must have the shape of the input")
    needs_grad = _needs_grad(*tensors)
    if needs_grad or _is_f16(x, fc1_weight) or not (_fused_width(d_model) and hidden % 32 == 0):
        if token_rows is not None or out is not None:
            raise RuntimeError("silu_mlp: token_rows / out belong to the fused inference route (width 128 / 256, hidden "
                               "size a multiple of 32, no gradient)")
        h = x
        if norm_weight is not None:
            from taac_2026_amd.accelerators.normalization import rms_norm

            h = rms_norm(x, norm_weight, eps)
        return linear(torch.nn.functional.silu(linear(h, fc1_weight, fc1_bias)), fc2_weight, fc2_bias, residual=residual)
    _check_bf16(name, *tensors)
    rows, shape = _as_rows(x)
    packed = _packed_cache.get((fc1_weight, fc2_weight), lambda: pack_mlp_weights(fc1_weight, fc2_weight), variant=2)
    res_rows = None
    if residual is not None:
        res_rows = residual.reshape(-1, d_model)
        if res_rows.stride(-1) != 1 or res_rows.stride(0) % 8 != 0:
            res_rows = res_rows.contiguous()
    index, count = _token_rows(name, token_rows, rows)
    out = _output_rows(name, out, (rows.shape[0], d_model), index is not None, x)
    library = _native.load_library()
    status = library.taac_silu_mlp_fwd(
        rows.data_ptr(), rows.stride(0), _native.ptr(norm_weight), float(eps), _native.ptr(fc1_bias), _native.ptr(fc2_bias),
        packed.data_ptr(), _native.ptr(res_rows), res_rows.stride(0) if res_rows is not None else d_model, out.data_ptr(),
        d_model, rows.shape[0], d_model, hidden, _native.ptr(index), _native.ptr(count), _native.current_stream(x.device),
    )
    _native.check(status, "silu_mlp")
    return out.reshape(shape)


def attention_out_ffn(
    attn: torch.Tensor,
    out_weight: torch.Tensor,
    out_bias: torch.Tensor | None,
    residual: torch.Tensor,
    up_weight: torch.Tensor,
    up_bias: torch.Tensor | None,
    down_weight: torch.Tensor,
    down_bias: torch.Tensor | None,
    *,
    norm_weight: torch.Tensor | None = None,
    eps: float = 1e-6,
    token_rows: tuple[torch.Tensor, torch.Tensor] | None = None,
    input_rows: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
    update_gate: torch.Tensor | None = None,
    fold_activation: bool | None = None,
) -> torch.Tensor:
    """Second half of a ``UnifiedInteractionBlock`` (experiments/symbiosis/backbone.py:47, 64-67) as ONE kernel:
    ``x1 = residual + F.linear(attn, out_weight, out_bias)`` then ``x1 + down(silu(gate) * value)`` with
    ``gate, value = up(rmsnorm(x1)).chunk(2, -1)``. ``x1`` never reaches memory. Model width 128 / 256 and a hidden
    size that is a multiple of 32 only (``taac_attn_out_ffn_fwd``); ``token_rows`` / ``out`` as in :func:`swiglu_ffn`
    (``out`` may be ``residual``). ``input_rows`` (with ``token_rows``): the row of ``attn`` that holds each token when
    ``attn`` is laid out differently from ``residual`` / ``out`` (:func:`front_rows`).

    ``update_gate`` (shape of ``residual``): the second half of a ``TokenFormerBlock`` (experiments/tokenformer/
    model.py:209-214) instead - ``x1 = residual + sigmoid(update_gate) * F.linear(attn, out_weight, out_bias)``, with
    ``update_gate`` the output of the block's ``nlir_gate`` layer before the sigmoid (``taac_attn_out_gate_ffn_fwd``).
    ``fold_activation`` as in :func:`swiglu_ffn` (the kernel with an update gate takes the plain blob)."""
    name = "hip attention_out_ffn"
    tensors = (attn, out_weight, out_bias, residual, up_weight, up_bias, down_weight, down_bias, norm_weight, update_gate)
    require_cuda_tensors(name, *tensors)
    require_inference(name, *tensors)
    _check_bf16(name, *tensors)
    rows, shape = _as_rows(attn)
    _check_weight(name, rows, out_weight, out_bias)
    _check_weight(name, rows, up_weight, up_bias)
    d_model, hidden = rows.shape[1], up_weight.shape[0] // 2
    if out_weight.shape != (d_model, d_model) or up_weight.shape[0] % 2 != 0 or down_weight.shape != (d_model, hidden):
        raise ValueError("attention_out_ffn expects out_weight [D, D], up_weight [2F, D] and down_weight [D, F]")
    if residual.shape != shape:
        raise ValueError("attention_out_ffn residual must have the shape of the attention output")
    if not (_fused_width(d_model) and hidden % 32 == 0):
        raise RuntimeError("attention_out_ffn: needs model width 128 / 256 and a hidden size that is a multiple of 32")
    packed_out = _packed_cache.get((out_weight,), lambda: pack_linear_weight(out_weight))
    if update_gate is not None and fold_activation:
        raise RuntimeError("attention_out_ffn: the kernel with an update gate takes the plain blob (fold_activation=False)")
    fold = update_gate is None and _fold_choice("attention_out_ffn", fold_activation, d_model, hidden)
    packed_ffn = _packed_ffn(up_weight, down_weight, True, norm_weight, fold)
    res_rows = residual.reshape(-1, d_model)
    if res_rows.stride(-1) != 1 or res_rows.stride(0) % 8 != 0:
        res_rows = res_rows.contiguous()
    index, count = _token_rows(name, token_rows, rows)
    out = _output_rows(name, out, (rows.shape[0], d_model), index is not None, attn)
    library = _native.load_library()
    if update_gate is not None:
        if update_gate.shape != shape:
            raise ValueError("attention_out_ffn update_gate must have the shape of the attention output")
        gate_rows = update_gate.reshape(-1, d_model)
        if gate_rows.stride(-1) != 1 or gate_rows.stride(0) % 8 != 0:
            gate_rows = gate_rows.contiguous()
        status = library.taac_attn_out_gate_ffn_fwd(
            rows.data_ptr(), rows.stride(0), _native.ptr(out_bias), packed_out.data_ptr(), gate_rows.data_ptr(),
            gate_rows.stride(0), res_rows.data_ptr(), res_rows.stride(0), _native.ptr(norm_weight), float(eps),
            _native.ptr(up_bias), _native.ptr(down_bias), packed_ffn.data_ptr(), out.data_ptr(), d_model, rows.shape[0],
            d_model, hidden, _native.ptr(index), _native.ptr(count),
            _native.ptr(_input_rows(name, input_rows, index, rows)), int(norm_weight is not None),
            _native.current_stream(attn.device),
        )
        _native.check(status, "attention_out_ffn")
        return out.reshape(shape)
    status = library.taac_attn_out_ffn_fwd(
        rows.data_ptr(), rows.stride(0), _native.ptr(out_bias), packed_out.data_ptr(), res_rows.data_ptr(),
        res_rows.stride(0), _native.ptr(norm_weight), float(eps), _native.ptr(up_bias), _native.ptr(down_bias),
        packed_ffn.data_ptr(), out.data_ptr(), d_model, rows.shape[0], d_model, hidden, _native.ptr(index),
        _native.ptr(count), _native.ptr(_input_rows(name, input_rows, index, rows)), _folded_flags(norm_weight, fold),
        _native.current_stream(attn.device),
    )
    _native.check(status, "attention_out_ffn")
    return out.reshape(shape)


def norm_linear(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None = None,
    *,
    norm_weight: torch.Tensor | None = None,
    eps: float = 1e-6,
    residual: torch.Tensor | None = None,
    token_rows: tuple[torch.Tensor, torch.Tensor] | None = None,
    input_rows: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """``residual + F.linear(rmsnorm(x, norm_weight, eps), weight, bias)`` (norm and residual optional) as one
    kernel when ``in_features`` is 128 / 256 and ``out_features`` a multiple of 64; otherwise composed from the
    stand-alone kernels. ``input_rows`` (with ``token_rows``, fused shapes): the row of ``x`` that holds each token when
    ``x`` is laid out differently from ``residual`` / ``out`` (:func:`front_rows`)."""
    name = "hip norm_linear"
    require_cuda_tensors(name, x, weight, bias, residual, norm_weight)
    if _is_f16(x, weight):
        _f16_inference_only(name, x, weight, bias, residual, norm_weight)
    elif _needs_grad(x, weight, bias, residual, norm_weight):
        if token_rows is not None or input_rows is not None or out is not None:
            raise RuntimeError("hip norm_linear: token_rows / input_rows / out belong to the inference route; "
                               "call it under torch.no_grad() or pass dense tensors when a gradient is needed")
        return _NormLinearFunction.apply(x, weight, bias, norm_weight, residual, float(eps))
    half = _check_16(name, x, weight, bias, residual, norm_weight) == torch.float16
    rows, shape = _as_rows(x)
    _check_weight(name, rows, weight, bias)
    in_features, out_features = weight.shape[1], weight.shape[0]
    if half or not (_fused_width(in_features) and out_features % 64 == 0):  # float16: the tiled kernel
        if token_rows is not None or out is not None or input_rows is not None:
            raise RuntimeError("norm_linear: token_rows / out need a fused shape (K 128 / 256, N a multiple of 64)")
        h = rows
        if norm_weight is not None:
            from taac_2026_amd.accelerators.normalization import rms_norm

            h = rms_norm(rows, norm_weight, eps)
        res = residual.reshape(-1, out_features) if residual is not None else None
        return linear(h, weight, bias, residual=res).reshape(*shape[:-1], out_features)
    packed = _packed_linear(weight, norm_weight)
    res_rows = None
    if residual is not None:
        if residual.shape != (*shape[:-1], out_features):
            raise ValueError("norm_linear residual must have the shape of the output")
        res_rows = residual.reshape(-1, out_features)
        if res_rows.stride(-1) != 1 or res_rows.stride(0) % 8 != 0:
            res_rows = res_rows.contiguous()
    index, count = _token_rows(name, token_rows, rows)
    out = _output_rows(name, out, (rows.shape[0], out_features), index is not None, x)
    library = _native.load_library()
    status = library.taac_norm_linear_fwd(
        rows.data_ptr(), rows.stride(0), _native.ptr(norm_weight), float(eps), None, _native.ptr(bias),
        packed.data_ptr(), _native.ptr(res_rows), res_rows.stride(0) if res_rows is not None else out_features, out.data_ptr(),
        out_features, rows.shape[0], out_features, in_features, _native.ptr(index), _native.ptr(count),
        _native.ptr(_input_rows(name, input_rows, index, rows)), int(norm_weight is not None),
        _native.current_stream(x.device),
    )
    _native.check(status, "norm_linear")
    return out.reshape(*shape[:-1], out_features)


def norm_linear_heads(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None = None,
    *,
    head_dim: int,
    norm_weight: torch.Tensor | None = None,
    eps: float = 1e-6,
    token_rows: tuple[torch.Tensor, torch.Tensor] | None = None,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """:func:`norm_linear` (model width 128 / 256, no residual) writing its output as a stack of per-head planes
    ``[out_features / head_dim, rows, head_dim]`` instead of rows ``[rows, out_features]`` (``taac_norm_linear_heads_fwd``;
    ``head_dim`` 32 or 64): plane ``p`` holds columns ``p * head_dim ..`` of every row, so the rows of one head are
    contiguous. For a packed q | k | v projection ``planes.view(3, H, B, T, head_dim)[i].transpose(0, 1)`` is q / k / v as
    a ``(B, H, T, head_dim)`` view for :func:`flash_attention`, whose output keeps that layout and is what
    :func:`attention_out_ffn_heads` reads. Same values as :func:`norm_linear`, bit for bit."""
    name = "hip norm_linear_heads"
    require_cuda_tensors(name, x, weight, bias, norm_weight)
    require_inference(name, x, weight, bias, norm_weight)
    _check_bf16(name, x, weight, bias, norm_weight)
    rows, _ = _as_rows(x)
    _check_weight(name, rows, weight, bias)
    out_features, in_features = weight.shape
    if not _fused_width(in_features) or out_features % 64 != 0 or head_dim not in (32, 64):
        raise RuntimeError(f"{name}: needs in_features 128 / 256, out_features a multiple of 64 and head_dim 32 or 64")
    packed = _packed_linear(weight, norm_weight)
    index, count = _token_rows(name, token_rows, rows)
    shape = (out_features // head_dim, rows.shape[0], head_dim)
    if out is None:
        out = (torch.zeros if index is not None else torch.empty)(shape, dtype=x.dtype, device=x.device)
    elif out.dtype != x.dtype or out.numel() != out_features * rows.shape[0] or not out.is_contiguous():
        raise ValueError(f"{name}: out must be a contiguous {x.dtype} tensor of {out_features * rows.shape[0]} elements")
    library = _native.load_library()
    status = library.taac_norm_linear_heads_fwd(
        rows.data_ptr(), rows.stride(0), _native.ptr(norm_weight), float(eps), _native.ptr(bias), packed.data_ptr(),
        out.data_ptr(), int(head_dim), rows.shape[0], out_features, in_features, _native.ptr(index), _native.ptr(count),
        int(norm_weight is not None), _native.current_stream(x.device))
    _native.check(status, "norm_linear_heads")
    return out.view(shape)


def attention_out_ffn_heads(
    attn: torch.Tensor,
    out_weight: torch.Tensor,
    out_bias: torch.Tensor | None,
    residual: torch.Tensor,
    up_weight: torch.Tensor,
    up_bias: torch.Tensor | None,
    down_weight: torch.Tensor,
    down_bias: torch.Tensor | None,
    *,
    norm_weight: torch.Tensor | None = None,
    eps: float = 1e-6,
    token_rows: tuple[torch.Tensor, torch.Tensor] | None = None,
    out: torch.Tensor | None = None,
    fold_activation: bool | None = None,
) -> torch.Tensor:
    """:func:`attention_out_ffn` whose attention output is a contiguous stack of per-head planes ``[H, rows, head_dim]``
    (``taac_attn_out_ffn_heads_fwd``; the layout :func:`flash_attention` leaves behind for queries taken from
    :func:`norm_linear_heads`). ``residual`` / ``out`` are ``[.., D]`` rows as usual. Same values, bit for bit (for the
    same ``fold_activation``)."""
    name = "hip attention_out_ffn_heads"
    tensors = (attn, out_weight, out_bias, residual, up_weight, up_bias, down_weight, down_bias, norm_weight)
    require_cuda_tensors(name, *tensors)
    require_inference(name, *tensors)
    _check_bf16(name, *tensors)
    if attn.ndim != 3 or not attn.is_contiguous() or attn.shape[2] not in (32, 64):
        raise ValueError(f"{name}: attn must be a contiguous [H, rows, head_dim] stack with head_dim 32 or 64")
    heads, row_count, head_dim = attn.shape
    d_model, hidden = heads * head_dim, up_weight.shape[0] // 2
    res_rows, shape = _as_rows(residual)
    if res_rows.shape != (row_count, d_model):
        raise ValueError(f"{name}: residual must hold {row_count} rows of {d_model}")
    if out_weight.shape != (d_model, d_model) or up_weight.shape != (2 * hidden, d_model) or down_weight.shape != (d_model, hidden):
        raise ValueError(f"{name} expects out_weight [D, D], up_weight [2F, D] and down_weight [D, F]")
    if not (_fused_width(d_model) and hidden % 32 == 0):
        raise RuntimeError(f"{name}: needs model width 128 / 256 and a hidden size that is a multiple of 32")
    packed_out = _packed_cache.get((out_weight,), lambda: pack_linear_weight(out_weight))
    fold = _fold_choice(name, fold_activation, d_model, hidden)
    packed_ffn = _packed_ffn(up_weight, down_weight, True, norm_weight, fold)
    if res_rows.stride(-1) != 1 or res_rows.stride(0) % 8 != 0:
        res_rows = res_rows.contiguous()
    index, count = _token_rows(name, token_rows, res_rows)
    out = _output_rows(name, out, (row_count, d_model), index is not None, residual)
    library = _native.load_library()
    status = library.taac_attn_out_ffn_heads_fwd(
        attn.data_ptr(), int(head_dim), _native.ptr(out_bias), packed_out.data_ptr(), res_rows.data_ptr(), res_rows.stride(0),
        _native.ptr(norm_weight), float(eps), _native.ptr(up_bias), _native.ptr(down_bias), packed_ffn.data_ptr(),
        out.data_ptr(), d_model, row_count, d_model, hidden, _native.ptr(index), _native.ptr(count),
        _folded_flags(norm_weight, fold), _native.current_stream(attn.device))
    _native.check(status, "attention_out_ffn_heads")
    return out.reshape(shape)


def qkv_projection(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None = None,
    *,
    num_heads: int,
    norm_weight: torch.Tensor | None = None,
    eps: float = 1e-6,
    query_weight: torch.Tensor | None = None,
    key_weight: torch.Tensor | None = None,
    qk_eps: float = 1e-6,
    rope_base: float | None = None,
    token_rows: tuple[torch.Tensor, torch.Tensor] | None = None,
    input_rows: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
    scales_out: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor | None, torch.Tensor | None, torch.Tensor | None]:
    """The packed ``[q | k | v]`` projection of an attention layer with the query / key preparation of the reference's
    layers folded into its epilogue: ``x (batch, tokens, d_model) -> (qkv (batch, tokens, 3 d_model), q_row_scale,
    k_row_scale, q_col_scale)``; hand the three factors to the attention call
    (``scaled_dot_product_attention(..., q_row_scale=, k_row_scale=, q_col_scale=)``).

    ``qkv = F.linear(rmsnorm(x, norm_weight, eps), weight, bias)``. ``RMSNorm(d_model)`` of the query and of the key
    (experiments/symbiosis/backbone.py:33-36) splits into one positive factor per token, ``rsqrt(mean(q^2) + qk_eps)``,
    whose statistic the epilogue collects and which is returned as ``q_row_scale`` / ``k_row_scale`` (float32
    (batch, tokens)), and the norm weights. Without a rotation the two weights act on a score only through their
    product, returned as ``q_col_scale`` (float32 (d_model,)) and applied to the query inside the attention kernel: the
    q and k columns of ``qkv`` are then the plain projection. With ``rope_base`` the epilogue multiplies the query and
    key columns by their weights and rotates them over the token positions (experiments/tokenformer/model.py:165-192)
    and ``q_col_scale`` is None. Either way the preparation costs no pass over q and k. ``out`` (bf16, batch * tokens
    rows of 3 d_model) and ``scales_out`` (float32 (2, batch, tokens)) let a caller reuse its buffers; with ``token_rows``
    the rows outside the index are left as they are in them. ``input_rows`` (with ``token_rows``): the row of ``x`` that
    holds each token when the projection is to be written in another layout (:func:`front_rows`); the factors follow the
    rows of the output, the rotation the positions of the rows of ``x``."""
    name = "hip qkv_projection"
    require_cuda_tensors(name, x, weight, bias, norm_weight, query_weight, key_weight)
    require_inference(name, x, weight, bias, norm_weight, query_weight, key_weight)
    _check_bf16(name, x, weight, bias, norm_weight, query_weight, key_weight)
    if x.ndim != 3:
        raise ValueError("qkv_projection expects x of shape (batch, tokens, d_model)")
    batch, tokens, d_model = x.shape
    rows, _ = _as_rows(x)
    _check_weight(name, rows, weight, bias)
    if weight.shape[0] != 3 * d_model:
        raise ValueError("qkv_projection weight must have 3 * d_model rows")
    if d_model % int(num_heads) != 0:
        raise ValueError("d_model must be divisible by num_heads")
    if (query_weight is None) != (key_weight is None):
        raise ValueError("qkv_projection takes both norm weights or neither")
    if query_weight is None and rope_base is None:
        raise ValueError("qkv_projection needs norm weights, a rope_base, or both; use norm_linear otherwise")
    if not (_fused_width(d_model) and d_model % 64 == 0):
        raise RuntimeError("qkv_projection is built for d_model 128 / 256")
    qk_weight = col_scale = None
    if query_weight is not None:
        if query_weight.shape != (d_model,) or key_weight.shape != (d_model,):
            raise ValueError("rms_norm weight must be 1D and match the normalized dimension")
        if rope_base is None:
            col_scale = (query_weight.detach().float() * key_weight.detach().float()).contiguous()
        else:
            qk_weight = torch.cat((query_weight.detach(), key_weight.detach())).contiguous()
    table = None
    if rope_base is not None:
        from taac_2026_amd.accelerators.attention import rope_table

        table = rope_table(tokens, d_model // int(num_heads), rope_base, x.dtype, x.device)
    packed = _packed_linear(weight, norm_weight)
    index, count = _token_rows(name, token_rows, rows)
    out = _output_rows(name, out, (rows.shape[0], 3 * d_model), index is not None, x)
    sumsq = scales = None
    if query_weight is not None:
        sumsq = torch.empty(2 * d_model // 64, rows.shape[0], dtype=torch.float32, device=x.device)
        if scales_out is not None:
            require_cuda_tensors(name, scales_out)
            if scales_out.dtype != torch.float32 or scales_out.shape != (2, batch, tokens) or not scales_out.is_contiguous():
                raise ValueError(f"{name}: scales_out must be a contiguous float32 tensor of shape (2, batch, tokens)")
            scales = scales_out
        else:
            scales = (torch.ones if index is not None else torch.empty)(2, batch, tokens, dtype=torch.float32, device=x.device)
    library = _native.load_library()
    stream = _native.current_stream(x.device)
    status = library.taac_norm_linear_qk_fwd(
        rows.data_ptr(), rows.stride(0), _native.ptr(norm_weight), float(eps), None, _native.ptr(bias), packed.data_ptr(),
        out.data_ptr(), 3 * d_model, rows.shape[0], d_model, int(num_heads), tokens, _native.ptr(qk_weight),
        _native.ptr(table), _native.ptr(sumsq), _native.ptr(index), _native.ptr(count),
        _native.ptr(_input_rows(name, input_rows, index, rows)), int(norm_weight is not None), stream,
    )
    _native.check(status, "qkv_projection")
    if scales is None:
        return out.view(batch, tokens, 3 * d_model), None, None, None
    status = library.taac_row_rstd(sumsq.data_ptr(), rows.shape[0], d_model, float(qk_eps), scales.data_ptr(),
                                   _native.ptr(index), _native.ptr(count), stream)
    _native.check(status, "row_rstd")
    return out.view(batch, tokens, 3 * d_model), scales[0], scales[1], col_scale


# ---- FP8 (OCP e4m3fn, per-tensor scale = amax / 448) ---------------------------------------------------------------


def amax(x: torch.Tensor) -> torch.Tensor:
    """``x.abs().max()`` as a float32 scalar tensor on x's device."""
    name = "hip amax"
    require_cuda_tensors(name, x)
    x = x.contiguous()
    out = torch.empty((), dtype=torch.float32, device=x.device)
    library = _native.load_library()
    status = library.taac_amax(x.data_ptr(), x.numel(), _native.dtype_code(x.dtype), out.data_ptr(),
                               _native.current_stream(x.device))
    _native.check(status, "amax")
    return out


def quantize_fp8(x: torch.Tensor, amax_value: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """Quantise to e4m3fn with scale ``amax / 448``. Returns ``(q as torch.float8_e4m3fn, amax float32 scalar)``."""
    name = "hip quantize_fp8"
    require_cuda_tensors(name, x, amax_value)
    x = x.contiguous()
    if amax_value is None:
        amax_value = amax(x)
    if amax_value.dtype != torch.float32 or amax_value.numel() != 1:
        raise ValueError("quantize_fp8 amax must be a float32 scalar tensor")
    q = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    library = _native.load_library()
    status = library.taac_quantize_fp8(x.data_ptr(), x.numel(), _native.dtype_code(x.dtype), amax_value.data_ptr(),
                                       q.data_ptr(), _native.current_stream(x.device))
    _native.check(status, "quantize_fp8")
    return q.view(torch.float8_e4m3fn), amax_value


def linear_fp8(
    x: torch.Tensor,
    weight_fp8: torch.Tensor,
    amax_x: torch.Tensor,
    amax_w: torch.Tensor,
    bias: torch.Tensor | None = None,
    *,
    residual: torch.Tensor | None = None,
    swiglu: bool = False,
    gate_first: bool = True,
) -> torch.Tensor:
    """``epilogue((q_x @ q_w^T) * s_x * s_w + bias)`` with e4m3 MFMA operands, bf16 result.

    ``x`` is bf16 (quantised on load with scale ``amax_x / 448``) or already ``float8_e4m3fn``;
    ``weight_fp8`` is ``float8_e4m3fn`` ``[out, in]`` quantised with scale ``amax_w / 448``.
    ``swiglu`` selects the ``silu(gate) * value`` epilogue (output has ``out / 2`` features), ``residual`` the
    fused residual add; they are exclusive.
    """
    name = "hip linear_fp8"
    require_cuda_tensors(name, x, weight_fp8, amax_x, amax_w, bias, residual)
    require_inference(name, x, bias, residual)
    _check_bf16(name, bias, residual)
    if weight_fp8.dtype != torch.float8_e4m3fn:
        raise RuntimeError("linear_fp8 weight must be float8_e4m3fn")
    if x.dtype not in (torch.bfloat16, torch.float8_e4m3fn):
        raise RuntimeError(f"linear_fp8 activations must be bfloat16 or float8_e4m3fn, got {x.dtype}")
    if swiglu and residual is not None:
        raise ValueError("linear_fp8 cannot combine the swiglu and residual epilogues")
    if x.ndim < 2:
        raise ValueError("linear expects input with at least 2 dimensions")
    shape = x.shape
    rows = x.reshape(-1, shape[-1]).contiguous()
    _check_weight(name, rows, weight_fp8, bias)
    weight_fp8 = weight_fp8.contiguous()
    n = weight_fp8.shape[0]
    if swiglu and n % 2 != 0:
        raise ValueError("swiglu weight must have an even number of output features")
    out_features = n // 2 if swiglu else n
    out = torch.empty((rows.shape[0], out_features), dtype=torch.bfloat16, device=x.device)
    res_rows = residual.reshape(-1, out_features).contiguous() if residual is not None else None
    epilogue = _native.EPI_SWIGLU if swiglu else (_native.EPI_RESIDUAL if res_rows is not None else _native.EPI_NONE)
    library = _native.load_library()
    status = library.taac_linear_fp8(
        rows.data_ptr(), int(x.dtype == torch.float8_e4m3fn), rows.stride(0), weight_fp8.data_ptr(),
        amax_x.data_ptr(), amax_w.data_ptr(), _native.ptr(bias), _native.ptr(res_rows), out.data_ptr(), out_features,
        rows.shape[0], n, weight_fp8.shape[1], epilogue, int(bool(gate_first)), _native.current_stream(x.device),
    )
    _native.check(status, "linear_fp8")
    return out.reshape(*shape[:-1], out_features)


def norm_linear_fp8(
    x: torch.Tensor,
    weight_fp8: torch.Tensor,
    amax_x: torch.Tensor,
    amax_w: torch.Tensor,
    bias: torch.Tensor | None = None,
    *,
    norm_weight: torch.Tensor | None = None,
    eps: float = 1e-6,
    residual: torch.Tensor | None = None,
    token_rows: tuple[torch.Tensor, torch.Tensor] | None = None,
    out: torch.Tensor | None = None,
    out_norm_weight: torch.Tensor | None = None,
    out_eps: float = 1e-6,
    want_amax_out: bool = False,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """``residual + linear_fp8(rmsnorm(x, norm_weight), weight_fp8)`` (norm and residual optional) as one kernel for
    ``in_features == 256`` (``taac_norm_linear_fp8_fwd``): the rows are normalised, rounded to bf16 and quantised with
    ``amax_x / 448`` on their way into registers. ``amax_x`` is the float32 scalar max of the tensor that is quantised
    (of the normalised rows when ``norm_weight`` is given). ``token_rows`` / ``out`` as in :func:`norm_linear`.
    Returns ``(out, amax_out)``; with ``want_amax_out`` (or an ``out_norm_weight``) the epilogue also reduces the scale
    of the layer that consumes the output: the max of ``|rmsnorm(out, out_norm_weight)|`` (of ``|out|`` without a
    weight), so that no pass of its own is needed for it."""
    name = "hip norm_linear_fp8"
    require_cuda_tensors(name, x, weight_fp8, amax_x, amax_w, bias, norm_weight, residual, out_norm_weight)
    require_inference(name, x, bias, norm_weight, residual)
    _check_bf16(name, x, bias, norm_weight, residual, out_norm_weight)
    if weight_fp8.dtype != torch.float8_e4m3fn:
        raise RuntimeError("norm_linear_fp8 weight must be float8_e4m3fn")
    rows, shape = _as_rows(x)
    _check_weight(name, rows, weight_fp8, bias)
    out_features, in_features = weight_fp8.shape
    if in_features != 256 or out_features % 64 != 0:
        raise RuntimeError("norm_linear_fp8 is built for in_features = 256 and out_features a multiple of 64")
    weight_fp8 = weight_fp8.contiguous()
    res_rows = None
    if residual is not None:
        if residual.shape != (*shape[:-1], out_features):
            raise ValueError("norm_linear_fp8 residual must have the shape of the output")
        res_rows = residual.reshape(-1, out_features)
        if res_rows.stride(-1) != 1 or res_rows.stride(0) % 8 != 0:
            res_rows = res_rows.contiguous()
    index, count = _token_rows(name, token_rows, rows)
    out = _output_rows(name, out, (rows.shape[0], out_features), index is not None, x)
    amax_out = None
    if want_amax_out or out_norm_weight is not None:
        amax_out = torch.empty((), dtype=torch.float32, device=x.device)
    library = _native.load_library()
    status = library.taac_norm_linear_fp8_fwd(
        rows.data_ptr(), rows.stride(0), _native.ptr(norm_weight), float(eps), weight_fp8.data_ptr(), _native.ptr(bias),
        amax_x.data_ptr(), amax_w.data_ptr(), _native.ptr(res_rows), res_rows.stride(0) if res_rows is not None else out_features,
        out.data_ptr(), out_features, rows.shape[0], out_features, in_features, _native.ptr(index), _native.ptr(count),
        _native.ptr(out_norm_weight), float(out_eps), _native.ptr(amax_out), _native.current_stream(x.device),
    )
    _native.check(status, "norm_linear_fp8")
    return out.reshape(*shape[:-1], out_features), amax_out


def pack_ffn_weights_fp8(up_weight: torch.Tensor, down_weight: torch.Tensor, *, gate_first: bool = True
                         ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Quantises ``(up_weight [2F, D], down_weight [D, F])`` to e4m3 with their per-tensor scales and lays them out in
    the fragment order of :func:`swiglu_ffn_fp8`. Returns ``(blob uint8, amax_up, amax_down)``."""
    name = "hip pack_ffn_weights_fp8"
    require_cuda_tensors(name, up_weight, down_weight)
    _check_bf16(name, up_weight, down_weight)
    library = _native.load_library()
    d_model, hidden = down_weight.shape
    if up_weight.shape != (2 * hidden, d_model):
        raise ValueError("pack_ffn_weights_fp8 expects up_weight [2F, D] and down_weight [D, F]")
    nbytes = library.taac_ffn_fp8_packed_bytes(d_model, hidden)
    if nbytes < 0:
        raise RuntimeError(f"pack_ffn_weights_fp8: unsupported shape D={d_model}, F={hidden} (D 128 / 256, F a multiple of 64)")
    up_weight, down_weight = up_weight.detach().contiguous(), down_weight.detach().contiguous()
    amax_up, amax_down = amax(up_weight), amax(down_weight)
    packed = torch.empty(nbytes, dtype=torch.uint8, device=up_weight.device)
    status = library.taac_ffn_fp8_pack_weights(up_weight.data_ptr(), down_weight.data_ptr(), amax_up.data_ptr(),
                                               amax_down.data_ptr(), packed.data_ptr(), d_model, hidden,
                                               int(bool(gate_first)), _native.current_stream(up_weight.device))
    _native.check(status, "pack_ffn_weights_fp8")
    return packed, amax_up, amax_down


def swiglu_ffn_fp8(
    x: torch.Tensor,
    packed_weights: tuple[torch.Tensor, torch.Tensor, torch.Tensor],
    up_bias: torch.Tensor | None,
    down_bias: torch.Tensor | None,
    amax_x: torch.Tensor,
    *,
    hidden_size: int,
    residual: torch.Tensor | None = None,
    gate_first: bool = True,
    norm_weight: torch.Tensor | None = None,
    eps: float = 1e-6,
    token_rows: tuple[torch.Tensor, torch.Tensor] | None = None,
    out: torch.Tensor | None = None,
    next_norm_weight: torch.Tensor | None = None,
    next_eps: float = 1e-6,
    want_amax_next: bool = False,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor | None]:
    """The feed-forward half with e4m3 MFMA operands and per-tensor scales as ONE fused layer (two launches: the first
    finds the scale of the gated hidden state, the second evaluates the layer; the hidden state never reaches memory):
    ``residual + down_fp8(silu(gate) * value)``, ``gate, value = up_fp8(rmsnorm(x)).chunk(2, -1)``, each ``*_fp8`` the
    quantize -> matmul -> dequantize layer of :func:`linear_fp8`. ``packed_weights`` is the triple returned by
    :func:`pack_ffn_weights_fp8` (packed with the same ``gate_first``); ``amax_x`` the float32 scalar max of the tensor
    the up projection quantises (``rmsnorm(x) * norm_weight`` rounded to bf16 when ``norm_weight`` is given). Returns
    ``(out, amax_hidden, amax_next)``; ``amax_next`` (with ``want_amax_next``) is the max of
    ``|rmsnorm(out, next_norm_weight)|`` (of ``|out|`` without a weight), i.e. the ``amax_x`` of the layer that consumes
    ``out``. ``token_rows`` / ``out`` as in :func:`swiglu_ffn`."""
    name = "hip swiglu_ffn_fp8"
    blob, amax_up, amax_down = packed_weights
    require_cuda_tensors(name, x, blob, amax_up, amax_down, up_bias, down_bias, amax_x, residual, norm_weight, next_norm_weight)
    require_inference(name, x, up_bias, down_bias, residual, norm_weight)
    _check_bf16(name, x, up_bias, down_bias, residual, norm_weight, next_norm_weight)
    rows, shape = _as_rows(x)
    d_model, hidden = rows.shape[1], int(hidden_size)
    library = _native.load_library()
    if library.taac_ffn_fp8_packed_bytes(d_model, hidden) != blob.numel():
        raise ValueError(f"swiglu_ffn_fp8: the packed weights do not match D={d_model}, F={hidden}")
    for scale in (amax_x, amax_up, amax_down):
        if scale.dtype != torch.float32 or scale.numel() != 1:
            raise ValueError("swiglu_ffn_fp8 scales must be float32 scalar tensors")
    if residual is not None and residual.shape != shape:
        raise ValueError("swiglu_ffn_fp8 residual must have the shape of the input")
    res_rows = None
    if residual is not None:
        res_rows = residual.reshape(-1, d_model)
        if res_rows.stride(-1) != 1 or res_rows.stride(0) % 8 != 0:
            res_rows = res_rows.contiguous()
    index, count = _token_rows(name, token_rows, rows)
    out = _output_rows(name, out, (rows.shape[0], d_model), index is not None, x)
    amax_hidden = torch.empty((), dtype=torch.float32, device=x.device)
    amax_next = torch.empty((), dtype=torch.float32, device=x.device) if (want_amax_next or next_norm_weight is not None) else None
    status = library.taac_swiglu_ffn_fp8_fwd(
        rows.data_ptr(), rows.stride(0), _native.ptr(norm_weight), float(eps), blob.data_ptr(), _native.ptr(up_bias),
        _native.ptr(down_bias), amax_x.data_ptr(), amax_up.data_ptr(), amax_down.data_ptr(), amax_hidden.data_ptr(),
        _native.ptr(res_rows), res_rows.stride(0) if res_rows is not None else d_model, out.data_ptr(), d_model,
        rows.shape[0], d_model, hidden, int(bool(gate_first)), _native.ptr(index), _native.ptr(count),
        _native.ptr(next_norm_weight), float(next_eps), _native.ptr(amax_next), _native.current_stream(x.device),
    )
    _native.check(status, "swiglu_ffn_fp8")
    return out.reshape(shape), amax_hidden, amax_next


__all__ = [
    "FP8_MAX",
    "amax",
    "clear_packed_weight_cache",
    "linear",
    "linear_fp8",
    "linear_wgrad",
    "swiglu_ffn_backward_hidden",
    "swiglu_ffn_dropout",
    "swiglu_backward",
    "norm_linear",
    "pack_ffn_weights",
    "pack_mlp_weights",
    "silu_mlp",
    "norm_linear_fp8",
    "pack_ffn_weights_fp8",
    "swiglu_ffn_fp8",
    "valid_rows",
    "pack_linear_weight",
    "qkv_projection",
    "quantize_fp8",
    "swiglu_ffn",
    "swiglu_linear",
]
