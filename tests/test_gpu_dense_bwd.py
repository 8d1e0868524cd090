"""GPU parity: backward of the dense layers (weight gradient, SiLU-gate backward, and the autograd routes of norm_linear /
swiglu_ffn / the interaction block) against torch autograd of the CPU oracle's formulas evaluated in float64. Tolerance:
the reference's gradient tolerance for its 16-bit GPU kernels (tests/gpu/infrastructure/accelerators/
test_tilelang_ops_cuda.py:98-141), 3e-2, relative to the largest expected value of each gradient."""

from __future__ import annotations

import pytest
import torch
import torch.nn.functional as F

from oracle import reference as oracle
from taac_2026_amd.api import (UnifiedInteractionBlock, linear, linear_wgrad, norm_linear, swiglu_backward, swiglu_ffn,
                               swiglu_ffn_backward_hidden)

pytestmark = pytest.mark.gpu


def _close(got: torch.Tensor, want: torch.Tensor, tol: float = 3e-2) -> None:
    want = want.double()
    scale = want.abs().max().item()
    assert (got.detach().cpu().double() - want).abs().max().item() <= tol * max(scale, 1e-6), (
        (got.detach().cpu().double() - want).abs().max().item(), scale)


@pytest.mark.parametrize("m,n,k", [(1, 8, 8), (33, 64, 256), (1000, 768, 256), (5000, 256, 1024), (4099, 2048, 256),
                                   (777, 72, 40)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_weight_gradient_is_the_product_over_the_tokens(device, m, n, k, dtype):
    g = torch.Generator().manual_seed(m + n)
    dy = torch.randn(m, n, generator=g).to(torch.bfloat16)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    grad_w, grad_b = linear_wgrad(dy.to(device), a.to(device), dtype=dtype)
    assert grad_w.dtype == dtype and grad_w.shape == (n, k) and grad_b.shape == (n,)
    _close(grad_w, dy.double().t() @ a.double(), 1e-2)
    _close(grad_b, dy.double().sum(0), 1e-2)
    again_w, again_b = linear_wgrad(dy.to(device), a.to(device), dtype=dtype)
    assert torch.equal(again_w, grad_w) and torch.equal(again_b, grad_b)      # fixed summation order
    without, none = linear_wgrad(dy.to(device), a.to(device), with_bias=False, dtype=dtype)
    assert none is None and torch.equal(without, grad_w)


def test_weight_gradient_of_strided_rows_and_errors(device):
    g = torch.Generator().manual_seed(2)
    packed = torch.randn(300, 3 * 64, generator=g).to(torch.bfloat16).to(device)
    a = torch.randn(300, 128, generator=g).to(torch.bfloat16).to(device)
    dy = packed[:, 64:128]                                                   # a column slice: row stride 192
    grad_w, _ = linear_wgrad(dy, a, dtype=torch.float32)
    _close(grad_w, dy.cpu().double().t() @ a.cpu().double(), 1e-2)
    with pytest.raises(ValueError, match="same number of rows"):
        linear_wgrad(dy[:10], a)
    with pytest.raises(RuntimeError, match="multiples of 8"):
        linear_wgrad(torch.zeros(4, 12, dtype=torch.bfloat16, device=device), torch.zeros(4, 16, dtype=torch.bfloat16, device=device))


@pytest.mark.parametrize("gate_first", [True, False])
def test_silu_gate_backward(device, gate_first):
    g = torch.Generator().manual_seed(int(gate_first))
    pre = (2 * torch.randn(257, 2 * 96, generator=g)).to(torch.bfloat16)
    grad_hidden = torch.randn(257, 96, generator=g).to(torch.bfloat16)
    hidden, grad_pre = swiglu_backward(pre.to(device), grad_hidden.to(device), gate_first=gate_first)
    ref = pre.double().requires_grad_(True)
    gate, value = ref.chunk(2, dim=-1)
    want = F.silu(gate) * value if gate_first else gate * F.silu(value)
    want.backward(grad_hidden.double())
    _close(hidden, want.detach(), 1e-2)
    _close(grad_pre, ref.grad, 1e-2)
    only_hidden, none = swiglu_backward(pre.to(device), None, gate_first=gate_first)
    assert none is None and torch.equal(only_hidden, hidden)


@pytest.mark.parametrize("m,d,f,gate_first,with_bias", [(1, 128, 32, True, True), (255, 256, 96, False, True),
                                                          (257, 256, 1024, True, True), (1000, 128, 2048, True, False),
                                                          (4096, 256, 512, False, False)])
def test_feed_forward_backward_hidden_kernel(device, m, d, f, gate_first, with_bias):
    """The one-kernel activation backward (up projection and ``dy @ w_down`` recomputed in registers) against float64
    autograd of the same expression, and against the three-kernel route it replaces (equal up to the roundings of
    bfloat16: that route rounds the up projection and ``dy @ w_down`` to bfloat16 on the way, the kernel keeps them in
    float32)."""
    g = torch.Generator().manual_seed(m + f)
    bf = lambda t: t.to(torch.bfloat16)  # noqa: E731
    h = bf(torch.randn(m, d, generator=g))
    dy = bf(torch.randn(m, d, generator=g))
    up_w = bf(torch.randn(2 * f, d, generator=g) * d ** -0.5)
    up_b = bf(0.5 * torch.randn(2 * f, generator=g)) if with_bias else None
    down_w = bf(torch.randn(d, f, generator=g) * f ** -0.5)
    on = lambda t: None if t is None else t.to(device)  # noqa: E731
    hidden, grad_pre = swiglu_ffn_backward_hidden(on(h), on(dy), on(up_w), on(up_b), on(down_w), gate_first=gate_first)
    assert hidden.shape == (m, f) and grad_pre.shape == (m, 2 * f)
    pre = (F.linear(h.double(), up_w.double(), None if up_b is None else up_b.double())).requires_grad_(True)
    gate, value = pre.chunk(2, dim=-1)
    want = F.silu(gate) * value if gate_first else gate * F.silu(value)
    want.backward(dy.double() @ down_w.double())
    _close(hidden, want.detach(), 1e-2)
    _close(grad_pre, pre.grad, 1.5e-2)
    with torch.no_grad():
        pre_rows = linear(on(h), on(up_w), on(up_b))
        grad_hidden = linear(on(dy), on(down_w).t().contiguous())
    hidden_steps, grad_steps = swiglu_backward(pre_rows, grad_hidden, gate_first=gate_first)
    _close(hidden, hidden_steps.cpu(), 1e-2)
    _close(grad_pre, grad_steps.cpu(), 1e-2)


def test_feed_forward_backward_hidden_kernel_shapes(device):
    z = lambda *shape: torch.zeros(*shape, dtype=torch.bfloat16, device=device)  # noqa: E731
    assert swiglu_ffn_backward_hidden(z(4, 64), z(4, 64), z(2 * 32, 64), None, z(64, 32)) is None     # width 64: not built
    assert swiglu_ffn_backward_hidden(z(4, 256), z(4, 256), z(2 * 40, 256), None, z(256, 40)) is None  # F not a multiple of 32
    with pytest.raises(ValueError, match="expected h and grad_out"):
        swiglu_ffn_backward_hidden(z(4, 256), z(5, 256), z(64, 256), None, z(256, 32))
    hidden, grad_pre = swiglu_ffn_backward_hidden(z(0, 256), z(0, 256), z(64, 256), None, z(256, 32))
    assert hidden.shape == (0, 32) and grad_pre.shape == (0, 64)


def _dense_case(m, d, n, seed):
    g = torch.Generator().manual_seed(seed)
    bf = lambda t: t.to(torch.bfloat16)  # noqa: E731
    x = bf(torch.randn(m, d, generator=g))
    w = bf(torch.randn(n, d, generator=g) * d ** -0.5)
    b = bf(0.1 * torch.randn(n, generator=g))
    nw = bf(1 + 0.1 * torch.randn(d, generator=g))
    res = bf(torch.randn(m, n, generator=g))
    dy = bf(torch.randn(m, n, generator=g))
    return x, w, b, nw, res, dy


@pytest.mark.parametrize("m,d,n", [(300, 256, 768), (129, 128, 128), (50, 64, 96)])
@pytest.mark.parametrize("with_norm,with_residual", [(True, False), (False, True), (True, True)])
def test_norm_linear_takes_a_gradient(device, m, d, n, with_norm, with_residual):
    """RMSNorm -> linear -> + residual, fused widths (128 / 256) and the composed route (64): every gradient against float64
    autograd of the oracle's formulas."""
    x, w, b, nw, res, dy = _dense_case(m, d, n, seed=m + n)
    dev = [t.to(device).requires_grad_(True) for t in (x, w, b, nw, res)]
    out = norm_linear(dev[0], dev[1], dev[2], norm_weight=dev[3] if with_norm else None,
                      residual=dev[4] if with_residual else None)
    out.backward(dy.to(device))
    ref = [t.double().requires_grad_(True) for t in (x, w, b, nw, res)]
    h = oracle.rms_norm(ref[0], ref[3]) if with_norm else ref[0]
    want = F.linear(h, ref[1], ref[2]) + (ref[4] if with_residual else 0)
    want.backward(dy.double())
    _close(out, want.detach(), 2e-2)
    for index, (got, expected) in enumerate(zip(dev, ref)):
        if (index == 3 and not with_norm) or (index == 4 and not with_residual):
            assert got.grad is None
        else:
            _close(got.grad, expected.grad)


def test_linear_takes_a_gradient_and_the_forward_is_the_inference_kernel(device):
    x, w, b, _, _, dy = _dense_case(200, 256, 512, seed=9)
    xd, wd, bd = (t.to(device).requires_grad_(True) for t in (x, w, b))
    out = linear(xd.view(4, 50, 256), wd, bd)
    with torch.no_grad():
        assert torch.equal(out.detach(), linear(xd.view(4, 50, 256), wd, bd))
    out.backward(dy.to(device).view(4, 50, 512))
    _close(wd.grad, dy.double().t() @ x.double())
    _close(xd.grad, dy.double() @ w.double())
    _close(bd.grad, dy.double().sum(0))
    with pytest.raises(RuntimeError, match="inference route"):
        norm_linear(xd, wd, bd, out=torch.empty(200, 512, dtype=torch.bfloat16, device=device))


@pytest.mark.parametrize("m,d,f,gate_first,with_norm", [(300, 256, 512, True, True), (100, 128, 96, False, True),
                                                          (64, 64, 80, True, False), (513, 256, 1024, True, True)])
def test_swiglu_ffn_takes_a_gradient(device, m, d, f, gate_first, with_norm):
    g = torch.Generator().manual_seed(m + f)
    bf = lambda t: t.to(torch.bfloat16)  # noqa: E731
    x = bf(torch.randn(m, d, generator=g))
    nw = bf(1 + 0.1 * torch.randn(d, generator=g))
    up_w, up_b = bf(torch.randn(2 * f, d, generator=g) * d ** -0.5), bf(0.1 * torch.randn(2 * f, generator=g))
    down_w, down_b = bf(torch.randn(d, f, generator=g) * f ** -0.5), bf(0.1 * torch.randn(d, generator=g))
    dy = bf(torch.randn(m, d, generator=g))
    tensors = (x, nw, up_w, up_b, down_w, down_b)
    dev = [t.to(device).requires_grad_(True) for t in tensors]
    out = swiglu_ffn(dev[0], dev[2], dev[3], dev[4], dev[5], residual=dev[0], gate_first=gate_first,
                     norm_weight=dev[1] if with_norm else None)
    out.backward(dy.to(device))
    ref = [t.double().requires_grad_(True) for t in tensors]
    h = oracle.rms_norm(ref[0], ref[1]) if with_norm else ref[0]
    want = ref[0] + oracle.swiglu_ffn(h, ref[2], ref[3], ref[4], ref[5], gate_first=gate_first)
    want.backward(dy.double())
    _close(out, want.detach(), 2e-2)
    for index, (got, expected) in enumerate(zip(dev, ref)):
        if index == 1 and not with_norm:
            assert got.grad is None
        else:
            _close(got.grad, expected.grad)


@pytest.mark.parametrize("qk_norm", [False, True])
def test_interaction_block_takes_a_gradient_end_to_end(device, qk_norm):
    """``UnifiedInteractionBlock`` in training mode (plain attention layer or the reference's default with query / key
    norms, key-length mask): output and the gradient of the input and of every parameter against float64 autograd of
    ``oracle.interaction_block`` (experiments/symbiosis/backbone.py:58-68)."""
    batch, tokens, d_model, heads, mult = 3, 48, 128, 4, 2
    g = torch.Generator().manual_seed(1)
    block = UnifiedInteractionBlock(d_model, heads, mult, qk_norm=qk_norm)
    with torch.no_grad():
        for parameter in block.parameters():
            if parameter.ndim == 1:
                parameter.copy_((1.0 if parameter.shape[0] == d_model and parameter.mean() > 0.5 else 0.0)
                                + 0.1 * torch.randn(parameter.shape, generator=g))
            else:
                parameter.copy_(torch.randn(parameter.shape, generator=g) * parameter.shape[1] ** -0.5)
    block = block.to(torch.bfloat16)
    weights = {
        "attn_norm.weight": block.attn_norm.weight, "qkv.weight": block.attention.qkv.weight,
        "qkv.bias": block.attention.qkv.bias, "out.weight": block.attention.out.weight, "out.bias": block.attention.out.bias,
        "ffn_norm.weight": block.ffn_norm.weight, "up.weight": block.ffn.up.weight, "up.bias": block.ffn.up.bias,
        "down.weight": block.ffn.down.weight, "down.bias": block.ffn.down.bias,
    }
    if qk_norm:
        weights["query_norm.weight"] = block.attention.query_norm.weight
        weights["key_norm.weight"] = block.attention.key_norm.weight
    reference = {name: value.detach().double().requires_grad_(True) for name, value in weights.items()}
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)
    lengths = torch.tensor([48, 17, 33], dtype=torch.int32)
    padding = torch.arange(tokens)[None, :] >= lengths[:, None]
    grad_out = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)

    block = block.to(device).train()
    xd = x.to(device).requires_grad_(True)
    out, _ = block(xd, padding.to(device), None, key_lengths=lengths.to(device))
    out.backward(grad_out.to(device))

    xr = x.double().requires_grad_(True)
    mask = (~padding)[:, None, None, :].expand(batch, 1, tokens, tokens)
    want, _ = oracle.interaction_block(xr, padding, mask, reference, num_heads=heads)
    want.backward(grad_out.double())
    _close(out, want.detach(), 2e-2)
    _close(xd.grad, xr.grad)
    named = dict(block.named_parameters())
    lookup = {"attn_norm.weight": "attn_norm.weight", "qkv.weight": "attention.qkv.weight", "qkv.bias": "attention.qkv.bias",
              "out.weight": "attention.out.weight", "out.bias": "attention.out.bias", "ffn_norm.weight": "ffn_norm.weight",
              "up.weight": "ffn.up.weight", "up.bias": "ffn.up.bias", "down.weight": "ffn.down.weight",
              "down.bias": "ffn.down.bias"}
    if qk_norm:
        lookup.update({"query_norm.weight": "attention.query_norm.weight", "key_norm.weight": "attention.key_norm.weight"})
    for name, parameter_name in lookup.items():
        assert named[parameter_name].grad is not None, parameter_name
        _close(named[parameter_name].grad, reference[name].grad)


@pytest.mark.parametrize("d_model,heads,mult,use_attn_tokens,qk_norm", [(256, 8, 4, False, False), (256, 4, 2, True, False),
                                                                        (128, 4, 2, True, False), (256, 8, 4, False, True),
                                                                        (128, 2, 2, True, True)])
def test_block_training_route_over_the_valid_rows_equals_the_layer_by_layer_route(device, monkeypatch, d_model, heads, mult,
                                                                                 use_attn_tokens, qk_norm):
    """The one-function training route (valid rows compacted, gradients of the packed projection written in place)
    against the layer-by-layer autograd route of the same module: outputs, input gradient and every parameter gradient,
    with a sample of length zero, a full one, and a loss that also uses the block's second output."""
    import taac_2026_amd.modeling.backbone as backbone_module

    batch, tokens = 6, 96
    g = torch.Generator().manual_seed(d_model + heads)
    block = UnifiedInteractionBlock(d_model, heads, mult, qk_norm=qk_norm)
    with torch.no_grad():
        for parameter in block.parameters():
            if parameter.ndim == 1:
                parameter.copy_((1.0 if parameter.shape[0] == d_model and parameter.mean() > 0.5 else 0.0)
                                + 0.1 * torch.randn(parameter.shape, generator=g))
            else:
                parameter.copy_(torch.randn(parameter.shape, generator=g) * parameter.shape[1] ** -0.5)
    block = block.to(torch.bfloat16).to(device).train()
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    lengths = torch.tensor([96, 0, 33, 1, 64, 17], dtype=torch.int32, device=device)
    padding = torch.arange(tokens, device=device)[None, :] >= lengths[:, None]
    grad_out = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    grad_attn = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)

    def run(compact: bool):
        if not compact:
            monkeypatch.setattr(backbone_module, "training_route_applies", lambda *a, **k: False)
        xd = x.clone().requires_grad_(True)
        block.zero_grad(set_to_none=True)
        out, attn_tokens = block(xd, padding, None, key_lengths=lengths)
        loss_grads = [grad_out] + ([grad_attn] if use_attn_tokens else [])
        torch.autograd.backward([out] + ([attn_tokens] if use_attn_tokens else []), loss_grads)
        monkeypatch.undo()
        return out.detach(), attn_tokens.detach(), xd.grad, {n: p.grad.clone() for n, p in block.named_parameters()}

    out_c, attn_c, gx_c, grads_c = run(True)
    out_s, attn_s, gx_s, grads_s = run(False)
    _close(out_c, out_s.cpu(), 1e-2)
    _close(attn_c, attn_s.cpu(), 1e-2)
    valid = ~padding.cpu()
    assert torch.equal(out_c.cpu()[~valid], x.cpu()[~valid]) and torch.equal(attn_c.cpu()[~valid], x.cpu()[~valid])
    _close(gx_c, gx_s.cpu(), 2e-2)
    expected_padded = (grad_out + grad_attn if use_attn_tokens else grad_out).cpu()
    assert torch.equal(gx_c.cpu()[~valid], expected_padded[~valid])             # padded positions: identity
    for name in grads_s:
        _close(grads_c[name], grads_s[name].cpu(), 2e-2)


def test_rows_gather_and_merge_through_the_c_abi(device):
    """``taac_rows_gather`` compacts the valid rows of a padded tensor (also out of a column slice), ``taac_rows_merge``
    puts compact rows (one part, or the rounded sum of two) back between the pass-through rows: bit-exact against
    indexing, with an empty and a full sample."""
    from taac_2026_amd import _native
    from taac_2026_amd.api import valid_rows

    library = _native.load_library()
    batch, tokens, width = 5, 40, 72
    g = torch.Generator().manual_seed(3)
    lengths = torch.tensor([40, 0, 7, 1, 23], dtype=torch.int32, device=device)
    padded = torch.randn(batch * tokens, 2 * width, generator=g).to(torch.bfloat16).to(device)
    rows, count = valid_rows(lengths, tokens)
    valid = int(count.item())
    index = rows[:valid].long()
    stream = _native.current_stream(padded.device)
    source = padded[:, width:]                                                  # row stride 2 * width
    compact = torch.empty(valid, width, dtype=torch.bfloat16, device=device)
    _native.check(library.taac_rows_gather(source.data_ptr(), source.stride(0), rows.data_ptr(), valid, compact.data_ptr(),
                                           width, stream), "gather")
    assert torch.equal(compact, source[index])
    a = torch.randn(valid, width, generator=g).to(torch.bfloat16).to(device)
    b = torch.randn(valid, width, generator=g).to(torch.bfloat16).to(device)
    base = padded[:, :width].contiguous()
    for second in (None, b):
        out = torch.empty_like(base)
        _native.check(library.taac_rows_merge(base.data_ptr(), a.data_ptr(), _native.ptr(second), lengths.data_ptr(),
                                              rows.data_ptr() + 4 * batch * tokens, out.data_ptr(), batch, tokens, width,
                                              stream), "merge")
        expected = base.clone()
        expected[index] = a if second is None else (a.float() + b.float()).to(torch.bfloat16)
        assert torch.equal(out, expected)
    assert library.taac_rows_gather(source.data_ptr(), source.stride(0), rows.data_ptr(), valid, compact.data_ptr(), 12,
                                    stream) == _native.TAAC_ERR_UNSUPPORTED
    # padding that is not a prefix: validity bits, with and without the table of valid tokens in front of each word
    from taac_2026_amd.accelerators.attention import _pack_bits

    padding = torch.rand(batch, tokens, generator=g) < 0.4
    padding[1] = True
    padding[0] = False
    padding = padding.to(device)
    rows, count = valid_rows(None, tokens, padding_mask=padding)
    valid = int(count.item())
    index = rows[:valid].long()
    assert torch.equal(index, (~padding).flatten().nonzero().flatten())
    bits = _pack_bits((~padding).contiguous())
    words = bits.shape[1]
    per_word = torch.nn.functional.pad(~padding, (0, words * 32 - tokens)).view(batch, words, 32).sum(-1)
    prefix = (per_word.cumsum(1) - per_word).to(torch.int32).contiguous()
    a = torch.randn(valid, width, generator=g).to(torch.bfloat16).to(device)
    b = torch.randn(valid, width, generator=g).to(torch.bfloat16).to(device)
    for second in (None, b):
        for table in (None, prefix):
            out = torch.empty_like(base)
            _native.check(library.taac_rows_merge_bits(base.data_ptr(), a.data_ptr(), _native.ptr(second), bits.data_ptr(),
                                                       _native.ptr(table), rows.data_ptr() + 4 * batch * tokens,
                                                       out.data_ptr(), batch, tokens, width, stream), "merge_bits")
            expected = base.clone()
            expected[index] = a if second is None else (a.float() + b.float()).to(torch.bfloat16)
            assert torch.equal(out, expected)


def test_two_blocks_and_the_readout_train_end_to_end(device):
    """A stack of two blocks (shared key lengths: one row index, one host synchronisation) and the readout head under a
    binary cross-entropy loss: the loss and the gradient of the input and of every parameter against float64 autograd of
    the oracle's blocks and readout."""
    from types import SimpleNamespace

    from taac_2026_amd.api import CandidateReadoutHead

    batch, tokens, d_model, heads, mult = 4, 40, 128, 4, 2
    g = torch.Generator().manual_seed(11)
    modules = torch.nn.ModuleList([UnifiedInteractionBlock(d_model, heads, mult, qk_norm=False) for _ in range(2)]
                                  + [CandidateReadoutHead(d_model, 1)])
    with torch.no_grad():
        for parameter in modules.parameters():
            if parameter.ndim == 1:
                parameter.copy_((1.0 if parameter.mean() > 0.5 else 0.0) + 0.1 * torch.randn(parameter.shape, generator=g))
            else:
                parameter.copy_(torch.randn(parameter.shape, generator=g) * parameter.shape[1] ** -0.5)
    modules = modules.to(torch.bfloat16)
    reference = {name: value.detach().double().requires_grad_(True) for name, value in modules.named_parameters()}
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)
    lengths = torch.tensor([40, 9, 1, 25], dtype=torch.int32)
    padding = torch.arange(tokens)[None, :] >= lengths[:, None]
    labels = torch.tensor([[1.0], [0.0], [1.0], [0.0]])
    meta = SimpleNamespace(cls_index=0, candidate_index=3, padding_mask=None)

    modules = modules.to(device).train()
    xd = x.to(device).requires_grad_(True)
    stream, lengths_d, padding_d = xd, lengths.to(device), padding.to(device)
    for block in modules[:2]:
        stream, _ = block(stream, padding_d, None, key_lengths=lengths_d, return_attention_tokens=False)
    meta.padding_mask = padding_d
    logits = modules[2](stream, meta)
    loss = F.binary_cross_entropy_with_logits(logits, labels.to(device))
    loss.backward()

    xr = x.double().requires_grad_(True)
    mask = (~padding)[:, None, None, :].expand(batch, 1, tokens, tokens)
    stream_r = xr
    names = {"attn_norm.weight": "attn_norm.weight", "qkv.weight": "attention.qkv.weight", "qkv.bias": "attention.qkv.bias",
             "out.weight": "attention.out.weight", "out.bias": "attention.out.bias", "ffn_norm.weight": "ffn_norm.weight",
             "up.weight": "ffn.up.weight", "up.bias": "ffn.up.bias", "down.weight": "ffn.down.weight",
             "down.bias": "ffn.down.bias"}
    for index in range(2):
        weights = {short: reference[f"{index}.{full}"] for short, full in names.items()}
        stream_r, _ = oracle.interaction_block(stream_r, padding, mask, weights, num_heads=heads)
    _, logits_r = oracle.candidate_readout(
        stream_r, padding, cls_index=0, candidate_index=3, token_norm_weight=reference["2.final_norm.weight"],
        pool_norm_weight=reference["2.pooler.norm.weight"], eps=1e-6,
        classifier=(reference["2.classifier.0.weight"], reference["2.classifier.0.bias"], reference["2.classifier.3.weight"],
                    reference["2.classifier.3.bias"]), fp32=False)
    loss_r = F.binary_cross_entropy_with_logits(logits_r, labels.double())
    loss_r.backward()
    assert abs(loss.item() - loss_r.item()) <= 2e-2
    _close(xd.grad, xr.grad, 5e-2)
    for name, parameter in modules.named_parameters():
        assert parameter.grad is not None, name
        _close(parameter.grad, reference[name].grad, 5e-2)


@pytest.mark.parametrize("qk_norm", [True, False])
def test_block_trains_under_the_role_mask(device, qk_norm):
    """The block as the Symbiosis model runs it in training: scattered padding, the role mask of
    ``MetadataAttentionMask`` (experiments/symbiosis/attention.py:21-60) and, by default, query / key norms. Output and
    the gradient of the input and of every parameter against float64 autograd of the oracle's block under the dense
    mask."""
    from taac_2026_amd.api import MetadataAttentionMask

    batch, d_model, heads, mult = 3, 128, 4, 2
    roles = torch.tensor([0, 1] + [2] * 5 + [3] * 4 + [4] * 3 + [5] * 2 + [6] * 40 + [7] * 4)
    tokens = roles.numel()
    g = torch.Generator().manual_seed(21)
    block = UnifiedInteractionBlock(d_model, heads, mult, qk_norm=qk_norm)
    with torch.no_grad():
        for parameter in block.parameters():
            if parameter.ndim == 1:
                parameter.copy_((1.0 if parameter.mean() > 0.5 else 0.0) + 0.1 * torch.randn(parameter.shape, generator=g))
            else:
                parameter.copy_(torch.randn(parameter.shape, generator=g) * parameter.shape[1] ** -0.5)
    block = block.to(torch.bfloat16)
    reference = {name: value.detach().double().requires_grad_(True) for name, value in block.named_parameters()}
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)
    grad_out = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)
    padding = torch.rand(batch, tokens, generator=g) < 0.3
    padding[:, :2] = False

    block = block.to(device).train()
    xd = x.to(device).requires_grad_(True)
    mask = MetadataAttentionMask(enabled=True)(padding.to(device), roles.to(device))
    out, attn_tokens = block(xd, padding.to(device), mask)
    out.backward(grad_out.to(device))

    names = {"attn_norm.weight": "attn_norm.weight", "qkv.weight": "attention.qkv.weight", "qkv.bias": "attention.qkv.bias",
             "out.weight": "attention.out.weight", "out.bias": "attention.out.bias", "ffn_norm.weight": "ffn_norm.weight",
             "up.weight": "ffn.up.weight", "up.bias": "ffn.up.bias", "down.weight": "ffn.down.weight",
             "down.bias": "ffn.down.bias"}
    if qk_norm:
        names.update({"query_norm.weight": "attention.query_norm.weight", "key_norm.weight": "attention.key_norm.weight"})
    xr = x.double().requires_grad_(True)
    want, want_attn = oracle.interaction_block(xr, padding, mask.dense().cpu(), {s: reference[f] for s, f in names.items()},
                                               num_heads=heads)
    want.backward(grad_out.double())
    _close(out, want.detach(), 3e-2)
    _close(attn_tokens, want_attn.detach(), 3e-2)
    _close(xd.grad, xr.grad, 5e-2)
    for name, parameter in block.named_parameters():
        assert parameter.grad is not None, name
        _close(parameter.grad, reference[name].grad, 5e-2)


@pytest.mark.parametrize("model_mask", ["role", "window"])
def test_block_training_route_under_a_structured_mask_equals_the_layer_by_layer_route(device, monkeypatch, model_mask):
    """Scattered padding and a structured mask built from it (the Symbiosis role mask; a TokenFormer window layer whose
    padded queries keep themselves): the one-function route over the valid rows against the layer-by-layer autograd
    route of the same module - outputs, input gradient, every parameter gradient; padded positions pass through bit
    for bit, an all-padded sample included."""
    import taac_2026_amd.modeling.backbone as backbone_module
    from taac_2026_amd.api import MetadataAttentionMask, bfts_attention_mask, build_structured_mask

    batch, d_model, heads, mult = 4, 256, 8, 2
    if model_mask == "role":
        roles = torch.tensor([0, 1] + [2] * 9 + [3] * 7 + [4] * 3 + [5] * 2 + [6] * 100 + [7] * 5)
    else:
        roles = torch.tensor([0] * 10 + [4] + [1] * 90 + [4] + [2] * 10 + [5] * 7 + [3])
    tokens = roles.numel()
    g = torch.Generator().manual_seed(5)
    block = UnifiedInteractionBlock(d_model, heads, mult, qk_norm=True)
    with torch.no_grad():
        for parameter in block.parameters():
            if parameter.ndim == 1:
                parameter.copy_((1.0 if parameter.mean() > 0.5 else 0.0) + 0.1 * torch.randn(parameter.shape, generator=g))
            else:
                parameter.copy_(torch.randn(parameter.shape, generator=g) * parameter.shape[1] ** -0.5)
    block = block.to(torch.bfloat16).to(device).train()
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    padding = torch.rand(batch, tokens, generator=g) < 0.35
    padding[:, :2] = False
    padding[:, -1] = False
    padding[2] = True                                          # an all-padded sample
    padding = padding.to(device)
    if model_mask == "role":
        mask = MetadataAttentionMask(enabled=True)(padding, roles.to(device))
    else:
        layer = bfts_attention_mask(padding, roles.to(device), 4, 6, seq_causal=True, seq_keep_per_domain=32)
        # the layer's structure over exactly the non-padded keys, padded queries keeping themselves, stated as built from
        # this padding mask (which is what lets a block skip the padded rows)
        mask = build_structured_mask(layer.structural, ~padding, padding, padding_source=padding)
    assert mask.padding_source is padding
    grad_out = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    grad_attn = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    taken = []
    real = backbone_module.run_training_block

    def run(compact: bool):
        if compact:
            monkeypatch.setattr(backbone_module, "run_training_block", lambda *a, **k: (taken.append(1), real(*a, **k))[1])
        else:
            monkeypatch.setattr(backbone_module, "training_route_applies", lambda *a, **k: False)
        xd = x.clone().requires_grad_(True)
        block.zero_grad(set_to_none=True)
        out, attn_tokens = block(xd, padding, mask)
        torch.autograd.backward([out, attn_tokens], [grad_out, grad_attn])
        monkeypatch.undo()
        return out.detach(), attn_tokens.detach(), xd.grad, {n: p.grad.clone() for n, p in block.named_parameters()}

    out_c, attn_c, gx_c, grads_c = run(True)
    assert taken == [1]                                        # the call took the one-function route
    out_s, attn_s, gx_s, grads_s = run(False)
    _close(out_c, out_s.cpu(), 1e-2)
    _close(attn_c, attn_s.cpu(), 1e-2)
    pad = padding.cpu()
    assert torch.equal(out_c.cpu()[pad], x.cpu()[pad]) and torch.equal(attn_c.cpu()[pad], x.cpu()[pad])
    assert torch.equal(gx_c.cpu()[pad], (grad_out + grad_attn).cpu()[pad])
    _close(gx_c, gx_s.cpu(), 3e-2)
    for name in grads_s:
        _close(grads_c[name], grads_s[name].cpu(), 3e-2)


@pytest.mark.parametrize("qk_norm", [False, True])
def test_backbone_module_trains(device, qk_norm):
    """``PCVRBackbone`` under autograd (blocks through the one-function route, masked mean + head as tensor operations):
    probabilities, and the gradient of a binary cross-entropy loss with respect to the embeddings and every parameter,
    against float64 autograd of the oracle's backbone; under ``torch.no_grad()`` the same module runs the one-call
    forward and returns the same probabilities."""
    from taac_2026_amd.api import PCVRBackbone

    batch, tokens, d_model, heads, d_ff = 4, 40, 128, 4, 256
    g = torch.Generator().manual_seed(31)
    model = PCVRBackbone(d_model=d_model, num_heads=heads, d_ff=d_ff, n_blocks=2, qk_norm=qk_norm)
    with torch.no_grad():
        for parameter in model.parameters():
            if parameter.ndim == 1:
                parameter.copy_((1.0 if parameter.mean() > 0.5 else 0.0) + 0.1 * torch.randn(parameter.shape, generator=g))
            else:
                parameter.copy_(torch.randn(parameter.shape, generator=g) * parameter.shape[1] ** -0.5)
    model = model.to(torch.bfloat16)
    reference = {name: value.detach().double().requires_grad_(True) for name, value in model.named_parameters()}
    emb = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16)
    lengths = torch.tensor([40, 9, 1, 25], dtype=torch.int32)
    labels = torch.tensor([1.0, 0.0, 1.0, 0.0])

    model = model.to(device).train()
    emb_d = emb.to(device).requires_grad_(True)
    p = model(emb_d, lengths.to(device))
    assert p.dtype == torch.float32 and p.shape == (batch,)
    F.binary_cross_entropy(p, labels.to(device)).backward()
    with torch.no_grad():
        served = model(emb.to(device), lengths.to(device))
    torch.testing.assert_close(p.detach(), served, rtol=0, atol=1e-2)

    emb_r = emb.double().requires_grad_(True)
    blocks = [{name.split(".", 2)[2]: value for name, value in reference.items() if name.startswith(f"blocks.{i}.")}
              for i in range(2)]
    want = oracle.backbone(emb_r, lengths, blocks, reference["head.weight"], reference["head.bias"], num_heads=heads)
    F.binary_cross_entropy(want.double(), labels.double()).backward()
    torch.testing.assert_close(p.detach().cpu().double(), want.detach().double(), rtol=0, atol=2e-2)
    _close(emb_d.grad, emb_r.grad, 5e-2)
    for name, parameter in model.named_parameters():
        assert parameter.grad is not None, name
        _close(parameter.grad, reference[name].grad, 5e-2)


@pytest.mark.parametrize("gate_first", [True, False])
def test_feed_forward_with_dropout_of_the_hidden_state(device, gate_first):
    """``down(dropout(silu(gate) * value))`` (experiments/symbiosis/backbone.py:19-21) under a fixed keep mask: output and
    every gradient against float64 autograd of the same formula; without a mask one is drawn from torch's generator."""
    from taac_2026_amd.api import swiglu_ffn_dropout

    rows, d_model, hidden, p = 300, 128, 256, 0.25
    g = torch.Generator().manual_seed(8)
    x = torch.randn(rows, d_model, generator=g).to(torch.bfloat16)
    w_up = (torch.randn(2 * hidden, d_model, generator=g) * d_model ** -0.5).to(torch.bfloat16)
    b_up = (0.1 * torch.randn(2 * hidden, generator=g)).to(torch.bfloat16)
    w_down = (torch.randn(d_model, hidden, generator=g) * hidden ** -0.5).to(torch.bfloat16)
    b_down = (0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
    keep = torch.rand(rows, hidden, generator=g) >= p
    grad_out = torch.randn(rows, d_model, generator=g).to(torch.bfloat16)
    ref = [t.double().requires_grad_(True) for t in (x, w_up, b_up, w_down, b_down)]
    first, second = F.linear(ref[0], ref[1], ref[2]).chunk(2, dim=-1)
    hidden_r = (F.silu(first) * second) if gate_first else (first * F.silu(second))
    want = ref[0] + F.linear(hidden_r * keep.double() / (1.0 - p), ref[3], ref[4])
    want.backward(grad_out.double())
    dev = [t.to(device).requires_grad_(True) for t in (x, w_up, b_up, w_down, b_down)]
    out = swiglu_ffn_dropout(dev[0], dev[1], dev[2], dev[3], dev[4], dropout_p=p, residual=dev[0], gate_first=gate_first,
                             keep_mask=keep.to(device))
    out.backward(grad_out.to(device))
    _close(out, want.detach(), 2e-2)
    for got, expected in zip(dev, ref):
        _close(got.grad, expected.grad, 3e-2)
    torch.manual_seed(3)
    a = swiglu_ffn_dropout(dev[0].detach(), dev[1], dev[2], dev[3], dev[4], dropout_p=p)
    torch.manual_seed(3)
    b = swiglu_ffn_dropout(dev[0].detach(), dev[1], dev[2], dev[3], dev[4], dropout_p=p)
    c = swiglu_ffn_dropout(dev[0].detach(), dev[1], dev[2], dev[3], dev[4], dropout_p=p)
    assert torch.equal(a, b) and not torch.equal(a, c)


def test_block_training_route_takes_float32_master_parameters(device, monkeypatch):
    """Mixed-precision training keeps float32 parameters: the one-function route casts them to bf16 on the way in and the
    gradients arrive in float32, equal to those of the layer-by-layer route of the same module."""
    import taac_2026_amd.modeling.backbone as backbone_module

    batch, tokens, d_model, heads = 3, 64, 128, 4
    g = torch.Generator().manual_seed(13)
    block = UnifiedInteractionBlock(d_model, heads, 2, qk_norm=True).to(device).train()      # float32 parameters
    x = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    lengths = torch.tensor([64, 20, 1], dtype=torch.int32, device=device)
    padding = torch.arange(tokens, device=device)[None, :] >= lengths[:, None]
    grad_out = torch.randn(batch, tokens, d_model, generator=g).to(torch.bfloat16).to(device)
    taken = []
    real = backbone_module.run_training_block

    def run(compact: bool):
        if compact:
            monkeypatch.setattr(backbone_module, "run_training_block", lambda *a, **k: (taken.append(1), real(*a, **k))[1])
        else:
            monkeypatch.setattr(backbone_module, "training_route_applies", lambda *a, **k: False)
        xd = x.clone().requires_grad_(True)
        block.zero_grad(set_to_none=True)
        out, _ = block(xd, padding, None, key_lengths=lengths, return_attention_tokens=False)
        out.backward(grad_out)
        monkeypatch.undo()
        return out.detach(), xd.grad, {n: p.grad.clone() for n, p in block.named_parameters()}

    out_c, gx_c, grads_c = run(True)
    assert taken == [1]
    out_s, gx_s, grads_s = run(False)
    _close(out_c, out_s.cpu(), 1e-2)
    _close(gx_c, gx_s.cpu(), 3e-2)
    for name, grad in grads_c.items():
        assert grad.dtype == torch.float32, name
        _close(grad, grads_s[name].cpu(), 3e-2)
