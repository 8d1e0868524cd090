"""The entry point that allocates nothing (``taac_rmsnorm_bwd_static``: partial sums in a device array of the library
image) against ``taac_rmsnorm_bwd`` with a caller workspace: bit-identical, on two calls in a row, the second smaller."""

from __future__ import annotations

import pytest
import torch

from taac_2026_amd import _native

pytestmark = pytest.mark.gpu


def _unaligned(t: torch.Tensor, device) -> torch.Tensor:
    """A contiguous device copy of ``t`` whose base address is one element past a 16-byte boundary."""
    flat = torch.empty(t.numel() + 1, dtype=t.dtype, device=device)
    view = flat[1:].view(t.shape)
    view.copy_(t)
    assert view.data_ptr() % 16 != 0
    return view


def _call_pair(device, rows, cols, dtype, seed, *, unaligned=False, check_oracle=False):
    g = torch.Generator().manual_seed(seed)
    place = (lambda t: _unaligned(t, device)) if unaligned else (lambda t: t.to(device))
    x_cpu = torch.randn(rows, cols, generator=g).to(dtype)
    w_cpu = (1 + 0.1 * torch.randn(cols, generator=g)).to(dtype)
    dy_cpu = torch.randn(rows, cols, generator=g).to(dtype)
    x, w, dy = place(x_cpu), place(w_cpu), place(dy_cpu)
    library = _native.load_library()
    stream = _native.current_stream(device)
    code = _native.dtype_code(dtype)
    floats = int(library.taac_norm_bwd_workspace_floats(rows, cols, 0))
    workspace = torch.empty(floats, dtype=torch.float32, device=device)
    dx_ref, dw_ref = torch.empty_like(x), torch.empty_like(w)
    _native.check(library.taac_rmsnorm_bwd(x.data_ptr(), w.data_ptr(), dy.data_ptr(), dx_ref.data_ptr(), dw_ref.data_ptr(),
                                           workspace.data_ptr(), floats, rows, cols, 1e-6, code, stream), "rmsnorm_bwd")
    dx, dw = torch.full_like(x, float("nan")), torch.full_like(w, float("nan"))
    _native.check(library.taac_rmsnorm_bwd_static(x.data_ptr(), w.data_ptr(), dy.data_ptr(), dx.data_ptr(), dw.data_ptr(),
                                                  rows, cols, 1e-6, code, stream), "rmsnorm_bwd_static")
    torch.cuda.synchronize()
    assert torch.equal(dx, dx_ref), (rows, cols, dtype)
    assert torch.equal(dw, dw_ref), (rows, cols, dtype)
    assert torch.isfinite(dw.float()).all()
    if check_oracle:  # float64 autograd of the oracle's closed form from the stored (rounded) inputs
        import oracle.reference as oracle

        xr, wr = x_cpu.double().requires_grad_(True), w_cpu.double().requires_grad_(True)
        oracle.rms_norm(xr, wr, 1e-6).backward(dy_cpu.double())
        tol = 3e-2 if dtype == torch.bfloat16 else 1e-4
        torch.testing.assert_close(dx.cpu().double(), xr.grad, rtol=tol, atol=tol)
        torch.testing.assert_close(dw.cpu().double(), wr.grad, rtol=tol, atol=tol * max(1.0, wr.grad.abs().max().item()))


def test_static_scratch_variant_matches_the_workspace_variant(device):
    # two calls in a row share the device array; the second is smaller (fewer workgroups, narrower rows), so stale
    # partial rows of the first call lie behind what it writes and must not be read
    _call_pair(device, 40000, 2048, torch.bfloat16, seed=1)
    _call_pair(device, 777, 256, torch.bfloat16, seed=2)
    # a width that takes the generic kernel, fp32, then a wide fp32 row
    _call_pair(device, 300, 100, torch.float32, seed=3)
    _call_pair(device, 64, 2048, torch.float32, seed=4)
    # the generic kernel with 16-bit rows of an odd width at base addresses off the 16-byte grid, against the oracle too
    _call_pair(device, 1201, 101, torch.bfloat16, seed=5, unaligned=True, check_oracle=True)
    _call_pair(device, 97, 7, torch.bfloat16, seed=6, unaligned=True, check_oracle=True)


def test_static_scratch_variant_rejects_widths_beyond_the_array(device):
    library = _native.load_library()
    x = torch.zeros(4, 4096, dtype=torch.bfloat16, device=device)
    w = torch.ones(4096, dtype=torch.bfloat16, device=device)
    status = library.taac_rmsnorm_bwd_static(x.data_ptr(), w.data_ptr(), x.data_ptr(), x.data_ptr(), w.data_ptr(), 4, 4096,
                                             1e-6, _native.TAAC_BF16, _native.current_stream(device))
    assert status == _native.TAAC_ERR_UNSUPPORTED
    assert b"2048" in library.taac_last_error()
