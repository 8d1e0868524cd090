"""The entry point that allocates nothing (``taac_rmsnorm_bwd_static``: partial sums in a device array of the library
image) against ``taac_rmsnorm_bwd`` with a caller workspace: bit-identical, on two calls in a row, the second smaller."""

from __future__ import annotations

import pytest
import torch

from taac_2026_amd import _native

pytestmark = pytest.mark.gpu


def _call_pair(device, rows, cols, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g).to(dtype).to(device)
    w = (1 + 0.1 * torch.randn(cols, generator=g)).to(dtype).to(device)
    dy = torch.randn(rows, cols, generator=g).to(dtype).to(device)
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


def test_static_scratch_variant_matches_the_workspace_variant(device):
    # two calls in a row share the device array; the second is smaller (fewer workgroups, narrower rows), so stale
    # partial rows of the first call lie behind what it writes and must not be read
    _call_pair(device, 40000, 2048, torch.bfloat16, seed=1)
    _call_pair(device, 777, 256, torch.bfloat16, seed=2)
    # a width that takes the generic kernel, fp32, then a wide fp32 row
    _call_pair(device, 300, 100, torch.float32, seed=3)
    _call_pair(device, 64, 2048, torch.float32, seed=4)


def test_static_scratch_variant_rejects_widths_beyond_the_array(device):
    library = _native.load_library()
    x = torch.zeros(4, 4096, dtype=torch.bfloat16, device=device)
    w = torch.ones(4096, dtype=torch.bfloat16, device=device)
    status = library.taac_rmsnorm_bwd_static(x.data_ptr(), w.data_ptr(), x.data_ptr(), x.data_ptr(), w.data_ptr(), 4, 4096,
                                             1e-6, _native.TAAC_BF16, _native.current_stream(device))
    assert status == _native.TAAC_ERR_UNSUPPORTED
    assert b"2048" in library.taac_last_error()
