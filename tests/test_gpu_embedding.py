"""GPU parity: multi-hot embedding lookup with mean pooling (through the C ABI) against the CPU oracle."""

from __future__ import annotations

import pytest
import torch

from oracle import reference as oracle
from taac_2026_amd.api import embedding_bag_mean

pytestmark = pytest.mark.gpu

# tolerances of the reference's operator benchmark (pcvr_tilelang_ops_benchmark.py:177-184)
TOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 2e-2}


def test_reference_fixture(device):
    """The id matrix of the reference's own test (tests/unit/infrastructure/accelerators/test_tilelang_ops.py:123-140)."""
    weight = torch.randn(8, 5, generator=torch.Generator().manual_seed(0))
    values = torch.tensor([[1, 2, 0, 4], [0, 0, 0, 0], [3, 3, 7, 0]], dtype=torch.long)
    with torch.no_grad():
        got = embedding_bag_mean(weight.to(device), values.to(device)).cpu()
    torch.testing.assert_close(got, oracle.embedding_bag_mean(weight, values), rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(got, oracle.embedding_bag_mean_closed_form(weight, values), rtol=1e-6, atol=1e-6)
    assert got[1].abs().max().item() == 0.0


def test_golden_vectors(device):
    """The committed pure-Python float64 evaluations (tests/golden/qk_rope_embedding_small.json)."""
    import json
    from pathlib import Path

    golden = json.loads((Path(__file__).resolve().parent / "golden" / "qk_rope_embedding_small.json").read_text())
    for case in golden["bags"]:
        weight, values = torch.tensor(case["weight"]), torch.tensor(case["values"])
        for index_dtype in (torch.int32, torch.int64):
            with torch.no_grad():
                got = embedding_bag_mean(weight.to(device), values.to(index_dtype).to(device)).cpu()
            torch.testing.assert_close(got.double(), torch.tensor(case["out"], dtype=torch.float64), rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("vocab,dim,bags,bag_size", [(1000, 64, 257, 4), (50, 8, 33, 1), (4096, 128, 100, 7),
                                                      (300, 100, 19, 5), (2000, 1024, 9, 3), (64, 4096, 3, 2), (77, 5, 40, 9)])
def test_matches_oracle(device, dtype, index_dtype, vocab, dim, bags, bag_size):
    g = torch.Generator().manual_seed(vocab + dim + bags)
    weight = torch.randn(vocab, dim, generator=g).to(dtype)
    values = torch.randint(0, vocab, (bags, bag_size), generator=g)
    values[torch.rand(bags, bag_size, generator=g) < 0.25] = 0      # the reference benchmark's padding probability
    values[0] = 0                                                    # a bag of padding only
    expected = oracle.embedding_bag_mean_closed_form(weight, values)
    with torch.no_grad():
        got = embedding_bag_mean(weight.to(device), values.to(index_dtype).to(device))
    assert got.shape == (bags, dim) and got.dtype == dtype
    torch.testing.assert_close(got.cpu().float(), expected, rtol=TOL[dtype], atol=TOL[dtype])
    assert got[0].abs().max().item() == 0.0
    if dtype == torch.float32:
        torch.testing.assert_close(got.cpu(), oracle.embedding_bag_mean(weight, values), rtol=1e-5, atol=1e-5)


def test_benchmark_shape_and_properties(device):
    """The reference benchmark's default shape (vocabulary 1 000 000 x 64, bags of 4, fp16) at a batch that fills the
    device: a slice against the oracle, and two size-independent properties - a bag's mean does not depend on the
    order of its ids, and a table of constant rows returns that constant for every non-empty bag."""
    vocab, dim, bags, bag_size = 1_000_000, 64, 262_144, 4
    g = torch.Generator().manual_seed(42)
    weight = torch.randn(vocab, dim, generator=g).to(torch.float16)
    values = torch.randint(1, vocab, (bags, bag_size), generator=g)
    values[torch.rand(bags, bag_size, generator=g) < 0.25] = 0
    with torch.no_grad():
        dev_w, dev_v = weight.to(device), values.to(device)
        got = embedding_bag_mean(dev_w, dev_v)
        flipped = embedding_bag_mean(dev_w, dev_v.flip(1).contiguous())
        ones = embedding_bag_mean(torch.full_like(dev_w, 0.5), dev_v)
    pick = torch.arange(0, bags, 1021)
    torch.testing.assert_close(got[pick.to(device)].cpu().float(), oracle.embedding_bag_mean_closed_form(weight, values[pick]),
                               rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got.float(), flipped.float(), rtol=0, atol=2e-3)
    nonempty = (values != 0).any(dim=1).to(device)
    assert (ones[nonempty] == 0.5).all() and (ones[~nonempty] == 0).all()


def test_argument_errors_and_index_check(device):
    weight = torch.randn(16, 8, device=device)
    values = torch.tensor([[1, 2], [3, 0]], device=device)
    with pytest.raises(ValueError, match="weight must be a 2D tensor"):
        embedding_bag_mean(weight[0], values)
    with pytest.raises(ValueError, match="values must be a 2D tensor"):
        embedding_bag_mean(weight, values[0])
    with pytest.raises(RuntimeError, match="int32 or int64"):
        embedding_bag_mean(weight, values.float())
    with pytest.raises(RuntimeError, match="does not support dtype"):
        embedding_bag_mean(weight.double(), values)
    with pytest.raises(RuntimeError, match="CUDA"):
        embedding_bag_mean(weight.cpu(), values.cpu())
    with pytest.raises(ValueError, match="unsupported embedding_bag_mean backend"):
        embedding_bag_mean(weight, values, backend="numpy")
    bad = torch.tensor([[1, 99], [-3, 2]], device=device)
    with torch.no_grad():
        skipped = embedding_bag_mean(weight, bad)        # out-of-range ids are skipped like padding ...
        torch.testing.assert_close(skipped[0], weight[1])
        torch.testing.assert_close(skipped[1], weight[2])
        with pytest.raises(IndexError, match="2 ids are outside"):   # ... or reported, at the price of a host sync
            embedding_bag_mean(weight, bad, check_indices=True)
        assert embedding_bag_mean(weight, values, check_indices=True).shape == (2, 8)


def _loop_gradient(values: torch.Tensor, grad_out: torch.Tensor, num_embeddings: int) -> torch.Tensor:
    """The backward kernel's definition slot by slot (embedding/kernels/triton.py:105-150): each valid id of bag b
    receives grad_out[b] / count_b."""
    grad = torch.zeros(num_embeddings, grad_out.shape[1], dtype=torch.float64)
    for b in range(values.shape[0]):
        ids = [int(i) for i in values[b] if 0 < int(i) < num_embeddings]
        for i in ids:
            grad[i] += grad_out[b].double() / len(ids)
    return grad


def test_backward_reference_fixture(device):
    """The id matrix of the reference's own test: table gradient against float64 autograd of the torch operator and
    against the slot-by-slot loop."""
    g = torch.Generator().manual_seed(0)
    weight = torch.randn(8, 5, generator=g)
    values = torch.tensor([[1, 2, 0, 4], [0, 0, 0, 0], [3, 3, 7, 0]], dtype=torch.long)
    grad_out = torch.randn(3, 5, generator=g)
    dev_w = weight.to(device).requires_grad_(True)
    out = embedding_bag_mean(dev_w, values.to(device))
    out.backward(grad_out.to(device))
    ref_w = weight.double().requires_grad_(True)
    oracle.embedding_bag_mean(ref_w, values).backward(grad_out.double())
    torch.testing.assert_close(ref_w.grad, _loop_gradient(values, grad_out, 8), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(dev_w.grad.cpu().double(), ref_w.grad, rtol=1e-6, atol=1e-6)
    assert dev_w.grad[0].abs().max().item() == 0.0 and dev_w.grad[5].abs().max().item() == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("bags,bag_size,rows,dim", [(257, 7, 50, 64), (64, 1, 1000, 8), (33, 20, 9, 72), (5, 3, 40, 301),
                                                    (1000, 4, 3, 32)])
def test_backward_matches_autograd_of_the_oracle(device, dtype, index_dtype, bags, bag_size, rows, dim):
    g = torch.Generator().manual_seed(bags + dim)
    weight = torch.randn(rows, dim, generator=g).to(dtype)
    values = torch.randint(0, rows, (bags, bag_size), generator=g)
    values[torch.rand(bags, bag_size, generator=g) < 0.3] = 0
    values[0] = 0                                                            # a bag of padding only
    grad_out = torch.randn(bags, dim, generator=g).to(dtype)
    dev_w = weight.to(device).requires_grad_(True)
    out = embedding_bag_mean(dev_w, values.to(index_dtype).to(device))
    out.backward(grad_out.to(device))
    assert dev_w.grad.dtype == dtype and dev_w.grad.shape == weight.shape
    ref_w = weight.double().requires_grad_(True)
    oracle.embedding_bag_mean(ref_w, values).backward(grad_out.double())
    scale = ref_w.grad.abs().max().item()
    error = (dev_w.grad.cpu().double() - ref_w.grad).abs().max().item()
    # fp32 sums rounded once: half a unit in the last place of the largest sum for the 16-bit tables
    assert error <= {torch.float32: 1e-5, torch.float16: 2 ** -10, torch.bfloat16: 2 ** -7}[dtype] * max(scale, 1.0), (error, scale)
    untouched = torch.ones(rows, dtype=torch.bool)
    untouched[values.unique()] = False
    untouched[0] = True
    assert dev_w.grad[untouched.to(device)].abs().max().item() == 0.0


def test_backward_skips_ids_outside_the_table_and_needs_no_gradient_when_frozen(device):
    from taac_2026_amd.accelerators.embedding import hip_embedding_bag_mean_backward_kernel

    g = torch.Generator().manual_seed(4)
    values = torch.tensor([[1, 99, -3, 2], [0, 5, 5, 16], [99, -1, 0, 0]], dtype=torch.int64)
    grad_out = torch.randn(3, 16, generator=g)
    got = hip_embedding_bag_mean_backward_kernel(values.to(device), grad_out.to(device), 16)
    torch.testing.assert_close(got.cpu().double(), _loop_gradient(values, grad_out, 16), rtol=1e-6, atol=1e-6)
    empty = hip_embedding_bag_mean_backward_kernel(values[:0].to(device), grad_out[:0].to(device), 16)
    assert empty.shape == (16, 16) and empty.abs().max().item() == 0.0
    weight = torch.randn(16, 16, generator=g).to(device)
    assert not embedding_bag_mean(weight, values.clamp(0, 15).to(device)).requires_grad
