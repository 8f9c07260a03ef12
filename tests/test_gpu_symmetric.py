"""Symmetric policy: a matrix times its own transpose computes the lower triangle and mirrors it.

Mirrors the reference's test (tests/test_cuda.py:104-109: the result is close to the product, equal
to its own transpose bit for bit, and counted as `gram`), extended over both orders, ragged sizes,
padded operands and the calls the policy must leave alone. The answer is a CPU FP64 product.
"""

import pytest
import torch

from camblas_amd import _kernels as cb

pytestmark = pytest.mark.gpu
DTYPES = (torch.float32, torch.float64)


def assert_close(actual, expected):
    rtol, atol = (1e-5, 3e-6) if actual.dtype == torch.float32 else (2e-13, 3e-14)
    torch.testing.assert_close(actual.cpu(), expected.to(actual.dtype), rtol=rtol, atol=atol)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(512, 512), (300, 77), (77, 300), (1000, 130), (20, 9), (129, 64)])
def test_gram_is_counted_close_and_symmetric(device, dtype, shape):
    torch.manual_seed(shape[0])
    a = torch.randn(shape, device=device, dtype=dtype) / shape[0] ** 0.5
    host = a.double().cpu()
    with cb.algorithm("symmetric"):
        cb.stats(reset=True)
        inner = cb.matmul(a.T, a)
        outer = cb.matmul(a, a.T)
        counts = cb.stats()
    assert counts["gram"] == 2 and counts["classical"] == 0, counts
    assert_close(inner, host.T @ host)
    assert_close(outer, host @ host.T)
    assert torch.equal(inner, inner.T) and torch.equal(outer, outer.T)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gram_of_a_padded_operand_over_a_poisoned_output(device, dtype):
    torch.manual_seed(2)
    wide = torch.randn((260, 200), device=device, dtype=dtype) / 16
    a = wide[:, :150]  # row stride 200
    out = torch.full((150, 150), float("nan"), device=device, dtype=dtype)
    with cb.algorithm("symmetric"):
        cb.stats(reset=True)
        cb.matmul(a.T, a, out=out, alpha=0.5)
        assert cb.stats()["gram"] == 1
    host = a.double().cpu()
    assert_close(out, 0.5 * (host.T @ host))
    assert torch.equal(out, out.T)


@pytest.mark.parametrize("dtype", DTYPES)
def test_products_the_policy_leaves_alone(device, dtype):
    """Different operands, an accumulating call and an untransposed square are ordinary products."""
    torch.manual_seed(3)
    a = torch.randn((256, 256), device=device, dtype=dtype) / 16
    b = a.clone()
    c = torch.randn_like(a)
    host, start = a.double().cpu(), c.double().cpu()
    with cb.algorithm("symmetric"):
        cb.stats(reset=True)
        assert_close(cb.matmul(a.T, b), host.T @ host)
        assert_close(cb.matmul(a, a), host @ host)
        cb.matmul(a.T, a, out=c, beta=1.0)
        assert_close(c, host.T @ host + start)
        counts = cb.stats()
    assert counts["gram"] == 0, counts
    with cb.algorithm("auto"):
        cb.stats(reset=True)
        cb.matmul(a.T, a)
        assert cb.stats()["gram"] == 0
