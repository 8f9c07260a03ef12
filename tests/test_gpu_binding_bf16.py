"""BF16 products through the binding after the reference's tests/test_bfloat16.py:54-147: every
transpose pair under every policy with padding, strided views and nonzero beta on changed
operands; unused inputs for zero scalars; empty shapes; NaN placement; argument validation.
"""

import pytest
import torch

from camblas_amd import _native

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def binding():
    module = _native.tensor_module()
    assert module is not None
    return module


def assert_product(actual, a, b, alpha=1, beta=0, old=None):
    # ref: tests/test_bfloat16.py:24-52
    expected = alpha * (a.cpu().double() @ b.cpu().double())
    if beta:
        expected += beta * old.cpu().double()
    torch.testing.assert_close(actual.cpu().double(), expected, rtol=0.02, atol=0.02)


@pytest.mark.parametrize("policy", ["auto", "classical", "lt", "strassen4"])
def test_layouts_scalars_and_changed_weights(binding, device, policy):
    torch.manual_seed(54)
    algorithm = _native.ALGORITHMS[policy]
    for ta in (False, True):
        for tb in (False, True):
            a = torch.randn((13, 17) if ta else (17, 13), dtype=torch.bfloat16, device=device) / 4
            b = torch.randn((23, 13) if tb else (13, 23), dtype=torch.bfloat16, device=device) / 4
            a, b = (a.T if ta else a), (b.T if tb else b)
            assert_product(binding.matmul_public(a, b, algorithm=algorithm), a, b)
            c = torch.full((17, 23), float("nan"), dtype=torch.bfloat16, device=device)
            binding.matmul_public(a, b, out=c, algorithm=algorithm)
            assert_product(c, a, b)
            a.add_(0.125)
            b.mul_(-0.5)
            old = torch.randn_like(c)
            c.copy_(old)
            binding.matmul_public(a, b, out=c, alpha=-0.7, beta=0.3, algorithm=algorithm)
            assert_product(c, a, b, -0.7, 0.3, old)
    a = torch.randn((17, 26), dtype=torch.bfloat16, device=device)[:, ::2]
    b = torch.randn((13, 31), dtype=torch.bfloat16, device=device)[:, :23]
    assert_product(binding.matmul_public(a, b, algorithm=algorithm), a, b)


def test_empty_zero_alpha_exceptional_and_validation(binding, device):
    a = torch.full((5, 7), float("nan"), dtype=torch.bfloat16, device=device)
    b = torch.full((7, 3), float("inf"), dtype=torch.bfloat16, device=device)
    c = torch.full((5, 3), float("nan"), dtype=torch.bfloat16, device=device)
    binding.matmul_public(a, b, out=c, alpha=0.0, beta=0.0)
    assert not c.view(torch.int16).any()
    c.fill_(3)
    binding.matmul_public(a, b, out=c, alpha=0.0, beta=-0.5)
    torch.testing.assert_close(c, torch.full_like(c, -1.5), rtol=0, atol=0)
    for m, k, n in ((0, 7, 3), (5, 7, 0), (5, 0, 3)):
        a = torch.empty((m, k), dtype=torch.bfloat16, device=device)
        b = torch.empty((k, n), dtype=torch.bfloat16, device=device)
        output = binding.matmul_public(a, b)
        assert output.shape == (m, n) and not output.view(torch.int16).any()
    a = torch.eye(8, dtype=torch.bfloat16, device=device)
    b = torch.ones_like(a)
    b[2, 3] = float("nan")
    # every output of column 3 sums a 0 * NaN term: the whole column is NaN, nothing else is
    wanted = torch.ones((8, 8), dtype=torch.bfloat16)
    wanted[:, 3] = float("nan")
    for policy in ("auto", "lt"):
        got = binding.matmul_public(a, b, algorithm=_native.ALGORITHMS[policy])
        torch.testing.assert_close(got.cpu(), wanted, equal_nan=True, rtol=0, atol=0)
    with pytest.raises(ValueError):
        binding.matmul_public(a.half(), b.half())
    with pytest.raises(ValueError):
        binding.matmul_public(a, b.float())
    with pytest.raises(ValueError):
        binding.matmul_public(a, b, out=a)
    with pytest.raises(ValueError):
        binding.affine_public(a, b, torch.ones(8, dtype=a.dtype, device=a.device))
