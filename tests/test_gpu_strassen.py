"""Strassen policies of the FP32 / FP64 GEMM: accuracy, guard, counters, eligibility.

Mirrors the reference's tests (tests/test_cuda.py:90-123 changed inputs and guarded fallback,
:584-598 attention scores in scratch, :917-931 cancellation bound, :932-975 two and three levels)
with a CPU FP64 product as the independent answer. Element tolerances are the reference's:
rtol 1e-5 / atol 1.5e-5 for FP32, rtol 2e-13 / atol 1.5e-13 for FP64 (five times the classical atol).
"""

import pytest
import torch

from camblas_amd import _kernels as cb

pytestmark = pytest.mark.gpu
POLICIES = ("strassen", "strassen2", "strassen3", "strassen4")
DTYPES = (torch.float32, torch.float64)


def assert_close(actual, expected, strassen=True):
    rtol, atol = (1e-5, 3e-6) if actual.dtype == torch.float32 else (2e-13, 3e-14)
    if strassen:
        atol *= 5
    torch.testing.assert_close(actual.cpu(), expected.to(actual.dtype).cpu(), rtol=rtol, atol=atol,
                               equal_nan=True)


def product64(a, b):
    return a.double().cpu() @ b.double().cpu()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("policy", POLICIES)
def test_policy_counts_and_accuracy(device, dtype, policy):
    torch.manual_seed(73013)
    n = 512
    a = torch.randn((n, n), device=device, dtype=dtype) / n**0.5
    b = torch.randn_like(a) / n**0.5
    with cb.algorithm(policy):
        cb.stats(reset=True)
        assert_close(cb.matmul(a, b), product64(a, b))
        counts = cb.stats()
        assert counts["strassen"] == 1 and counts["guard_fallback"] == 0 and counts["classical"] == 0, counts
        # changed inputs are recomputed, alpha and beta are applied once, at the last recombination
        a.add_(0.02)
        b.mul_(0.5)
        assert_close(cb.matmul(a, b), product64(a, b))
        c = torch.randn_like(a) / n**0.5
        reference = 0.7 * product64(a, b) - 0.3 * c.double().cpu()
        cb.matmul(a, b, out=c, alpha=0.7, beta=-0.3)
        assert_close(c, reference)


@pytest.mark.parametrize("dtype", DTYPES)
def test_beta_zero_never_reads_output(device, dtype):
    torch.manual_seed(1)
    a = torch.randn((256, 256), device=device, dtype=dtype) / 16
    b = torch.randn_like(a) / 16
    c = torch.full_like(a, float("nan"))
    with cb.algorithm("strassen2"):
        cb.matmul(a, b, out=c)
    assert_close(c, product64(a, b))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [504, 514, 516, 520])
def test_level_boundaries_and_padded_operands(device, dtype, n):
    """Sizes divisible by 8, 2, 4 and 8: the depth follows divisibility; operands are column slices."""
    torch.manual_seed(n)
    host_a = torch.randn((n, n + 3), dtype=dtype) / n**0.5
    host_b = torch.randn((n, n + 5), dtype=dtype) / n**0.5
    a, b = host_a.to(device)[:, :n], host_b.to(device)[:, :n]
    expected = host_a[:, :n].double() @ host_b[:, :n].double()
    with cb.algorithm("strassen3"):
        cb.stats(reset=True)
        assert_close(cb.matmul(a, b), expected)
        assert cb.stats()["strassen"] == 1
        c = torch.randn((n, n), device=device, dtype=dtype)
        reference = 0.3 * expected + 0.2 * c.double().cpu()
        cb.matmul(a, b, out=c, alpha=0.3, beta=0.2)
        assert_close(c, reference)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("policy", ["strassen", "strassen3"])
def test_guarded_fallback(device, dtype, policy):
    """NaN, infinity and values whose quadrant sums could overflow take the ordinary kernel."""
    a = torch.eye(256, device=device, dtype=dtype)
    b = torch.eye(256, device=device, dtype=dtype)
    for value in (float("nan"), float("inf"), torch.finfo(dtype).max / 2):
        a[0, 0] = value
        cb.stats(reset=True)
        with cb.algorithm(policy):
            c = cb.matmul(a, b)
        assert_close(c, product64(a, b), strassen=False)  # NaN and infinity spread along their row
        counts = cb.stats()
        assert counts["guard_fallback"] == 1 and counts["strassen"] == 0, counts
    # the context stays usable, and a clean input takes the policy again
    a[0, 0] = 1.0
    cb.stats(reset=True)
    with cb.algorithm(policy):
        c = cb.matmul(a, b)
    assert torch.equal(c, a) and cb.stats()["strassen"] == 1


@pytest.mark.parametrize("dtype", DTYPES)
def test_shapes_outside_the_policy(device, dtype):
    """Odd, small, rectangular and transposed products run the ordinary kernels and count nothing."""
    torch.manual_seed(3)
    with cb.algorithm("strassen"):
        cb.stats(reset=True)
        for shape_a, shape_b in (((255, 255), (255, 255)), ((254, 254), (254, 254)),
                                 ((256, 258), (258, 256)), ((256, 256), (256, 260))):
            a = torch.randn(shape_a, device=device, dtype=dtype) / 16
            b = torch.randn(shape_b, device=device, dtype=dtype) / 16
            assert_close(cb.matmul(a, b), product64(a, b), strassen=False)
        a = torch.randn((256, 256), device=device, dtype=dtype) / 16
        b = torch.randn_like(a) / 16
        assert_close(cb.matmul(a.T, b), product64(a.T, b), strassen=False)
        counts = cb.stats()
        assert counts["strassen"] == 0 and counts["guard_fallback"] == 0, counts


@pytest.mark.parametrize("dtype", DTYPES)
def test_cancellation_bound(device, dtype):
    """Errors stay within 50 eps of the sum of the products' magnitudes when the terms cancel."""
    torch.manual_seed(5)
    a = torch.randn((256, 256), dtype=dtype) * 1e4
    b = torch.randn((256, 256), dtype=dtype) * 1e4
    a[:, 128:] = a[:, :128]
    b[128:, :] = -b[:128, :]
    b[0, 0] += 0.1
    expected = a.double() @ b.double()
    magnitudes = a.double().abs() @ b.double().abs()
    for policy in POLICIES:
        with cb.algorithm(policy):
            actual = cb.matmul(a.to(device), b.to(device)).cpu().double()
        scaled = (actual - expected).abs() / magnitudes.clamp_min(1)
        assert scaled.max().item() < 50 * torch.finfo(dtype).eps, policy


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_scores_in_scratch_are_not_split(device, dtype):
    """The second product of dense attention reads the context scratch, which the policy would reuse."""
    torch.manual_seed(7)
    q = torch.randn((512, 16), device=device, dtype=dtype) * 0.1
    k = torch.randn_like(q) * 0.1
    v = torch.randn((512, 512), device=device, dtype=dtype) * 0.1
    with cb.algorithm("strassen2"):
        cb.stats(reset=True)
        reference = torch.softmax((q.double().cpu() @ k.double().cpu().T) / 4, dim=-1) @ v.double().cpu()
        assert_close(cb.attention(q, k, v), reference, strassen=False)
        assert cb.stats()["strassen"] == 0
        q.add_(0.2)
        v.mul_(0.8)
        reference = torch.softmax((q.double().cpu() @ k.double().cpu().T) / 4, dim=-1) @ v.double().cpu()
        assert_close(cb.attention(q, k, v), reference, strassen=False)


def test_capture_runs_the_ordinary_kernel(device):
    """The guard needs a host read, so a capturing stream gets the classical product; replays agree."""
    torch.manual_seed(9)
    a = torch.randn((256, 256), device=device) / 16
    b = torch.randn_like(a) / 16
    out = torch.empty_like(a)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream), cb.algorithm("strassen"):
        cb.matmul(a, b, out=out)  # warm the context of this stream
        stream.synchronize()
        assert cb.stats(reset=True)["strassen"] == 1
        with torch.cuda.graph(graph, stream=stream):
            cb.matmul(a, b, out=out)
        counts = cb.stats()
        assert counts["strassen"] == 0 and counts["guard_fallback"] == 0, counts
    torch.cuda.current_stream().wait_stream(stream)
    for scale in (1.0, 0.5, -2.0):
        a.mul_(scale)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert_close(out, product64(a, b), strassen=False)


@pytest.mark.parametrize("dtype", DTYPES)
def test_default_policy_boundary(device, dtype):
    """Under the default policy even sizes from 8192 are split, smaller and odd ones are not
    (the reference's form of the test: tests/test_cuda.py:272-284). The answer is the FP64 classical
    product on the device, which other tests pin against the CPU."""
    torch.manual_seed(11)
    for size in (8190, 8192, 8193):
        a = torch.randn((size, size), device=device, dtype=dtype) / size**0.5
        b = torch.randn_like(a) / size**0.5
        with cb.algorithm("classical"):
            expected = cb.matmul(a.double(), b.double())
        cb.stats(reset=True)
        with cb.algorithm("auto"):
            actual = cb.matmul(a, b)
        counts = cb.stats()
        assert counts["strassen"] == int(size == 8192), (size, counts)
        difference = (actual.double() - expected).norm() / expected.norm()
        assert difference.item() <= (1e-5 if dtype == torch.float32 else 1e-13), size
        rtol, atol = (1e-5, 1.5e-5) if dtype == torch.float32 else (2e-13, 1.5e-13)
        torch.testing.assert_close(actual, expected.to(dtype), rtol=rtol, atol=atol)
        del a, b, expected, actual
