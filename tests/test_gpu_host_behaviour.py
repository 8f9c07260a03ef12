"""Host-side behaviour of the Python mirror and the tensor binding, after the reference's
tests/test_cuda.py: one context per stream (:449-462), out-tensor versions and autograd rejection
(:1091-1110), a captured product that recomputes changed inputs (:1127-1145), gradient subsets and
launch counters (:1112-1171), unaligned but contiguous views (:1201-1225), and a process that
closes its contexts, reuses the library and exits cleanly (:1173-1199).
"""

import subprocess
import sys
from pathlib import Path

import pytest
import torch

from camblas_amd import _kernels, _native

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]


def close(actual, expected):
    rtol, atol = (1e-5, 3e-6) if actual.dtype == torch.float32 else (2e-13, 3e-14)
    torch.testing.assert_close(actual.cpu(), expected.to(actual.dtype).cpu(), rtol=rtol, atol=atol)


def test_streams_get_their_own_contexts(device):
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    seen = []
    for stream in streams:
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            a = torch.randn((512, 512), device=device) / 512 ** 0.5
            b = torch.randn((512, 512), device=device) / 512 ** 0.5
            seen.append((_kernels.matmul(a, b), a, b, _native.context(device).handle.value))
    for stream in streams:
        stream.synchronize()
    assert seen[0][3] != seen[1][3]
    assert _native.context(device).handle.value not in (seen[0][3], seen[1][3])
    for actual, a, b, _ in seen:
        close(actual, a.double() @ b.double())


def test_out_tensor_versions_and_autograd_rejection(device):
    binding = _native.tensor_module()
    a = torch.eye(4, device=device)
    output = torch.ones_like(a, requires_grad=True)
    with pytest.raises(ValueError):
        binding.matmul_public(a, a, out=output)
    with torch.no_grad():
        version = output._version
        binding.matmul_public(a, a, out=output)
        assert output._version == version + 1
    # a tensor saved for backward and then overwritten through `out` is caught by autograd
    output = torch.ones_like(a)
    parameter = torch.ones_like(a, requires_grad=True)
    loss = (parameter * output).sum()
    binding.matmul_public(a, a, out=output)
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        loss.backward()
    with torch.inference_mode():
        output = torch.empty_like(a)
        binding.matmul_public(a, a, out=output)
        close(output, a)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_captured_product_recomputes_changed_inputs(device, dtype):
    a = (torch.randn((256, 256), device=device) / 16).to(dtype)
    b = (torch.randn((256, 256), device=device) / 16).to(dtype)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        for _ in range(3):
            _kernels.matmul(a, b)
        with torch.cuda.graph(graph, stream=stream):
            output = _kernels.matmul(a, b)
    torch.cuda.current_stream().wait_stream(stream)
    tolerance = 1e-5 if dtype == torch.float32 else 1e-2
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        want = a.double() @ b.double()
        assert (output.double() - want).norm() <= tolerance * want.norm()
        a.add_(0.1)
        b.mul_(0.5)
    graph.reset()


@pytest.mark.parametrize("requested", [(True, False), (False, True), (True, True)])
def test_matmul_gradient_subsets_and_counters(device, requested):
    binding = _native.tensor_module()
    a = torch.randn((7, 11), device=device, dtype=torch.float64).requires_grad_(requested[0])
    b = torch.randn((11, 5), device=device, dtype=torch.float64).requires_grad_(requested[1])
    wanted_a = a.detach().cpu().clone().requires_grad_(requested[0])
    wanted_b = b.detach().cpu().clone().requires_grad_(requested[1])
    binding.stats_all(0, True)
    output = binding.matmul_public(a, b)
    output.sum().backward()
    (wanted_a @ wanted_b).sum().backward()
    torch.cuda.synchronize()
    # one product forward and one per requested gradient (the autograd worker thread has a context
    # of its own: the total is taken over all threads)
    assert binding.stats_all(0, False)["classical"] == 1 + sum(requested)
    if requested[0]:
        close(a.grad, wanted_a.grad)
    if requested[1]:
        close(b.grad, wanted_b.grad)
    with pytest.raises(ValueError):
        binding.matmul_public(a, b, alpha=0.5)
    with torch.no_grad():
        close(binding.matmul_public(a, b, alpha=0.5), 0.5 * (wanted_a.detach() @ wanted_b.detach()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_unaligned_contiguous_views(device, dtype):
    # storage offset of one element: the data pointers are 4 or 8 bytes off every wider alignment
    a = torch.randn((128 * 256 + 1,), device=device, dtype=dtype)[1:].view(128, 256)
    b = torch.randn((256 * 64 + 1,), device=device, dtype=dtype)[1:].view(256, 64)
    bias = torch.randn((65,), device=device, dtype=dtype)[1:]
    expected = a.double().cpu() @ b.double().cpu()
    bound = 8 * torch.finfo(dtype).eps * (a.double().cpu().abs() @ b.double().cpu().abs()).clamp_min(1)
    for policy in ("auto", "lt"):
        with _native.algorithm(policy):
            assert ((_kernels.matmul(a, b).double().cpu() - expected).abs() <= bound).all()
            got = _kernels.affine(a, b, bias).double().cpu()
            assert ((got - expected - bias.double().cpu()).abs() <= bound).all()


def test_process_closes_contexts_reuses_them_and_exits_cleanly():
    code = """
import torch
from camblas_amd import _kernels as cb
from camblas_amd._native import close, stats
for repeat in range(2):
    for policy in ('classical', 'auto'):
        values = [torch.randn(s, device='cuda', requires_grad=True)
                  for s in ((11, 17), (17, 23), (23,), (23, 13), (13,))]
        with cb.algorithm(policy):
            output = cb.mlp(*values)
        output.square().mean().backward()
        assert all(torch.isfinite(x.grad).all() for x in values)
    assert stats(all_threads=True)['backward'] == 2
    close()
    assert not any(stats(all_threads=True).values())
print('ok')
"""
    result = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True,
                            timeout=120)
    assert result.returncode == 0 and "ok" in result.stdout, result.stdout + result.stderr


@pytest.mark.parametrize("kind,per_round", [(0, 16.0), (1, 64.0), (2, 48.0), (3, 2.0)])
def test_matrix_probe_counts_its_work(device, kind, per_round):
    # the bench-side calibration launch for the matrix cores (libcamblas_probes.so, not part of the
    # product library): with the value 1 in every operand lane each accumulator element grows by the
    # instruction's K per round (E2M1 reads the byte 0x38 as the nibbles -0 and 1.5: 32 * 1.5), so a
    # lane's sum over 8 accumulators x 16 elements is exact, and the reported operation count is
    # workgroups * 8 wavefronts * rounds * 8 instructions
    import ctypes as ct

    lib = ct.CDLL(str(_native.library_path().parent / "libcamblas_probes.so"))
    probe = lib.camblas_probe_matrix
    probe.argtypes = [ct.c_void_p, ct.c_int, ct.c_int, ct.c_int, ct.c_int, ct.c_void_p, ct.c_size_t,
                      ct.POINTER(ct.c_double)]
    assert not hasattr(_native.library(), "camblas_hip_matrix_probe")
    stream = ct.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    units = torch.cuda.get_device_properties(device).multi_processor_count
    sink = torch.zeros(units * 512, dtype=torch.float32, device=device)
    flops = ct.c_double(0.0)
    rounds = 25
    assert probe(stream, kind, units, rounds, 1, sink.data_ptr(), sink.numel() * 4, ct.byref(flops)) == 0
    torch.cuda.synchronize()
    assert (sink == 128 * rounds * per_round).all()
    k = {0: 16, 1: 64, 2: 64, 3: 2}[kind]
    assert flops.value == 2.0 * 32 * 32 * k * units * 8 * rounds * 8
    assert probe(stream, kind, units, rounds, 0, sink.data_ptr(), sink.numel() * 4, ct.byref(flops)) == 0
    torch.cuda.synchronize()
    assert torch.isfinite(sink).all() and (sink != 0).any()
    # refused without a launch: unknown kind, sink too small
    assert probe(stream, 9, units, rounds, 0, sink.data_ptr(), sink.numel() * 4, ct.byref(flops)) < 0
    assert probe(stream, 0, units, rounds, 0, sink.data_ptr(), 16, ct.byref(flops)) < 0
