"""The single-token FP8 mixture-of-experts step through the C ABI against the CPU oracle
(oracle.fp8_moe_decode_f64, pinned in tests/test_cpu_fp8_moe.py). Shapes, value ranges, the ×1.25
scale change, routing weights and the in-place call follow the reference's
tests/test_sglang.py:131-321; its bit-for-bit comparison with SGLang's Triton kernels on Hopper is
replaced by the FP8 bar of this build: relative Frobenius error <= 1e-2 against FP64 accumulation
(rounding points can flip one BF16 or E4M3 step where two evaluations of SiLU differ in the last
place), plus exact properties."""

import ctypes as ct

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _kernels, _native
from helpers import bf16_values, rel_frobenius

pytestmark = pytest.mark.gpu


def make_case(seed, experts, choices, hidden, width, outputs, magnitude, ids=None):
    rng = np.random.default_rng(seed)
    x = oracle.f32_to_bf16((rng.standard_normal(hidden) * magnitude).astype(np.float32))
    w1 = oracle.f32_to_e4m3((rng.standard_normal((experts, 2 * width, hidden)) * 0.6).astype(np.float32))
    w2 = oracle.f32_to_e4m3((rng.standard_normal((experts, outputs, width)) * 0.6).astype(np.float32))
    s1 = ((rng.random((experts, 2 * width // 128, hidden // 128)) * 0.001 + 0.001) * 1.25).astype(np.float32)
    s2 = ((rng.random((experts, (outputs + 127) // 128, width // 128)) * 0.001 + 0.001) * 1.25).astype(np.float32)
    ids = np.arange(choices, dtype=np.int32) if ids is None else np.asarray(ids, np.int32)
    routing = np.linspace(0.05, 1.0, choices).astype(np.float32)
    return x, w1, s1, w2, s2, ids, routing


def run(device, case, factor, inplace=False):
    x, w1, s1, w2, s2, ids, routing = case
    xt = torch.from_numpy(x.view(np.int16)).to(device).view(torch.bfloat16).reshape(1, -1)
    tensors = [torch.from_numpy(w1).to(device).view(torch.float8_e4m3fn),
               torch.from_numpy(w2).to(device).view(torch.float8_e4m3fn),
               torch.from_numpy(s1).to(device), torch.from_numpy(s2).to(device),
               torch.from_numpy(ids).to(device), torch.from_numpy(routing).to(device)]
    out = _kernels.fp8_moe_decode(xt, *tensors, factor=factor, out=xt if inplace else None)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("magnitude", [0.75, 80.0])
def test_reference_shapes_against_fp64(device, magnitude):
    # nine experts, all chosen in order, [9, 1024, 4096] gate/up and [9, 4096, 512] down weights
    case = make_case(842, 9, 9, 4096, 512, 4096, magnitude)
    want = oracle.fp8_moe_decode_f64(*case, 2.5)
    got = bf16_values(run(device, case, 2.5))[0]
    assert rel_frobenius(got, want) <= 1e-2
    assert (np.abs(got - want) <= 0.05 * np.abs(want) + 0.02 * np.abs(want).mean()).all()
    # output over the input (ref: tests/test_sglang.py:305-321) gives the same bits
    again = bf16_values(run(device, case, 2.5, inplace=True))[0]
    assert np.array_equal(again, got)


@pytest.mark.parametrize("experts,choices,hidden,width,outputs,ids", [
    (20, 5, 256, 128, 48, [17, 3, 3, 0, 19]),      # an expert chosen twice, outputs not a multiple of 128
    (4, 1, 128, 384, 16, [2]),                      # one choice, three down groups, the smallest output
    (33, 16, 1024, 256, 272, list(range(32, 16, -1))),  # the most choices, descending experts
])
def test_other_shapes_and_expert_choices(device, experts, choices, hidden, width, outputs, ids):
    case = make_case(7 + experts, experts, choices, hidden, width, outputs, 3.0, ids)
    want = oracle.fp8_moe_decode_f64(*case, 1.0)
    got = bf16_values(run(device, case, 1.0))[0]
    assert got.shape == (outputs,)
    assert rel_frobenius(got, want) <= 1e-2


def test_exact_properties(device):
    x, w1, s1, w2, s2, ids, routing = make_case(5, 12, 6, 512, 256, 512, 2.0, [4, 9, 0, 11, 2, 7])
    base = bf16_values(run(device, (x, w1, s1, w2, s2, ids, routing), 1.5))[0]
    # powers of two pass through every rounding: routing weights and the factor
    assert np.array_equal(bf16_values(run(device, (x, w1, s1, w2, s2, ids, routing * 2), 1.5))[0], base * 2)
    assert np.array_equal(bf16_values(run(device, (x, w1, s1, w2, s2, ids, routing), 3.0))[0], base * 2)
    # a choice with zero weight adds exactly nothing
    dropped = routing.copy()
    dropped[2] = 0.0
    keep = np.array([0, 1, 3, 4, 5])
    assert np.array_equal(bf16_values(run(device, (x, w1, s1, w2, s2, ids, dropped), 1.5))[0],
                          bf16_values(run(device, (x, w1, s1, w2, s2, ids[keep], routing[keep]), 1.5))[0])
    # doubling one expert's down scales doubles exactly that expert's contribution
    only = np.array([9], np.int32)
    one = bf16_values(run(device, (x, w1, s1, w2, s2, only, routing[:1] * 0 + 1), 1.0))[0]
    s2_changed = s2.copy()
    s2_changed[9] *= 2
    assert np.array_equal(bf16_values(run(device, (x, w1, s1, w2, s2_changed, only, routing[:1] * 0 + 1), 1.0))[0], one * 2)
    # a gate far above the limit is the gate at the limit: scale every gate row of one expert up
    # so that all its gate values exceed 10 either way
    big = s1.copy()
    big[4, : s1.shape[1] // 2] = 10.0
    bigger = big.copy()
    bigger[4, : s1.shape[1] // 2] = 40.0
    positive = np.abs(oracle.bf16_to_f32(x)) > 0
    assert positive.any()
    only4 = np.array([4], np.int32)
    w1_positive = w1.copy()
    w1_positive[4, : w1.shape[1] // 2] = 0x38                      # every gate weight 1.0
    x_positive = oracle.f32_to_bf16(np.abs(oracle.bf16_to_f32(x)) + 1.0)  # every input >= 1
    first = bf16_values(run(device, (x_positive, w1_positive, big, w2, s2, only4, routing[:1]), 1.0))[0]
    second = bf16_values(run(device, (x_positive, w1_positive, bigger, w2, s2, only4, routing[:1]), 1.0))[0]
    assert np.array_equal(first, second)


def test_invalid_arguments(device):
    native, lib = _native.context(device), _native.library()
    buffer = torch.zeros(4096, dtype=torch.uint8, device=device)
    p = ct.c_void_p(buffer.data_ptr())
    for arguments in ((0, 1, 128, 128, 16), (1, 0, 128, 128, 16), (1, 17, 128, 128, 16), (1, 1, 64, 128, 16),
                      (1, 1, 128, 192, 16), (1, 1, 128, 128, 24), (1, 16, 128, 4224, 16)):
        status = lib.camblas_cuda_fp8_moe_decode(native.handle, *arguments, p, p, p, p, p, p, p, 1.0, p)
        assert status == -1 and b"invalid FP8 expert dimensions" in lib.camblas_cuda_error(native.handle)
    status = lib.camblas_cuda_fp8_moe_decode(native.handle, 1, 1, 128, 128, 16, None, p, p, p, p, p, p, 1.0, p)
    assert status == -1 and b"invalid FP8 expert buffers" in lib.camblas_cuda_error(native.handle)
    odd = ct.c_void_p(buffer.data_ptr() + 8)
    status = lib.camblas_cuda_fp8_moe_decode(native.handle, 1, 1, 128, 128, 16, odd, p, p, p, p, p, p, 1.0, p)
    assert status == -1 and b"invalid FP8 expert buffers" in lib.camblas_cuda_error(native.handle)
    with pytest.raises(RuntimeError, match="1..16 choices"):
        case = make_case(1, 2, 1, 128, 128, 16, 1.0)
        x, w1, s1, w2, s2, ids, routing = case
        run(device, (x, w1, s1, w2, s2, np.zeros(17, np.int32), np.ones(17, np.float32)), 1.0)


def test_captured_step_replays_with_changed_token_and_choices(device):
    # the two launches captured once in a graph and replayed after the token, the chosen experts and
    # the routing weights change in place; every replay equals the eager call bit for bit (the step
    # has no reductions whose order depends on timing), with other work between the replays
    x, w1, s1, w2, s2, ids, routing = make_case(61, 24, 8, 512, 256, 512, 2.0, [5, 0, 23, 7, 11, 2, 19, 13])
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        xt = torch.from_numpy(x.view(np.int16)).to(device).view(torch.bfloat16).reshape(1, -1)
        tensors = [torch.from_numpy(w1).to(device).view(torch.float8_e4m3fn),
                   torch.from_numpy(w2).to(device).view(torch.float8_e4m3fn),
                   torch.from_numpy(s1).to(device), torch.from_numpy(s2).to(device)]
        ids_t, routing_t = torch.from_numpy(ids).to(device), torch.from_numpy(routing).to(device)
        out = torch.empty((1, 512), dtype=torch.bfloat16, device=device)
        for _ in range(2):  # creates the stream's context and its scratch outside the capture
            _kernels.fp8_moe_decode(xt, *tensors, ids_t, routing_t, factor=1.5, out=out)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        _kernels.fp8_moe_decode(xt, *tensors, ids_t, routing_t, factor=1.5, out=out)
    with torch.cuda.stream(stream):
        for round_ in range(3):
            xt.mul_(-0.75)
            ids_t.copy_((ids_t + 3 + round_) % 24)
            routing_t.mul_(1.25)
            graph.replay()
            stream.synchronize()
            eager = _kernels.fp8_moe_decode(xt, *tensors, ids_t, routing_t, factor=1.5)
            stream.synchronize()
            assert torch.equal(out, eager)
    want = oracle.fp8_moe_decode_f64(oracle.f32_to_bf16(xt.float().cpu().numpy()[0]), w1, s1, w2, s2,
                                     ids_t.cpu().numpy(), routing_t.cpu().numpy(), 1.5)
    assert rel_frobenius(bf16_values(out)[0], want) <= 1e-2
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    graph.reset()


def test_largest_intermediate_width(device):
    # 16 choices of 4096-wide experts: 512 (choice, group) pairs, the most the second launch holds
    case = make_case(91, 16, 16, 128, 4096, 32, 1.0)
    want = oracle.fp8_moe_decode_f64(*case, 1.0)
    got = bf16_values(run(device, case, 1.0))[0]
    assert rel_frobenius(got, want) <= 1e-2
