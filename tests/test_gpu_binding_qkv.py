"""The binding's grouped query/key/value projection after the reference's tests/test_qkv.py:19-101:
three bias-free projections of one input into three separately allocated outputs, every element
against an FP64 product before and after the input and the weights change in place; rejected
shapes, precisions and gradient-tracking inputs; and the call captured in a graph on a side
stream, replayed after its operands change."""

import pytest
import torch

from camblas_amd import _native

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def module():
    binding = _native.tensor_module()
    assert binding is not None and hasattr(binding, "qkv_linear")
    return binding


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_three_independent_outputs_follow_their_operands(module, device, dtype):
    generator = torch.Generator().manual_seed(20261004)
    x = (torch.randn((2, 7, 128), generator=generator) / 8).to(dtype).to(device)
    weights = [(torch.randn((width, 128), generator=generator) / 8).to(dtype).to(device) for width in (256, 32, 32)]
    relative, absolute = (2.0 ** -6, 2e-3) if dtype == torch.bfloat16 else (2e-5, 2e-6)
    with torch.inference_mode():
        for changed in (False, True):
            if changed:
                x.add_(0.125)
                for weight in weights:
                    weight.mul_(-0.5)
            outputs = module.qkv_linear(x, *weights)
            assert len({output.data_ptr() for output in outputs}) == 3
            for output, weight in zip(outputs, weights):
                assert output.shape == (2, 7, weight.shape[0]) and output.dtype == dtype
                want = (x.double().cpu() @ weight.double().cpu().T).to(dtype)
                torch.testing.assert_close(output.cpu(), want, rtol=relative, atol=absolute)
        # one weight of another inner size; a precision the path does not serve
        with pytest.raises(ValueError):
            module.qkv_linear(x, weights[0][:, :64], weights[1], weights[2])
        with pytest.raises(ValueError):
            module.qkv_linear(x.double(), *(weight.double() for weight in weights))
    # gradients wanted: this is an inference entry point
    tracked = torch.randn((1, 128), device=device, requires_grad=True)
    plain = [torch.randn((32, 128), device=device) for _ in range(3)]
    with pytest.raises(ValueError):
        module.qkv_linear(tracked, *plain)


def test_captured_call_follows_changed_operands(module, device):
    with torch.inference_mode():
        x = torch.randn((1, 1, 128), device=device)
        weights = [torch.randn((32, 128), device=device) / 8 for _ in range(3)]
        stream = torch.cuda.Stream(device=device)
        stream.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(stream):
            for _ in range(3):
                module.qkv_linear(x, *weights)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                outputs = module.qkv_linear(x, *weights)
            for round_ in range(3):  # replays with eager work and synchronisation between them
                x.add_(0.125)
                for weight in weights:
                    weight.mul_(-0.5)
                graph.replay()
                stream.synchronize()
                for output, weight in zip(outputs, weights):
                    want = (x.double().cpu() @ weight.double().cpu().T).float()
                    torch.testing.assert_close(output.cpu(), want, rtol=2e-5, atol=2e-6)
                module.qkv_linear(x, *weights)
        stream.synchronize()
        torch.cuda.current_stream(device).wait_stream(stream)
        graph.reset()
