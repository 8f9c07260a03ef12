"""Random shapes through the planner: whatever kernel it picks for a call, sampled output columns agree with
an FP64 product of the decoded operands. The shapes are drawn around the planner's thresholds (token counts
either side of 16 / 32 / 48 / 64 / 128 / 256, outputs and inner dimensions that are and are not multiples of
the tiles), with a fixed seed; the description of the plan is part of the failure message.

Bounds: BF16 results within the BF16 rounding of the FP64 value plus 2e-4 of the largest output; the FP8 and
E8M0 products within the BF16 rounding plus 2^-12 of the sum of the products' magnitudes, which is what the
scaled matrix instruction's internal alignment loses on operands spread over the whole exponent range."""
import random

import pytest
import torch

from camblas_amd import _kernels, _native

pytestmark = pytest.mark.gpu

TOKENS = [1, 2, 7, 8, 9, 15, 16, 17, 31, 32, 33, 40, 47, 48, 49, 63, 64, 65, 100, 128, 129, 200, 256, 300, 513]


def sampled(outputs, device):
    step = max(1, outputs // 41)
    return torch.unique(torch.cat([torch.arange(0, outputs, step, device=device),
                                   torch.tensor([outputs - 1], device=device)]))


def e4m3_table(device):
    return torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).double().to(device)


def finite_bytes(shape, device, generator):
    values = torch.randint(0, 256, shape, device=device, dtype=torch.uint8, generator=generator)
    values[(values & 0x7F) == 0x7F] = 0x38
    return values


def test_bf16_products(device):
    rng = random.Random(11)
    done = 0
    while done < 60:
        tokens = rng.choice(TOKENS)
        outputs = rng.choice([16, 40, 128, 1000, 2048, 4096, 4100, 6144, 8192, 8200, 10240, 12288, 16384, 28672])
        inner = rng.choice([64, 128, 200, 256, 328, 512, 1024, 2048, 4096, 4160, 8192, 8200, 14336, 28672])
        if outputs * inner > 240e6:
            continue
        done += 1
        layout = rng.choice(["linear", "linear", "linear", "row-major", "padded"])
        generator = torch.Generator(device=device).manual_seed(done)
        x = torch.randn((tokens, inner), device=device, generator=generator).to(torch.bfloat16)
        if layout == "row-major":
            operand = (torch.randn((inner, outputs), device=device, generator=generator) * 0.05).to(torch.bfloat16)
            plan = _native.plan_describe(2, "N", "N", outputs, tokens, inner, outputs, inner, outputs)[1]
        else:
            pad = rng.choice([8, 16, 24]) if layout == "padded" else 0
            rows = (torch.randn((outputs, inner + pad), device=device, generator=generator) * 0.05).to(torch.bfloat16)
            operand = rows[:, :inner].t()
            plan = _native.plan_describe(2, "T", "N", outputs, tokens, inner, inner + pad, inner, outputs)[1]
        case = (tokens, outputs, inner, layout, plan)
        y = _kernels.matmul(x, operand)
        columns = sampled(outputs, device)
        want = x.double() @ operand.double()[:, columns]
        got = y[:, columns].double()
        assert float((got - want).norm() / want.norm().clamp_min(1e-30)) <= 1e-2, case
        assert bool(((got - want).abs() <= 2.0**-7 * want.abs() + 2e-4 * want.abs().max()).all()), case


def test_fp8_block_scaled_products(device):
    rng = random.Random(12)
    table = e4m3_table(device)
    done = 0
    while done < 60:
        tokens = rng.choice(TOKENS + [1024])
        outputs = rng.choice([128, 256, 1000, 2048, 4096, 4104, 7168, 8192, 18432])
        inner = rng.choice([128, 256, 512, 1024, 2048, 3072, 4096, 7168, 8192, 18432])
        if outputs * inner > 140e6:
            continue
        done += 1
        generator = torch.Generator(device=device).manual_seed(done)
        a = finite_bytes((tokens, inner), device, generator)
        w = finite_bytes((outputs, inner), device, generator)
        a_scale = torch.rand((tokens, inner // 128), device=device, generator=generator) * 0.1 + 1e-3
        w_scale = torch.rand(((outputs + 127) // 128, inner // 128), device=device, generator=generator) * 0.1 + 1e-3
        case = (tokens, outputs, inner, _native.plan_describe(3, "T", "N", outputs, tokens, inner, inner, inner, outputs)[1])
        y = _kernels.fp8_block_matmul(a.view(torch.float8_e4m3fn), a_scale, w.view(torch.float8_e4m3fn), w_scale)
        columns = sampled(outputs, device)
        tokens64 = table[a.long()] * a_scale.double().repeat_interleave(128, dim=1)
        weights64 = table[w[columns].long()] * w_scale.double()[columns // 128].repeat_interleave(128, dim=1)
        want, magnitudes = tokens64 @ weights64.t(), tokens64.abs() @ weights64.abs().t()
        got = y[:, columns].double()
        assert bool(((got - want).abs() <= 2.0**-7 * want.abs() + 2.0**-12 * magnitudes).all()), case


def test_e8m0_products(device):
    rng = random.Random(13)
    e4m3 = e4m3_table(device)
    e2m1 = torch.tensor([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6], dtype=torch.float64, device=device)
    done = 0
    while done < 80:
        tokens = rng.choice(TOKENS + [1024, 2048])
        outputs = rng.choice([8, 128, 256, 1000, 2048, 4096, 4104, 7168, 18432])
        inner = rng.choice([32, 128, 256, 512, 1024, 2048, 3072, 4096, 7168, 18432])
        if outputs * inner > 140e6 or tokens * inner > 40e6:
            continue
        done += 1
        packed = rng.random() < 0.5
        block = 128 if packed and inner % 128 == 0 and rng.random() < 0.3 else 32
        generator = torch.Generator(device=device).manual_seed(done)
        x = finite_bytes((tokens, inner), device, generator)
        x_scale = torch.randint(118, 132, (tokens, inner // block), device=device, dtype=torch.uint8, generator=generator)
        if packed:  # two E2M1 values to a byte, the low nibble first; a scale byte per row and 32 inputs
            w = torch.randint(0, 256, (outputs, inner // 2), device=device, dtype=torch.uint8, generator=generator)
            w_scale = torch.randint(118, 132, (outputs, inner // 32), device=device, dtype=torch.uint8, generator=generator)
        else:       # a scale byte per 32 x 32 block
            w = finite_bytes((outputs, inner), device, generator)
            w_scale = torch.randint(118, 132, ((outputs + 31) // 32, inner // 32), device=device, dtype=torch.uint8,
                                    generator=generator)
        case = (tokens, outputs, inner, "e2m1" if packed else "e4m3", block)
        y = _kernels.quantized_matmul(x.view(torch.float8_e4m3fn), x_scale, w if packed else w.view(torch.float8_e4m3fn),
                                      w_scale, activation_block=block)
        columns = sampled(outputs, device)
        tokens64 = e4m3[x.long()] * torch.exp2(x_scale.double() - 127).repeat_interleave(block, dim=1)
        if packed:
            rows = w[columns].long()
            weights64 = torch.stack([e2m1[rows & 15], e2m1[rows >> 4]], dim=-1).reshape(len(columns), inner)
            weights64 = weights64 * torch.exp2(w_scale[columns].double() - 127).repeat_interleave(32, dim=1)
        else:
            weights64 = e4m3[w[columns].long()] * torch.exp2(w_scale[columns // 32].double() - 127).repeat_interleave(32, dim=1)
        want, magnitudes = tokens64 @ weights64.t(), tokens64.abs() @ weights64.abs().t()
        got = y[:, columns].double()
        assert bool(((got - want).abs() <= 2.0**-7 * want.abs() + 2.0**-12 * magnitudes).all()), case
