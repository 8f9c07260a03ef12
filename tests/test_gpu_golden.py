"""The HIP path against the committed golden vectors (tests/golden/linear_path.npz), through the
same entry points a caller uses. Bars: BF16/FP8 outputs within relative Frobenius 1e-2 of the stored
FP64-accumulated results (and within one BF16 unit element-wise where the arithmetic is a fixed
chain), integer/byte results (quantised bytes, scales, residual sums) bit-exact."""

from pathlib import Path

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _kernels
from helpers import (bf16_ulp_distance, bf16_values, from_device_bf16, from_device_fp8, rel_frobenius,
                     to_device_bf16, to_device_fp8)

pytestmark = pytest.mark.gpu
G = np.load(Path(__file__).parent / "golden" / "linear_path.npz")


def test_bf16_linear_alpha_beta(device):
    out = to_device_bf16(G["bf16_c"], device)
    _kernels.matmul(to_device_bf16(G["bf16_x"], device), to_device_bf16(G["bf16_w"], device).t(),
                    out=out, alpha=0.75, beta=-0.5)
    want = oracle.bf16_to_f32(G["bf16_y_alpha075_beta_m05"])
    assert rel_frobenius(bf16_values(out), want) <= 1e-2
    assert bf16_ulp_distance(from_device_bf16(out), G["bf16_y_alpha075_beta_m05"]).max() <= 1


def test_fp32_gemm(device):
    out = _kernels.matmul(torch.from_numpy(G["f32_a"]).to(device), torch.from_numpy(G["f32_b"]).to(device))
    assert rel_frobenius(out.cpu().numpy(), G["f32_c"]) <= 1e-5


def test_fp8_block_linear_and_quantiser(device):
    out = _kernels.fp8_block_matmul(to_device_fp8(G["fp8_a"], device),
                                    torch.from_numpy(G["fp8_a_scale"]).to(device),
                                    to_device_fp8(G["fp8_w"], device),
                                    torch.from_numpy(G["fp8_w_scale"]).to(device))
    assert rel_frobenius(bf16_values(out), oracle.bf16_to_f32(G["fp8_out"])) <= 1e-2
    q, scale = _kernels.fp8_quantise_1x128(to_device_bf16(G["quant_x"], device))
    assert np.array_equal(from_device_fp8(q), G["quant_q"])
    assert np.array_equal(scale.cpu().numpy(), G["quant_scale"])


def test_decode_epilogues(device):
    added, out = _kernels.add_rms_norm(to_device_bf16(G["rms_x"], device),
                                       to_device_bf16(G["rms_residual"], device),
                                       to_device_bf16(G["rms_weight"], device), 1e-5)
    assert np.array_equal(from_device_bf16(added), G["rms_added"])
    assert bf16_ulp_distance(from_device_bf16(out), G["rms_out"]).max() <= 1
    gate, up = to_device_bf16(G["act_gate"], device), to_device_bf16(G["act_up"], device)
    assert bf16_ulp_distance(from_device_bf16(_kernels.silu_multiply(gate, up)), G["silu_out"]).max() <= 1
    assert bf16_ulp_distance(from_device_bf16(_kernels.swiglu(gate, up)), G["swiglu_out"]).max() <= 1


def test_rope_and_decode_attention(device):
    out = _kernels.rope(to_device_bf16(G["rope_x"], device),
                        torch.from_numpy(G["rope_positions"]).to(device), 5e5)
    assert rel_frobenius(bf16_values(out), oracle.bf16_to_f32(G["rope_out"])) <= 1e-2
    assert np.array_equal(from_device_bf16(out)[0], G["rope_out"][0])
    attended = _kernels.gqa_decode_attention(to_device_bf16(G["attn_q"], device),
                                             to_device_bf16(G["attn_k"], device),
                                             to_device_bf16(G["attn_v"], device),
                                             torch.from_numpy(G["attn_lengths"]).to(device), 128**-0.5)
    assert rel_frobenius(bf16_values(attended), oracle.bf16_to_f32(G["attn_out"])) <= 1e-2
