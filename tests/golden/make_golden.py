"""Writes tests/golden/linear_path.npz: small seeded inputs of every operation on the linear path
with the outputs the CPU oracle computes for them.

The reference ships no fixture files for this path (its tests regenerate seeded torch inputs and
compute an FP64 product on the fly), so these vectors are produced by this repo's oracle after it
has been pinned by tests/test_cpu_oracle.py (reference CPU library, third-party codecs, closed
forms, brute force). They freeze the oracle's answers so that a later change to it, or to a
kernel, shows up as a diff against committed data. Run from the repository root:
    python tests/golden/make_golden.py
"""

import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

import oracle  # noqa: E402


def main():
    data = {}
    # BF16 linear, decode-shaped and with alpha/beta
    tokens, outputs, inner = 8, 64, 256
    x = oracle.fill_normal_bf16(9001, (tokens, inner))
    w = oracle.fill_normal_bf16(9002, (outputs, inner), std=0.05)
    c = oracle.fill_normal_bf16(9003, (tokens, outputs))
    y = c.copy()
    oracle.bgemm_f64("T", "N", outputs, tokens, inner, 0.75, w, inner, x, inner, -0.5, y.ravel(),
                     outputs)
    data.update(bf16_x=x, bf16_w=w, bf16_c=c, bf16_y_alpha075_beta_m05=y)
    # FP32 GEMM, row-major 48 x 40 x 56 through the swapped column-major call
    a = oracle.fill_uniform(9004, (48, 56))
    b = oracle.fill_uniform(9005, (56, 40))
    out = np.zeros((48, 40), np.float32)
    oracle.sgemm_f64("N", "N", 40, 48, 56, 1.0, b.ravel(), 40, a.ravel(), 56, 0.0, out.ravel(), 40)
    data.update(f32_a=a, f32_b=b, f32_c=out)
    # FP8 block-scaled linear, two K groups, two weight blocks (second one partial)
    rows, outs, k = 4, 192, 256
    qa, sa = oracle.fill_fp8_blocks(9006, rows, k, 1)
    qw, sw = oracle.fill_fp8_blocks(9007, outs, k, 128)
    data.update(fp8_a=qa, fp8_a_scale=sa, fp8_w=qw, fp8_w_scale=sw,
                fp8_out=oracle.fp8_block_matmul(qa, sa, qw, sw))
    xq = oracle.fill_normal_bf16(9008, (3, 256))
    q, s = oracle.quantise_1x128(xq)
    data.update(quant_x=xq, quant_q=q, quant_scale=s)
    # residual add + RMS norm, SiLU*up, SwiGLU
    h = oracle.fill_normal_bf16(9009, (4, 512))
    r = oracle.fill_normal_bf16(9010, (4, 512))
    g = oracle.fill_normal_bf16(9011, (512,), mean=1.0, std=0.05)
    added, normed = oracle.rms_norm(2, 2, 1e-5, h, g, residual=r)
    data.update(rms_x=h, rms_residual=r, rms_weight=g, rms_added=added, rms_out=normed)
    gate = oracle.fill_normal_bf16(9012, (4, 256), std=2.0)
    up = oracle.fill_normal_bf16(9013, (4, 256))
    data.update(act_gate=gate, act_up=up, silu_out=oracle.silu_multiply(2, gate, up),
                swiglu_out=oracle.swiglu(2, 256, 0.0, gate, up))
    # rotary embedding and GQA decode attention
    heads = oracle.fill_normal_bf16(9014, (3, 4, 128))
    positions = np.array([0, 5, 2047], np.int32)
    data.update(rope_x=heads, rope_positions=positions, rope_out=oracle.rope(heads, positions, 5e5))
    qh = oracle.fill_normal_bf16(9015, (2, 4, 128))
    kc = oracle.fill_normal_bf16(9016, (2, 300, 1, 128))
    vc = oracle.fill_normal_bf16(9017, (2, 300, 1, 128))
    lengths = np.array([300, 77], np.int32)
    data.update(attn_q=qh, attn_k=kc, attn_v=vc, attn_lengths=lengths,
                attn_out=oracle.gqa_decode(qh, kc, vc, lengths, 128**-0.5))
    np.savez_compressed(Path(__file__).with_name("linear_path.npz"), **data)
    print("wrote", Path(__file__).with_name("linear_path.npz"))


if __name__ == "__main__":
    main()
