"""The parts of bench.py that can be checked without a GPU: the refusal of more than one GPU, the
algorithmic byte count of the headline workload and the arithmetic of a roofline object."""

import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT))

import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    result = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                            timeout=120)
    assert result.returncode != 0
    assert "one GPU only" in result.stderr and result.stdout == ""


def test_algorithmic_bytes_of_the_decode_linear():
    # W read once, x read once, y written once, all BF16
    assert bench.decode_bytes(32) == 28672 * 8192 * 2 + 32 * 8192 * 2 + 32 * 28672 * 2 == 472121344
    assert bench.COPY_BYTES == 28672 * 8192 * 2


def test_roofline_object_arithmetic():
    memory = bench.roofline_of("hbm", 472121344, 73.0e-6)
    assert memory["bound"] == "hbm" and memory["unit"] == "GB/s" and memory["peak"] == 8000.0
    assert abs(memory["achieved"] - 472121344 / 73.0e-6 / 1e9) < 0.06 and abs(memory["frac"] - memory["achieved"] / 8000) < 1e-4
    matrix = bench.roofline_of("mfma fp8", 2.0 * 4096 * 18432 * 7168, 540e-6)
    assert matrix["bound"] == "mfma" and matrix["unit"] == "TFLOP/s" and matrix["peak"] == 5000.0
    assert abs(matrix["frac"] - 2.0 * 4096 * 18432 * 7168 / 540e-6 / 5e15) < 1e-4
    assert bench.roofline_of("mfma bf16", 1.0, 1.0)["peak"] == 2500.0
    assert bench.roofline_of("mfma fp32", 1.0, 1.0)["peak"] == 157.3
    assert bench.roofline_of("mfma fp64", 1.0, 1.0)["peak"] == 78.6


def test_roofline_object_carries_the_fraction_of_what_its_instruction_sustains():
    assert "frac_of_sustained" not in bench.roofline_of("mfma bf16", 2.0e12, 1e-3, "bf16_16x16x32")  # not measured yet
    bench.SUSTAINED["bf16_16x16x32"] = 2200.0
    try:
        found = bench.roofline_of("mfma bf16", 687.19e9, 450e-6, "bf16_16x16x32")
        assert found["instruction"] == "bf16_16x16x32" and found["sustained"] == 2200.0
        assert abs(found["frac_of_sustained"] - 687.19e9 / 450e-6 / 1e12 / 2200.0) < 1e-4
        assert "frac_of_sustained" not in bench.roofline_of("hbm", 1.0, 1.0, None)
    finally:
        bench.SUSTAINED.clear()
    assert bench.bf16_instruction("bf16 wave4-320x256x64s2") == "bf16_16x16x32_one_wavefront_per_simd"
    assert bench.bf16_instruction("bf16 dma16-128x256x64s3w8 split_k=4") == "bf16_16x16x32"
    assert bench.bf16_instruction("bf16 dma320x256x64s2w8") == "bf16_32x32x16"
