"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol the header
declares and every symbol the reference's loader resolves, the planner (a pure host function)
makes the documented choices, the Python surface mirrors the reference's contract, and bench.py
refuses more than one GPU."""

import ctypes as ct
import os
import re
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from camblas_amd import _kernels, _native

ROOT = Path(__file__).resolve().parents[1]
HEADER = (ROOT / "include" / "camblas_hip.h").read_text()


def declared_symbols():
    names = re.findall(r"\b(camblas_(?:cuda|hip)_[a-z0-9_]+)\s*\(", HEADER)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    lib = ct.CDLL(str(_native.library_path()))
    names = declared_symbols()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), name


def test_reference_loader_contract_symbols_present():
    # the names the reference's ctypes loader resolves at load time (camblas/_native.py:97-173);
    # only bgemm is optional there
    lib = _native.library()
    for name in ("create", "destroy", "error", "set_algorithm", "stats", "reset_stats", "affine",
                 "mlp", "sgemm", "dgemm", "bgemm", "attention"):
        assert hasattr(lib, "camblas_cuda_" + name)
    # every Python-side signature names an exported symbol
    for name in _native.SIGNATURES:
        assert hasattr(lib, _native.symbol_name(name)), name


def test_null_context_and_stats_errors_without_a_device():
    lib = _native.library()
    assert lib.camblas_cuda_destroy(None) == 0
    assert lib.camblas_cuda_set_algorithm(None, 0) == -1
    assert b"invalid algorithm failed (status 1)" in lib.camblas_cuda_error(None)
    assert lib.camblas_cuda_sgemm(None, b"N", b"N", 1, 1, 1, 1.0, None, 1, None, 1, 0.0, None, 1) == -1
    assert b"missing context" in lib.camblas_cuda_error(None)
    counts = (ct.c_uint64 * 8)()
    assert lib.camblas_cuda_stats(None, counts, 8) == -1
    assert lib.camblas_cuda_fp8_block_workspace_size(4, 256) == 4 * 256 + 4 * 2 * 4
    assert lib.camblas_cuda_fp8_block_workspace_size(4, 100) == 0


def test_planner_choices_for_the_baseline_shapes():
    describe = _native.plan_describe
    # decode linears: weight-streaming kernel, one workgroup per compute unit for the up-projection
    code, text = describe(2, "T", "N", 28672, 32, 8192, 8192, 8192, 28672)
    assert code // 1000 == 4 and "stream rows=112 tokens=32" in text
    assert "tokens=16" in describe(2, "T", "N", 28672, 1, 8192, 8192, 8192, 28672)[1]
    # the down projection (few rows, long K): 64-row tiles, K divided over two workgroups per tile;
    # a single token on a short K keeps the undivided 32-row tiles
    assert "rows=64 tokens=32 k_step=128 k_shares=2" in describe(2, "T", "N", 8192, 32, 28672, 28672, 28672, 8192)[1]
    assert "rows=32 tokens=16 k_step=256 k_shares=1" in describe(2, "T", "N", 8192, 1, 8192, 8192, 8192, 8192)[1]
    # prefill: the 320 x 256 tile divides 10240 x 4096 into exactly two rounds of workgroups; with K a
    # multiple of 128 it runs on four wavefronts with the K loop in assembly, else on eight
    assert describe(2, "T", "N", 10240, 4096, 8192, 8192, 8192, 10240) == (5019, "bf16 wave4-320x256x64s2")
    assert describe(2, "T", "N", 10240, 4096, 8256, 8256, 8256, 10240) == (5012, "bf16 dma16-320x256x64s2w8")
    # 2.8 rounds of 320 x 256 tiles: two whole rounds, and the last 4096 outputs as one round of 256 x 256
    assert describe(2, "T", "N", 14336, 4096, 4096, 4096, 4096, 14336) == (
        5019, "bf16 wave4-320x256x64s2, last 4096 outputs wave4-256x256x64s2")
    # 28672 x 4096 outputs are exactly seven rounds of 256 x 256 tiles
    assert describe(2, "T", "N", 28672, 4096, 8192, 8192, 8192, 28672) == (5018, "bf16 wave4-256x256x64s2")
    # a K beyond 16384 keeps the eight-wavefront tiles
    assert describe(2, "T", "N", 8192, 4096, 28672, 28672, 28672, 8192) == (5013, "bf16 dma16-256x256x64s2w8")
    # 65..1536 tokens: tile, shares of K and a second launch by estimated time (one round of
    # workgroups where the tiles alone would leave compute units idle)
    assert describe(2, "T", "N", 8192, 256, 8192, 8192, 8192, 8192) == (5015, "bf16 dma16-128x256x64s3w8 split_k=4")
    assert describe(2, "T", "N", 10240, 128, 8192, 8192, 8192, 10240) == (5017, "bf16 dma16-128x128x64s3w4 split_k=3")
    assert describe(2, "T", "N", 28672, 1024, 8192, 8192, 8192, 28672) == (
        5019, "bf16 wave4-320x256x64s2, last 8192 outputs dma16-128x256x64s3w8")
    assert describe(2, "T", "N", 8192, 256, 8200, 8200, 8200, 8192) == (2002, "bf16 mfma128x128x64 split_k=4")
    # K not a multiple of 64: register-staged MFMA tiles; unaligned operands and the other transpose
    # pairs: the layout-agnostic matrix-core kernel; slivers and the classical policy: vector-ALU tiles
    assert describe(2, "T", "N", 10240, 4096, 8200, 8200, 8200, 10240)[0] // 1000 == 2
    assert describe(2, "T", "N", 1024, 64, 1001, 1001, 1001, 1024)[0] // 1000 == 9
    assert describe(2, "N", "N", 1024, 64, 1024, 1024, 1024, 1024) == (
        10000, "bf16 outputs-contiguous stream 128x64 split_k=2")
    assert describe(2, "N", "N", 1024, 600, 1024, 1024, 1024, 1024) == (9001, "bf16 mfma any-layout 128x64x32")
    assert describe(2, "N", "T", 8192, 8192, 4096, 8192, 8192, 8192) == (9000, "bf16 mfma any-layout 128x128x32")
    assert describe(2, "T", "N", 1024, 64, 1024, 1024, 1024, 1024, aligned16=False)[0] // 1000 == 9
    assert describe(2, "N", "N", 1024, 16, 1024, 1024, 1024, 1024)[0] // 1000 == 10
    assert describe(2, "N", "N", 1024, 16, 1000, 1024, 1000, 1024)[0] // 1000 == 0  # K not a multiple of 64
    assert describe(2, "T", "N", 1024, 64, 1024, 1024, 1024, 1024, algorithm="classical")[0] // 1000 == 0
    # FP32: single-vector shortcut only under auto (ref: src/cuda/backend.cu:810-815)
    assert describe(0, "T", "N", 4096, 1, 4096, 4096, 4096, 4096)[0] // 1000 == 1
    # (otherwise a handful of columns against a large A: matrix-core tiles with K divided over workgroups;
    # a small A stays on the vector-ALU tiles)
    assert describe(0, "T", "N", 4096, 1, 4096, 4096, 4096, 4096, algorithm="lt") == (8002, "f32 mfma 128x32x32 split_k=16")
    assert describe(0, "T", "N", 1000, 1, 4096, 4096, 4096, 1000) == (8002, "f32 mfma 128x32x32 split_k=16")
    assert describe(0, "T", "N", 8192, 16, 8192, 8192, 8192, 8192) == (8002, "f32 mfma 128x32x32 split_k=16")
    assert describe(0, "T", "N", 200, 1, 4096, 4096, 4096, 200)[0] // 1000 == 0
    assert describe(0, "T", "N", 4096, 4, 4096, 4096, 4096, 4096, algorithm="classical")[0] // 1000 == 0
    # FP32 products: matrix-core tiles, 128 x 64 until every compute unit gets two 128 x 128 tiles
    assert describe(0, "N", "N", 2048, 2048, 2048, 2048, 2048, 2048) == (8001, "f32 mfma 128x64x32")
    assert describe(0, "T", "N", 4096, 4096, 4096, 4096, 4096, 4096) == (8000, "f32 mfma 128x128x32")
    assert describe(0, "N", "N", 2048, 16, 2048, 2048, 2048, 2048) == (8002, "f32 mfma 128x32x32 split_k=8")
    assert describe(0, "N", "N", 2048, 48, 2048, 2048, 2048, 2048) == (8001, "f32 mfma 128x64x32 split_k=8")
    assert describe(0, "N", "N", 128, 16, 2048, 128, 2048, 128)[0] // 1000 == 0
    # FP8: the streaming kernel for decode batches (one launch; up to 8 tokens only where the 16-row
    # tiles fill the compute units, else small tiles with divided K), direct-to-LDS tiles for prefill
    code, text = describe(3, "T", "N", 18432, 1, 7168, 7168, 7168, 18432)
    assert code // 1000 == 7 and "stream rows=80 tokens=16" in text
    assert describe(3, "T", "N", 2048, 1, 7168, 7168, 7168, 2048)[0] // 1000 == 3
    code, text = describe(3, "T", "N", 18432, 16, 7168, 7168, 7168, 18432)
    assert code // 1000 == 7 and "stream rows=80 tokens=16" in text
    # 33 to 64 tokens: the streaming kernel where its workgroups of five or six row tiles come to about one per
    # compute unit; otherwise tiles with divided K when K is long enough to divide, else the streaming kernel
    assert "stream rows=80 tokens=48" in describe(3, "T", "N", 18432, 33, 7168, 7168, 7168, 18432)[1]
    assert "stream rows=80 tokens=64" in describe(3, "T", "N", 18432, 64, 7168, 7168, 7168, 18432)[1]
    assert "split_k=6" in describe(3, "T", "N", 7168, 64, 18432, 18432, 18432, 7168)[1]
    assert "tokens=64" in describe(3, "T", "N", 7168, 64, 2048, 2048, 2048, 7168)[1]
    # the streaming kernel holds K / 128 scales per token in LDS: K beyond 24576 goes to the tiles
    assert "stream" not in describe(3, "T", "N", 7168, 16, 32768, 32768, 32768, 7168)[1]
    # 4.5 rounds of 256 x 256 tiles: four whole rounds, and the last 2048 outputs as one round of 256 x 128
    assert describe(3, "T", "N", 18432, 4096, 7168, 7168, 7168, 18432) == (
        6010, "fp8-block128 fp8dma16-256x256x128w8 split_k=1, last 2048 outputs fp8dma256x128x128s3w8")
    assert describe(3, "T", "N", 18432, 2048, 7168, 7168, 7168, 18432) == (6014, "fp8-block128 fp8dma16-192x256x128w8 split_k=1")
    # tiles and K shares are priced: 96 tiles of 192 rows fill the compute units at 256 tokens, a
    # narrow projection with a long K divides its groups, 256 x 256 tiles where 256 divides the outputs well
    assert describe(3, "T", "N", 18432, 256, 7168, 7168, 7168, 18432)[1].endswith("fp8dma16-192x128x128s3w8 split_k=1")
    assert describe(3, "T", "N", 7168, 256, 18432, 18432, 18432, 7168)[1].endswith("fp8dma16-192x128x128s3w8 split_k=3")
    assert "fp8dma16-256x256x128w8 split_k=1" in describe(3, "T", "N", 7168, 4096, 18432, 18432, 18432, 7168)[1]
    assert describe(3, "T", "N", 24576, 512, 1536, 1536, 1536, 24576)[1].endswith("split_k=1")  # 12 groups: too few to divide
    # the plan is a pure function of its arguments
    assert describe(3, "T", "N", 18432, 16, 7168, 7168, 7168, 18432) == describe(
        3, "T", "N", 18432, 16, 7168, 7168, 7168, 18432)


def test_operand_layout_mapping():
    # ref: src/cuda/torch_bindings.cpp:146-153
    base = torch.zeros(6, 8)
    assert _kernels._operand(base)[1:] == (b"N", 8)
    assert _kernels._operand(base.t())[1:] == (b"T", 8)
    assert _kernels._operand(base[:, :5])[1:] == (b"N", 8)          # padded rows keep their stride
    assert _kernels._operand(base[:, ::2])[1:] == (b"N", 4)         # neither: made contiguous
    assert _kernels._operand(torch.zeros(1, 8))[1:] == (b"N", 8)
    assert _kernels._operand(torch.zeros(8, 1).t())[1:] == (b"T", 1)        # [1, 8] view of a column


def test_python_surface_contract(monkeypatch):
    assert _native.ALGORITHMS["lt"] == 3 and _native.COUNTERS[4] == "lt"
    with pytest.raises(ValueError):
        _native.set_algorithm("fastest")
    import camblas_amd

    monkeypatch.delenv("CAMBLAS_ENABLE", raising=False)
    assert camblas_amd._autoload() is None  # disabled processes touch nothing
    with pytest.raises(RuntimeError):
        _kernels.matmul(torch.zeros(2, 2), torch.zeros(2, 2))  # CPU tensors are rejected, no fallback


def test_autoload_environment_contract(monkeypatch):
    # ref: camblas/__init__.py:6-29 — CAMBLAS_ENABLE=1 installs the backend with the policy named by
    # CAMBLAS_CUDA_ALGORITHM, else CAMBLAS_SGLANG_ALGORITHM, else "lt"; a missing binding is a
    # RuntimeError, an unknown policy a ValueError
    import types

    import camblas_amd

    installed = []
    monkeypatch.setattr(_native, "tensor_module",
                        lambda: types.SimpleNamespace(install_torch_backend=installed.append))
    monkeypatch.setenv("CAMBLAS_ENABLE", "1")
    for variable in ("CAMBLAS_CUDA_ALGORITHM", "CAMBLAS_SGLANG_ALGORITHM"):
        monkeypatch.delenv(variable, raising=False)
    camblas_amd._autoload()
    monkeypatch.setenv("CAMBLAS_SGLANG_ALGORITHM", "classical")
    camblas_amd._autoload()
    monkeypatch.setenv("CAMBLAS_CUDA_ALGORITHM", "auto")
    camblas_amd._autoload()
    assert installed == [_native.ALGORITHMS["lt"], _native.ALGORITHMS["classical"], _native.ALGORITHMS["auto"]]
    monkeypatch.setenv("CAMBLAS_CUDA_ALGORITHM", "fastest")
    with pytest.raises(ValueError, match="Unknown CAMBLAS CUDA algorithm"):
        camblas_amd._autoload()
    monkeypatch.setattr(_native, "tensor_module", lambda: None)
    with pytest.raises(RuntimeError, match="tensor binding"):
        camblas_amd._autoload()
    assert len(installed) == 3


def test_missing_library_fails_loudly(tmp_path):
    code = "from camblas_amd import _native; _native.library()"
    env = dict(os.environ, CAMBLAS_CUDA_LIBRARY=str(tmp_path / "absent.so"), PYTHONPATH=str(ROOT))
    result = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env)
    assert result.returncode != 0 and "libcamblas_hip.so not found" in result.stderr


def test_bench_refuses_more_than_one_gpu():
    result = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"],
                            capture_output=True, text=True)
    assert result.returncode != 0 and "one GPU" in result.stderr


def test_tensor_binding_loads_and_exports_the_reference_surface():
    # names the reference's Python layer looks up on its compiled binding
    # (ref: src/cuda/torch_bindings.cpp:1194-1294, camblas/_native.py:278-283, :327-336)
    module = _native.tensor_module()
    assert module is not None, "camblas_amd/lib/_camblas_cuda_torch*.so is not built"
    for name in ("install_torch_backend", "set_default_algorithm", "stats", "stats_all", "close",
                 "matmul", "matmul_public", "linear_public", "qkv_linear", "gated_mlp",
                 "silu_multiply", "swiglu", "rms_norm", "add_rms_norm", "fp8_block_matmul",
                 "fp8_decode_supported", "fp8_decode", "fp8_linear", "quantized_matmul",
                 "QuantizedGroups", "route_groups", "reduce_groups", "affine", "affine_public", "mlp_public",
                 "mlp", "mlp_backward", "attention_public", "attention"):
        assert callable(getattr(module, name)), name
    import torch

    from camblas_amd import _kernels

    assert _kernels.QuantizedGroups is module.QuantizedGroups
    with pytest.raises(AttributeError):
        _kernels.no_such_operation
    with pytest.raises(ValueError, match="GPU"):
        module.matmul_public(torch.zeros(2, 2), torch.zeros(2, 2))


def test_contexts_inherited_through_fork_are_refused(monkeypatch):
    # ref: camblas/_native.py:266-268 — the check is on the process id, before any device call
    import os
    import types

    table = _native._LOCAL.__dict__.setdefault("contexts", {})
    inherited = types.SimpleNamespace(pid=os.getpid() + 1, handle=1, set_algorithm=lambda name: None)
    monkeypatch.setitem(table, (0, 4242), inherited)
    monkeypatch.setattr(torch.cuda, "current_stream", lambda device=None: types.SimpleNamespace(cuda_stream=4242))
    with pytest.raises(RuntimeError, match="fork"):
        _native.context(0)


def test_plugin_entry_points_are_registered():
    # pyproject.toml and the hand-written dist-info at the repository root both name the two plugin
    # groups the reference registers (ref: pyproject.toml:12-16); importlib.metadata finds the
    # dist-info for any process that has the repository root on its module search path
    from importlib.metadata import entry_points

    sys.path.insert(0, str(ROOT))
    try:
        found = {(group, entry.name, entry.value) for group in ("torch.backends", "sglang.srt.plugins")
                 for entry in entry_points(group=group)}
    finally:
        sys.path.remove(str(ROOT))
    assert ("torch.backends", "camblas", "camblas_amd:_autoload") in found
    assert ("sglang.srt.plugins", "camblas", "camblas_amd.sglang:install") in found
    text = (ROOT / "pyproject.toml").read_text()
    assert 'camblas = "camblas_amd:_autoload"' in text and 'camblas = "camblas_amd.sglang:install"' in text


def test_generated_assembly_loops_are_in_step_with_their_generator(tmp_path):
    # the K loops of the four-wavefront prefill tiles are committed as generated text: regenerate
    # them and compare, so that an edit to one side alone is caught
    import subprocess
    import sys
    from pathlib import Path

    sources = Path(__file__).resolve().parents[1] / "camblas_amd" / "csrc"
    subprocess.run([sys.executable, str(sources / "gen_wave4_loop.py"), "--out", str(tmp_path)], check=True)
    for name in ("wave4_loop_256x256.inc", "wave4_loop_320x256.inc", "wave4_loop_256x256_nn.inc"):
        assert (tmp_path / name).read_text() == (sources / name).read_text(), name


def test_fp8_four_wavefront_loop_generator_writes_whole_steps(tmp_path):
    # the FP8 loop is generated at build time; its shape is fixed by the tile: three variants (where
    # the wavefront's rows cross a scale block) x three slabs of eight K groups x 48 tiles, each tile
    # one matrix instruction and four scaled accumulates, and the same number of barriers per variant
    import subprocess
    import sys
    from pathlib import Path

    sources = Path(__file__).resolve().parents[1] / "camblas_amd" / "csrc"
    subprocess.run([sys.executable, str(sources / "gen_fp8_wave4_loop.py"), "--out", str(tmp_path)], check=True)
    text = (tmp_path / "fp8_wave4_loop_192x256.inc").read_text()
    variants = text.split("asm volatile(")[1:]
    assert len(variants) == 3
    for variant in variants:
        assert variant.count("v_mfma_scale_f32_16x16x128_f8f6f4") == 3 * 8 * 48
        assert variant.count("v_fmac_f32_e32") == 3 * 8 * 48 * 4
        assert variant.count("s_barrier") == variants[0].count("s_barrier") == 2 + 3 * 8 - 1
        assert "v_pk_" not in variant
