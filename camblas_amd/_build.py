"""Build recipe for libcamblas_hip.so (hipcc, gfx950 only) and the optional ATen tensor binding.

The counterpart of the reference's scripts/build_cuda.py:68-155: the core library and the tensor
binding land side by side in one directory (`camblas_amd/lib/`), which is where the loader looks
when CAMBLAS_CUDA_LIBRARY is not set.
"""

import hashlib
import json
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PACKAGE = Path(__file__).resolve().parent
ROOT = PACKAGE.parent
CSRC = PACKAGE / "csrc"
LIB_DIR = PACKAGE / "lib"
CORE = LIB_DIR / "libcamblas_hip.so"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

CORE_SOURCES = (
    "abi_context.hip",
    "abi_dense.hip",
    "abi_fusion.hip",
    "abi_quantized.hip",
    "planner.cpp",
    "bgemm_any.hip",
    "gemm_generic.hip",
    "gemv_f32.hip",
    "bgemm_tn.hip",
    "bgemv_stream.hip",
    "bgemv_stream_deep.hip",
    "bgemv_stream_norm.hip",
    "bgemv_stream_residual.hip",
    "bgemv_stream_gated.hip",
    "bgemv_stream_many.hip",
    "bgemm_dma.hip",
    "bgemm_wave4.hip",
    "bgemm_nn.hip",
    "fp8_block.hip",
    "fp8_dma.hip",
    "fp8_wave4.hip",
    "fp8_stream.hip",
    "fp8_block32.hip",
    "fp8_moe.hip",
    "mx_matmul.hip",
    "mx_dma.hip",
    "mx_wave4.hip",
    "routing.hip", "dense_ops.hip", "sgemm_mfma.hip", "dgemm_mfma.hip", "strassen.hip",
    "fusion.hip",
    "attention_decode.hip",
)

HIP_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wextra",
    "-Wno-unused-parameter",
    # packed FP32 instructions stay disabled for all device code
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]


def _run(command):
    result = subprocess.run([str(c) for c in command], capture_output=True, text=True)
    if result.returncode != 0:
        sys.stderr.write(result.stdout + result.stderr)
        raise RuntimeError("command failed: " + " ".join(str(c) for c in command))
    return result


def build_core(jobs=8, verbose=False):
    """Compile every HIP translation unit for gfx950 and link libcamblas_hip.so."""
    objects = LIB_DIR / "obj"
    objects.mkdir(parents=True, exist_ok=True)
    # the K loops of fp8_wave4.hip and mx_wave4.hip are generated text of a megabyte and more: written here, not kept in
    # the repository (the smaller loops of bgemm_wave4.hip are kept, and checked against their generator)
    _run([sys.executable, CSRC / "gen_fp8_wave4_loop.py", "--out", CSRC])
    _run([sys.executable, CSRC / "gen_mx_wave4_loop.py", "--out", CSRC])

    def compile_unit(name):
        source = CSRC / name
        target = objects / (source.stem + ".o")
        language = ["-x", "hip"] if source.suffix == ".cpp" else []
        _run([HIPCC, *HIP_FLAGS, *language, "-c", source, "-o", target])
        if verbose:
            print("compiled", name, flush=True)
        return target

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        built = list(pool.map(compile_unit, CORE_SOURCES))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *built, "-o", CORE,
          "-Wl,-soname,libcamblas_hip.so"])
    record = {
        "library": CORE.name,
        "sources": {
            name: hashlib.sha256((CSRC / name).read_bytes()).hexdigest() for name in CORE_SOURCES
        },
        "flags": HIP_FLAGS[:-2],
    }
    (LIB_DIR / "build.json").write_text(json.dumps(record, indent=1))
    return CORE


def build_probes():
    """Compile csrc/bench_probes.hip into lib/libcamblas_probes.so: calibration launches (a copy of
    known traffic, a stream of matrix instructions) that bench.py loads; not part of the product
    library."""
    target = LIB_DIR / "libcamblas_probes.so"
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    _run([HIPCC, *HIP_FLAGS, "-shared", CSRC / "bench_probes.hip", "-o", target])
    return target


BINDING_SOURCES = ("tensor_binding.cpp", "binding_dense.cpp", "binding_fusion.cpp", "binding_quantized.cpp")


def build_tensor_binding(jobs=4):
    """Compile the binding units (host code only: ATen + pybind11 + the C ABI) into
    lib/_camblas_cuda_torch<ext>.so, linked against libcamblas_hip.so beside it."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    torch_lib = Path(torch.__file__).resolve().parent / "lib"
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    target = LIB_DIR / ("_camblas_cuda_torch" + suffix)
    includes = [f"-I{path}" for path in cpp_extension.include_paths()]
    includes += [f"-I{sysconfig.get_paths()['include']}", "-I/opt/rocm/include",
                 f"-I{ROOT / 'include'}"]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    compiler = os.environ.get("CXX", "g++")
    flags = [
        "-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-Wno-deprecated-declarations",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
        "-DTORCH_API_INCLUDE_EXTENSION_H", "-DTORCH_EXTENSION_NAME=_camblas_cuda_torch", *includes,
        f"-I{CSRC}",
    ]
    objects = LIB_DIR / "obj"
    objects.mkdir(parents=True, exist_ok=True)
    # the K loops of fp8_wave4.hip and mx_wave4.hip are generated text of a megabyte and more: written here, not kept in
    # the repository (the smaller loops of bgemm_wave4.hip are kept, and checked against their generator)
    _run([sys.executable, CSRC / "gen_fp8_wave4_loop.py", "--out", CSRC])
    _run([sys.executable, CSRC / "gen_mx_wave4_loop.py", "--out", CSRC])

    def compile_unit(name):
        unit = objects / (Path(name).stem + ".binding.o")
        _run([compiler, *flags, "-c", CSRC / name, "-o", unit])
        return unit

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        units = list(pool.map(compile_unit, BINDING_SOURCES))
    command = [
        compiler, "-shared", *units, "-o", target, f"-L{LIB_DIR}", "-lcamblas_hip", f"-L{torch_lib}",
        "-ltorch_python", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip", "-L/opt/rocm/lib",
        "-lamdhip64", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}",
    ]
    _run(command)
    return target


if __name__ == "__main__":
    print(build_core(verbose=True))
    print(build_probes())
    if "--no-binding" not in sys.argv:
        print(build_tensor_binding())
