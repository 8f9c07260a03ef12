"""Benchmark of the linear hot path on one MI355X.

`python bench.py --gpus 1 --steps K --warmup W` prints ONE JSON line. The headline workload is the
BF16 decode linear y = x W^T with W [28672, 8192] (Llama-70B up-projection) and x [M, 8192] for
M in {1, 8, 32}: one "step" is one pass over the three batch sizes, each through
camblas_cuda_bgemm('T','N') on resident operands. Three weight copies (3 x 470 MB, more than the
256 MB last-level cache) are rotated so every launch streams its weights from HBM. `value` is the
algorithmic HBM traffic of the timed steps divided by wall time (host clock around K steps with a
device synchronisation on both sides).

When the K timed steps last less than 200 ms (a wall clock around a few milliseconds measures mostly
the loop's start and the final synchronisation) the same loop is timed once more over enough steps
to fill 200 ms, and `value`, `steps` and `ms_per_step` are those of the longer region; the K-step
region is kept as `config.short_run`, K as `config.requested_steps`.

The line also carries
  roofline      the dominant kernel (M=32 launch) timed with HIP events on the launch stream; its
                `traffic` is measured live: two child runs of this file under `rocprofv3 --pmc`
                (FETCH_SIZE, then WRITE_SIZE), each holding a plain copy of known size to scale by,
  cpu_baseline  PyTorch's own CPU BF16 F.linear on the same shape, all host threads of this process,
  also          the other configurations (BF16 prefill linear and addmm, FP8 block-scaled linear,
                E8M0 products, FP32 SGEMM, decode attention, decoder-layer decode step), each with
                a `roofline` object of its own (the matrix-bound ones also with the rate the
                matrix instruction they run on sustains on varied operand bits, measured in the same
                run, and the fraction of it they reach); PyTorch's CPU FP8 dequantise-then-mm; the CPU
                oracle port; the reference's own CPU SGEMM when oracle/_ref is present.
"""

import argparse
import csv
import json
import os
import shutil
import subprocess
import sys
import tempfile
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK = 8.0e12
BF16_PEAK = 2.5e15
FP8_PEAK = 5.0e15
FP32_PEAK = 157.3e12
FP64_PEAK = 78.6e12
PEAKS = {"hbm": (HBM_PEAK, 1e9, "GB/s"), "mfma bf16": (BF16_PEAK, 1e12, "TFLOP/s"),
         "mfma fp8": (FP8_PEAK, 1e12, "TFLOP/s"), "mfma fp32": (FP32_PEAK, 1e12, "TFLOP/s"),
         "mfma fp64": (FP64_PEAK, 1e12, "TFLOP/s")}
LONG_REGION = 0.2  # seconds of wall clock the headline loop should fill


SUSTAINED = {}  # matrix instruction -> TFLOP/s it sustains on varied operands (filled by measure_sustained)


def roofline_of(bound, amount, seconds, instruction=None):
    """The roofline object of one configuration: `amount` algorithmic bytes (bound "hbm") or flops
    (bound "mfma <type>") per launch over the launch time measured with events. instruction: the
    matrix instruction the kernel runs on; the object then also carries what that instruction
    sustains on operands of varied bits with nothing else going on (measured in this run) and the
    fraction of it that the kernel reaches."""
    peak, unit_scale, unit = PEAKS[bound]
    found = {"bound": bound.split()[0], "algorithmic": int(amount), "achieved": round(amount / seconds / unit_scale, 1),
             "peak": peak / unit_scale, "unit": unit, "frac": round(amount / seconds / peak, 4),
             "launch_us": round(seconds * 1e6, 2)}
    if instruction in SUSTAINED:
        found["instruction"] = instruction
        found["sustained"] = SUSTAINED[instruction]
        found["frac_of_sustained"] = round(amount / seconds / 1e12 / SUSTAINED[instruction], 4)
    return found


def bf16_instruction(plan_text):
    """The matrix instruction of a planned BF16 product, from the planner's description of it."""
    if "wave4" in plan_text:
        return "bf16_16x16x32_one_wavefront_per_simd"
    return "bf16_16x16x32" if "dma16" in plan_text else "bf16_32x32x16"


def measure_sustained(torch, device):
    """What the matrix cores sustain: independent matrix instructions with no memory traffic (the
    part's clock under matrix load included), per instruction the prefill kernels use, on constant
    and on varied operand bits. Fills SUSTAINED and returns the table for the report."""
    import ctypes as ct

    units = torch.cuda.get_device_properties(device).multi_processor_count
    sink = torch.empty(units * 512, dtype=torch.float32, device=device)
    flops = ct.c_double(0.0)
    table = {}
    # (rounds sized for launches of 2-3 ms, long enough for the clock to settle)
    for name, kind, rounds, single in (
            ("bf16_32x32x16", 0, 16000, False), ("bf16_16x16x32", 4, 16000, False),
            ("bf16_16x16x32_one_wavefront_per_simd", 4, 32000, True),
            ("e4m3_scaled_32x32x64", 1, 8000, False), ("e4m3_scaled_16x16x128", 5, 8000, False),
            ("e2m1_x_e4m3_scaled_32x32x64", 2, 8000, False), ("e2m1_x_e4m3_scaled_16x16x128", 6, 8000, False),
            ("fp32_32x32x2", 3, 8000, False)):
        launch = probes().camblas_probe_matrix_single if single else probes().camblas_probe_matrix
        entry = {}
        for operands, constant in (("varied", 0), ("constant", 1)):
            seconds = event_time(
                torch, lambda i: launch(ct.c_void_p(torch.cuda.current_stream(device).cuda_stream), kind, units,
                                        rounds, constant, ct.c_void_p(sink.data_ptr()), sink.numel() * 4,
                                        ct.byref(flops)), 2, 5)
            entry[operands + "_operands_tflops"] = round(flops.value / seconds / 1e12, 1)
        table[name] = entry
        SUSTAINED[name] = entry["varied_operands_tflops"]
    return table

OUTPUTS, INNER = 28672, 8192
BATCHES = (1, 8, 32)


def decode_bytes(tokens):
    return OUTPUTS * INNER * 2 + tokens * INNER * 2 + tokens * OUTPUTS * 2


def event_time(torch, launch, warmup, iterations):
    """Average seconds per launch measured with events on torch's current stream, which is the
    stream the library context enqueues on."""
    for index in range(warmup):
        launch(index)
    stream = torch.cuda.current_stream()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record(stream)
    for index in range(iterations):
        launch(index)
    stop.record(stream)
    stop.synchronize()
    return start.elapsed_time(stop) * 1e-3 / iterations


def host_threads():
    return len(os.sched_getaffinity(0))


def cpu_torch_linear(budget_seconds=10.0):
    """PyTorch's CPU BF16 F.linear on the headline shape (M = 32, W [28672, 8192]) with every host
    thread this process may use: what a user without the GPU library would run."""
    import torch
    import torch.nn.functional as F

    torch.set_num_threads(host_threads())
    tokens = 32
    generator = torch.Generator().manual_seed(7)
    w = (torch.randn((OUTPUTS, INNER), generator=generator) * 0.02).to(torch.bfloat16)
    x = torch.randn((tokens, INNER), generator=generator).to(torch.bfloat16)
    F.linear(x, w)
    elapsed, passes = 0.0, 0
    while elapsed < budget_seconds and passes < 1000:
        begin = time.perf_counter()
        F.linear(x, w)
        elapsed += time.perf_counter() - begin
        passes += 1
    return {
        "value": round(passes * decode_bytes(tokens) / elapsed / 1e9, 3),
        "unit": "GB/s",
        "cores": host_threads(),
        "kind": "torch-cpu",
        "sample": f"torch.nn.functional.linear, BF16, x [32, {INNER}] W [{OUTPUTS}, {INNER}] (the whole M=32 "
                  f"launch), torch.set_num_threads({host_threads()}), {passes} passes in {elapsed:.1f} s",
    }


def cpu_torch_fp8(budget_seconds=8.0):
    """PyTorch's CPU route for the FP8 block-scaled linear at 16 tokens: dequantise both operands
    to FP32 with their block scales, then mm: the plain PyTorch formulation of the same product."""
    import torch

    torch.set_num_threads(host_threads())
    tokens, outputs, inner = 16, 18432, 7168
    generator = torch.Generator().manual_seed(8)
    w = torch.randint(0, 0x7E, (outputs, inner), generator=generator, dtype=torch.uint8).view(torch.float8_e4m3fn)
    a = torch.randint(0, 0x7E, (tokens, inner), generator=generator, dtype=torch.uint8).view(torch.float8_e4m3fn)
    w_scale = torch.rand((outputs // 128, inner // 128), generator=generator) * 0.1 + 1e-4
    a_scale = torch.rand((tokens, inner // 128), generator=generator) * 0.1 + 1e-4

    def once():
        wide = w.to(torch.float32).view(outputs // 128, 128, inner // 128, 128) * w_scale[:, None, :, None]
        rows = a.to(torch.float32).view(tokens, inner // 128, 128) * a_scale[:, :, None]
        return (rows.view(tokens, inner) @ wide.view(outputs, inner).t()).to(torch.bfloat16)

    once()
    elapsed, passes = 0.0, 0
    while elapsed < budget_seconds and passes < 1000:
        begin = time.perf_counter()
        once()
        elapsed += time.perf_counter() - begin
        passes += 1
    traffic = outputs * inner + w_scale.numel() * 4 + tokens * (inner + inner // 128 * 4 + outputs * 2)
    return {
        "value": round(passes * traffic / elapsed / 1e9, 3),
        "unit": "GB/s",
        "cores": host_threads(),
        "kind": "torch-cpu",
        "sample": f"E4M3 -> FP32 dequantise with the 1x128 / 128x128 scales, then torch.mm, 16 tokens x "
                  f"[{outputs}, {inner}], torch.set_num_threads({host_threads()}), {passes} passes in {elapsed:.1f} s",
    }


def cpu_port_baseline(budget_seconds=6.0):
    """Time the CPU oracle's BF16 linear (FP64 accumulate, OpenMP) on a bounded sample of rows."""
    import oracle

    cores = len(os.sched_getaffinity(0))
    tokens = 32
    x = oracle.fill_normal_bf16(1, (tokens, INNER))
    rows = 4096
    w = oracle.fill_normal_bf16(2, (rows, INNER), std=0.02)
    out = oracle.f32_to_bf16(oracle.fill_uniform(3, (tokens, rows)) * 0)
    elapsed, passes = 0.0, 0
    while elapsed < budget_seconds and passes < 4096:
        begin = time.perf_counter()
        oracle.bgemm_f64("T", "N", rows, tokens, INNER, 1.0, w, INNER, x, INNER, 0.0, out, rows)
        elapsed += time.perf_counter() - begin
        passes += 1
    traffic = passes * (rows * INNER * 2 + tokens * INNER * 2 + tokens * rows * 2)
    return {
        "value": round(traffic / elapsed / 1e9, 3),
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "sample": f"oracle_bgemm_f64 (OpenMP, FP64 accumulate) on {rows} of {OUTPUTS} weight rows "
                  f"x {passes} passes, M=32, K={INNER}, {elapsed:.1f} s",
    }


def cpu_reference_sgemm():
    """The reference's own CPU library on the FP32 2048^3 product, when it was built."""
    import oracle

    if oracle.ref() is None:
        return None
    size = 2048
    a = oracle.fill_uniform(101, (size * size,))
    b = oracle.fill_uniform(102, (size * size,))
    c = oracle.fill_uniform(103, (size * size,)) * 0
    threads = oracle.ref_threads_available()
    oracle.ref_sgemm_packed(threads, "N", "N", size, size, size, 1.0, b, size, a, size, 0.0, c, size)
    begin = time.perf_counter()
    oracle.ref_sgemm_packed(threads, "N", "N", size, size, size, 1.0, b, size, a, size, 0.0, c, size)
    elapsed = time.perf_counter() - begin
    return {
        "value": round(2.0 * size**3 / elapsed / 1e9, 2),
        "unit": "GFLOP/s",
        "cores": threads,
        "kind": "reference",
        "sample": f"camblas_sgemm shape-aware + pthread pool, 2048^3, {elapsed:.3f} s",
    }


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=1000)
    parser.add_argument("--warmup", type=int, default=50)
    parser.add_argument("--skip-extras", action="store_true")
    parser.add_argument("--skip-cpu", action="store_true")
    parser.add_argument("--skip-traffic", action="store_true", help="do not run the rocprofv3 counter passes")
    parser.add_argument("--only", choices=("decode1", "decode8", "decode32", "prefill", "prefillnn", "copy", "traffic",
                                 "fp8m1", "fp8m16", "fp8m256", "fp8m4096", "fp8block32", "mxe4m3m16", "mxe2m1m16",
                                 "mxe4m3m4096", "mxe2m1m4096", "fp8moe", "attention", "layer", "layergraph", "sgemm2048", "dgemm4096"),
                        help="profiling aid: launch just this kernel --steps times, print nothing")
    args = parser.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (no collectives exist in the linear "
                 "path); run with --gpus 1")

    import torch

    from camblas_amd import _kernels, _native

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    generator = torch.Generator(device=device).manual_seed(20261125)

    def normal(shape, std=1.0, dtype=torch.bfloat16):
        return (torch.randn(shape, device=device, generator=generator) * std).to(dtype)

    weights = [normal((OUTPUTS, INNER), 0.02) for _ in range(3)]
    inputs = {m: normal((m, INNER)) for m in BATCHES}
    outputs = {m: torch.empty((m, OUTPUTS), dtype=torch.bfloat16, device=device) for m in BATCHES}

    if args.only:
        profile_only(args, torch, _kernels, _native, device, normal, weights, inputs, outputs)
        return

    def step(index):
        for position, m in enumerate(BATCHES):
            weight = weights[(index * len(BATCHES) + position) % 3]
            _kernels.matmul(inputs[m], weight.t(), out=outputs[m])

    def timed(steps):
        torch.cuda.synchronize()
        begin = time.perf_counter()
        for index in range(steps):
            step(index)
        torch.cuda.synchronize()
        return time.perf_counter() - begin

    for index in range(args.warmup):
        step(index)
    elapsed = timed(args.steps)
    step_bytes = sum(decode_bytes(m) for m in BATCHES)
    steps = args.steps
    short_run = None
    if elapsed < LONG_REGION:
        # too short a region for a wall clock (a few milliseconds are mostly the loop's start and the
        # last synchronisation): enough steps to fill LONG_REGION are timed, and those are reported;
        # the requested region is kept beside them
        short_run = {"steps": args.steps, "ms": round(elapsed * 1e3, 2),
                     "value": round(step_bytes * args.steps / elapsed / 1e9, 1)}
        steps = int(LONG_REGION * 1.1 / (elapsed / max(args.steps, 1))) + 1
        elapsed = timed(steps)
    value = step_bytes * steps / elapsed / 1e9

    # dominant kernel: the M=32 launch, timed alone with events on the launch stream
    per_launch = {}
    for m in BATCHES:
        seconds = event_time(
            torch, lambda i, m=m: _kernels.matmul(inputs[m], weights[i % 3].t(), out=outputs[m]),
            5, 30)
        per_launch[m] = seconds
    _, plan_text = _native.plan_describe(2, "T", "N", OUTPUTS, 32, INNER, INNER, INNER, OUTPUTS)
    achieved = decode_bytes(32) / per_launch[32]
    roofline = {
        "bound": "hbm",
        "kernel": plan_text,
        "achieved": round(achieved / 1e9, 1),
        "peak": HBM_PEAK / 1e9,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK, 4),
        "traffic": None,
        "launch_us": round(per_launch[32] * 1e6, 2),
    }

    also = {
        "decode_linear_us": {str(m): round(per_launch[m] * 1e6, 2) for m in BATCHES},
        "decode_linear_gbps": {str(m): round(decode_bytes(m) / per_launch[m] / 1e9, 1)
                               for m in BATCHES},
    }
    if not args.skip_extras:
        also.update(extras(torch, _kernels, _native, device, normal))
    if not args.skip_traffic:  # after every timed launch of this process: the child runs leave the GPU idle
        counters = measured_traffic()
        roofline["traffic"] = counters.pop("traffic")
        roofline["traffic_source"] = counters
    result = {
        "metric": "decode-GEMV HBM GB/s (BF16 linear W[28672,8192], M in {1,8,32}); TFLOP/s of the "
                  "BF16/FP8 prefill linears under 'also'",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": args.warmup,
        "ms_per_step": round(elapsed / steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "BF16 decode linear y = x W^T, W [28672, 8192] ~N(0,0.02), x [M, 8192] "
                        "~N(0,1), M in {1,8,32}, fp32 accumulate, BF16 out; 3 rotating weight "
                        "copies (HBM-cold)",
            "entry_point": "camblas_cuda_bgemm('T','N')",
            "peak_fraction": round(value * 1e9 / HBM_PEAK, 4),
            "timed_region_ms": round(elapsed * 1e3, 2),
            "requested_steps": args.steps,
            "short_run": short_run,
        },
        "roofline": roofline,
        "cpu_baseline": None if args.skip_cpu else cpu_torch_linear(),
        "also": also,
    }
    if not args.skip_cpu:
        also["cpu_torch_fp8_dequantise_mm_m16"] = cpu_torch_fp8()
        also["cpu_oracle_port_bf16_linear"] = cpu_port_baseline()
        reference = cpu_reference_sgemm()
        if reference:
            also["cpu_reference_sgemm_2048"] = reference
    print(json.dumps(result))


def probes():
    """The bench-side calibration library (a copy of known traffic, a stream of matrix instructions);
    built by camblas_amd._build.build_probes(), never part of libcamblas_hip.so."""
    import ctypes as ct

    if not hasattr(probes, "library"):
        from camblas_amd import _native

        lib = ct.CDLL(str(_native.library_path().parent / "libcamblas_probes.so"))
        lib.camblas_probe_copy.argtypes = [ct.c_void_p, ct.c_size_t, ct.c_void_p, ct.c_void_p]
        lib.camblas_probe_matrix.argtypes = [ct.c_void_p, ct.c_int, ct.c_int, ct.c_int, ct.c_int,
                                             ct.c_void_p, ct.c_size_t, ct.POINTER(ct.c_double)]
        lib.camblas_probe_matrix_single.argtypes = lib.camblas_probe_matrix.argtypes
        probes.library = lib
    return probes.library


def counter_pass(counter):
    """One child run of this file under `rocprofv3 --pmc <counter>`: mean KiB per dispatch of the
    copy probe and of the M = 32 decode kernel."""
    tool = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    with tempfile.TemporaryDirectory(prefix="camblas_pmc_", dir="/tmp") as directory:
        command = [tool, "--pmc", counter, "--output-format", "csv", "-d", directory, "-o", "t", "--",
                   sys.executable, str(ROOT / "bench.py"), "--only", "traffic", "--steps", "6", "--warmup", "0"]
        environment = dict(os.environ, TMPDIR="/tmp")
        subprocess.run(command, cwd=directory, env=environment, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL,
                       timeout=180, check=True)
        sums, counts = {"copy": 0.0, "decode": 0.0}, {"copy": 0, "decode": 0}
        for path in Path(directory).rglob("*counter_collection.csv"):
            with open(path, newline="") as handle:
                for row in csv.DictReader(handle):
                    if row.get("Counter_Name") != counter:
                        continue
                    name = row.get("Kernel_Name", "")
                    kind = "copy" if "copy_probe" in name else "decode" if "bgemv_stream" in name else None
                    if kind:
                        sums[kind] += float(row["Counter_Value"])
                        counts[kind] += 1
        if not counts["copy"] or not counts["decode"]:
            raise RuntimeError("no counter rows for the copy probe or the decode kernel")
        return sums["copy"] / counts["copy"], sums["decode"] / counts["decode"]


def measured_traffic():
    """HBM bytes of one M = 32 launch from the L2-to-fabric byte counters, measured now: FETCH_SIZE and
    WRITE_SIZE (KiB per dispatch) each in a run of its own, each scaled by what the same counter
    reads for a plain copy of COPY_BYTES in that run. {"traffic": None, ...} when the profiler is
    missing or a pass fails."""
    try:
        copy_fetch, decode_fetch = counter_pass("FETCH_SIZE")
        copy_write, decode_write = counter_pass("WRITE_SIZE")
    except (OSError, subprocess.SubprocessError, RuntimeError, KeyError, ValueError) as problem:
        return {"traffic": None, "problem": str(problem)[:200]}
    kib = COPY_BYTES / 1024
    fetch_factor, write_factor = kib / copy_fetch, kib / copy_write
    traffic = (decode_fetch * fetch_factor + decode_write * write_factor) * 1024
    return {"traffic": int(traffic), "fetch_kib": round(decode_fetch, 1), "write_kib": round(decode_write, 1),
            "fetch_factor": round(fetch_factor, 4), "write_factor": round(write_factor, 4),
            "copy_bytes_each_way": COPY_BYTES, "algorithmic": decode_bytes(32)}


COPY_BYTES = 448 << 20


def profile_only(args, torch, _kernels, _native, device, normal, weights, inputs, outputs):
    """Launch one kernel repeatedly under an external profiler."""
    import ctypes as ct

    if args.only.startswith("decode"):
        m = int(args.only[6:])

        def launch(i):
            _kernels.matmul(inputs[m], weights[i % 3].t(), out=outputs[m])
    elif args.only in ("copy", "traffic"):
        source, target = weights[0], weights[1]
        also_decode = args.only == "traffic"  # the counter passes want both kernels in one run

        def launch(i):
            status = probes().camblas_probe_copy(
                ct.c_void_p(torch.cuda.current_stream(device).cuda_stream), COPY_BYTES,
                ct.c_void_p(source.data_ptr()), ct.c_void_p(target.data_ptr()))
            assert status == 0, status
            if also_decode:
                _kernels.matmul(inputs[32], weights[2].t(), out=outputs[32])
    elif args.only.startswith("fp8m") and args.only != "fp8moe":
        tokens, features, inner = int(args.only[4:]), 18432, 7168
        rotate = 3 if tokens <= 256 else 1
        copies = [torch.randint(0, 0x7E, (features, inner), device=device, dtype=torch.uint8)
                  .view(torch.float8_e4m3fn) for _ in range(rotate)]
        w_scale = torch.rand((features // 128, inner // 128), device=device) * 0.1 + 1e-4
        a = torch.randint(0, 0x7E, (tokens, inner), device=device, dtype=torch.uint8)
        a = a.view(torch.float8_e4m3fn)
        a_scale = torch.rand((tokens, inner // 128), device=device) * 0.1 + 1e-4
        out = torch.empty((tokens, features), dtype=torch.bfloat16, device=device)

        def launch(i):
            _kernels.fp8_block_matmul(a, a_scale, copies[i % rotate], w_scale, out=out)
    elif args.only == "fp8moe":
        step = moe_step(torch, _kernels, device, normal)

        def launch(i):
            step(i)
    elif args.only == "fp8block32":
        features, inner = 18432, 7168
        copies = [torch.randint(0, 0x7E, (features, inner), device=device, dtype=torch.uint8)
                  .view(torch.float8_e4m3fn) for _ in range(3)]
        token = torch.randint(0, 0x7E, (1, inner), device=device, dtype=torch.uint8).view(torch.float8_e4m3fn)
        token_scale = torch.rand((1, inner // 32), device=device) * 0.1 + 1e-4
        block_scale = torch.rand((features // 32, inner // 32), device=device) * 0.1 + 1e-4

        def launch(i):
            _kernels.fp8_decode(token, token_scale, copies[i % 3], block_scale)
    elif args.only.startswith("mx"):
        packed, tokens, features, inner = args.only.startswith("mxe2m1"), int(args.only[7:]), 18432, 7168
        rotate = 1 if tokens > 256 else 6 if packed else 3  # few tokens: weights from HBM, not the last-level cache
        sets = [mx_operands(torch, device, packed, tokens, features, inner) for _ in range(rotate)]

        def launch(i):
            w, scale, a, a_scale = sets[i % rotate]
            _kernels.quantized_matmul(a, a_scale, w, scale)
    elif args.only == "sgemm2048":
        size = 2048
        a32, b32 = torch.rand((size, size), device=device) * 2 - 1, torch.rand((size, size), device=device) * 2 - 1
        c32 = torch.empty((size, size), device=device)

        def launch(i):
            _kernels.matmul(a32, b32, out=c32)
    elif args.only == "dgemm4096":
        size = 4096
        a64 = torch.rand((size, size), device=device, dtype=torch.float64) * 2 - 1
        b64 = torch.rand((size, size), device=device, dtype=torch.float64) * 2 - 1
        c64 = torch.empty((size, size), device=device, dtype=torch.float64)

        def launch(i):
            _kernels.matmul(a64, b64, out=c64)
    elif args.only == "prefillnn":
        size = 4096
        x, w = normal((size, size)), normal((size, size), 0.02)
        y = torch.empty((size, size), dtype=torch.bfloat16, device=device)

        def launch(i):
            _kernels.matmul(x, w, out=y)
    elif args.only in ("attention", "layer"):
        layer, attention = layer_step(torch, _kernels, device, normal)
        launch = (lambda i: layer()) if args.only == "layer" else (lambda i: attention())
    elif args.only == "layergraph":  # the layer step replayed from a one-step graph
        layer, _ = layer_step(torch, _kernels, device, normal)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            layer()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            layer()

        def launch(i):
            graph.replay()
    else:
        tokens, features = 4096, 10240
        x, w = normal((tokens, INNER)), normal((features, INNER), 0.02)
        y = torch.empty((tokens, features), dtype=torch.bfloat16, device=device)

        def launch(i):
            _kernels.matmul(x, w.t(), out=y)
    for index in range(args.warmup + args.steps):
        launch(index)
    torch.cuda.synchronize()


MOE_SHAPE = (289, 4096, 512, 9)  # experts, hidden, expert width, choices per token


def moe_step(torch, _kernels, device, normal):
    """Single-token FP8 expert step at the shapes of the reference's hook: 9 of 289 experts, gate/up
    [1024, 4096] and down [4096, 512] per expert; the chosen experts rotate over 32 disjoint sets so
    that the weights come from HBM."""
    experts, hidden, width, choices = MOE_SHAPE
    w1 = torch.randint(0, 0x7E, (experts, 2 * width, hidden), device=device, dtype=torch.uint8).view(torch.float8_e4m3fn)
    w2 = torch.randint(0, 0x7E, (experts, hidden, width), device=device, dtype=torch.uint8).view(torch.float8_e4m3fn)
    s1 = torch.rand((experts, 2 * width // 128, hidden // 128), device=device) * 0.001 + 0.001
    s2 = torch.rand((experts, hidden // 128, width // 128), device=device) * 0.001 + 0.001
    token = normal((1, hidden))
    routing = torch.linspace(0.05, 1.0, choices, device=device)
    chosen = [torch.arange(choices * i, choices * i + choices, device=device, dtype=torch.int32) for i in range(32)]
    result = torch.empty((1, hidden), dtype=torch.bfloat16, device=device)
    return lambda i: _kernels.fp8_moe_decode(token, w1, w2, s1, s2, chosen[i % 32], routing, factor=2.5, out=result)


def mx_operands(torch, device, packed, tokens, features, inner):
    """Random E8M0 block-scaled operands: weights [features, inner] E4M3 (scales per 32 x 32 block) or
    packed E2M1 (scales per row and 32 inputs), E4M3 tokens with one scale per 32 inputs."""
    if packed:
        w = torch.randint(0, 256, (features, inner // 2), device=device, dtype=torch.uint8)
        scale = torch.randint(120, 130, (features, inner // 32), device=device, dtype=torch.uint8)
    else:
        w = torch.randint(0, 0x7E, (features, inner), device=device, dtype=torch.uint8).view(torch.float8_e4m3fn)
        scale = torch.randint(120, 130, (features // 32, inner // 32), device=device, dtype=torch.uint8)
    a = torch.randint(0, 0x7E, (tokens, inner), device=device, dtype=torch.uint8).view(torch.float8_e4m3fn)
    a_scale = torch.randint(120, 130, (tokens, inner // 32), device=device, dtype=torch.uint8)
    return w, scale, a, a_scale


KV_BYTES = 2 * 32 * 2048 * 8 * 128 * 2
LAYER_BYTES = 2 * (10240 * 8192 + 8192 * 8192 + 3 * 28672 * 8192) + KV_BYTES + 10e6


def layer_step(torch, _kernels, device, normal):
    """Llama-3.1-70B decoder-layer shapes at batch 32 and KV context 2048, random-init weights, all
    positions at the last slot; returns closures running the whole step and the attention alone."""
    batch, hidden, q_heads, kv_heads, dim, ffn, context = 32, 8192, 64, 8, 128, 28672, 2048
    weights = {
        "input_norm": normal((hidden,), 0.02) + 1, "post_norm": normal((hidden,), 0.02) + 1,
        "qkv": normal(((q_heads + 2 * kv_heads) * dim, hidden), 0.02),
        "o": normal((hidden, q_heads * dim), 0.02), "gate": normal((ffn, hidden), 0.02),
        "up": normal((ffn, hidden), 0.02), "down": normal((hidden, ffn), 0.02),
    }
    k_cache = normal((batch, context, kv_heads, dim))
    v_cache = normal((batch, context, kv_heads, dim))
    hidden_in, residual = normal((batch, hidden)), normal((batch, hidden))
    positions = torch.full((batch,), context - 1, dtype=torch.int32, device=device)
    lengths = positions + 1
    q = normal((batch, q_heads, dim))
    # the attention alone is timed over three rotating caches (805 MB) so that it reads HBM
    caches = [(k_cache, v_cache)] + [(normal((batch, context, kv_heads, dim)),
                                      normal((batch, context, kv_heads, dim))) for _ in range(2)]
    turn = [0]

    def step():
        return _kernels.decoder_layer_decode(
            hidden_in, residual, weights, k_cache, v_cache, positions, lengths, q_heads=q_heads,
            kv_heads=kv_heads, head_dim=dim)

    def attention():
        turn[0] = (turn[0] + 1) % 3
        return _kernels.gqa_decode_attention(q, caches[turn[0]][0], caches[turn[0]][1], lengths)

    # the same step with both residual-add + RMSNorm launches fused into the linears around them: it
    # takes and returns the state the layers pass along (the added residual stream and its rows'
    # partial sums of squares)
    state = _kernels.add_residual_squares(hidden_in, residual)

    def fused_step():
        return _kernels.decoder_layer_decode_fused(
            state, weights, k_cache, v_cache, positions, lengths, q_heads=q_heads, kv_heads=kv_heads, head_dim=dim)

    step.fused = fused_step
    return step, attention


def extras(torch, _kernels, _native, device, normal):
    """The other configurations, each as absolute rate and fraction of its roofline."""
    found = {}
    found["matrix_instruction_issue_rate"] = measure_sustained(torch, device)
    # BF16 prefill linear and addmm (beta = 1)
    tokens, outputs, inner = 4096, 10240, 8192
    prefill_instruction = bf16_instruction(
        _native.plan_describe(2, "T", "N", outputs, tokens, inner, inner, inner, outputs)[1])
    x, w = normal((tokens, inner)), normal((outputs, inner), 0.02)
    y = torch.empty((tokens, outputs), dtype=torch.bfloat16, device=device)
    c = normal((tokens, outputs))
    flops = 2.0 * tokens * outputs * inner
    # (matrix-bound lines run 50 + 100 launches: the first launches after a memory-bound phase run at a
    # lower clock, which a short loop would fold into the average)
    seconds = event_time(torch, lambda i: _kernels.matmul(x, w.t(), out=y), 50, 100)
    found["bf16_prefill_linear"] = {
        "shape": [tokens, outputs, inner], "us": round(seconds * 1e6, 1),
        "tflops": round(flops / seconds / 1e12, 1),
        "roofline": roofline_of("mfma bf16", flops, seconds, prefill_instruction),
    }
    seconds = event_time(torch, lambda i: _kernels.addmm(c, x, w.t(), beta=1.0), 10, 50)
    found["bf16_prefill_addmm_beta1"] = {
        "us": round(seconds * 1e6, 1), "tflops": round(flops / seconds / 1e12, 1),
        "roofline": roofline_of("mfma bf16", flops, seconds, prefill_instruction),
        "note": "full [tokens, outputs] addend read by the product's epilogue (no expand+clone copy)",
    }
    row = normal((outputs,))
    seconds = event_time(torch, lambda i: _kernels.addmm(row, x, w.t(), beta=1.0), 10, 50)
    found["bf16_prefill_addmm_bias_row"] = {
        "us": round(seconds * 1e6, 1), "tflops": round(flops / seconds / 1e12, 1),
        "roofline": roofline_of("mfma bf16", flops, seconds, prefill_instruction),
        "note": "[outputs] bias row of a linear layer, read by the product's epilogue",
    }
    del x, w, y, c, row
    # BF16 products of square operands: row-major a @ b with neither operand K-contiguous ('N','N': W is
    # copied into LDS as it lies) at 4096^3, and the linear layout ('T','N') and 'N','N' at 8192^3, whose
    # 256 x 256 tiles make four whole rounds of workgroups
    for size in (4096, 8192):
        x, w = normal((size, size)), normal((size, size), 0.02)
        y = torch.empty((size, size), dtype=torch.bfloat16, device=device)
        layouts = (("nn", lambda i: _kernels.matmul(x, w, out=y), "N"),) + (
            (("tn", lambda i: _kernels.matmul(x, w.t(), out=y), "T"),) if size == 8192 else ())
        for name, launch, trans_a in layouts:
            seconds = event_time(torch, launch, 10, 30)
            plan_text = _native.plan_describe(2, trans_a, "N", size, size, size, size, size, size)[1]
            found[f"bf16_matmul_{name}_{size}"] = {
                "us": round(seconds * 1e6, 1), "tflops": round(2.0 * size**3 / seconds / 1e12, 1), "plan": plan_text,
                "roofline": roofline_of("mfma bf16", 2.0 * size**3, seconds, bf16_instruction(plan_text))}
        del x, w, y
    # BF16 linear at 256 tokens on a square projection (64 tiles of 128 x 256 for 256 compute units:
    # K is divided over workgroups); five weight copies rotate so that the weights come from HBM
    outputs, inner, tokens = 8192, 8192, 256
    copies = [normal((outputs, inner), 0.02) for _ in range(5)]
    x = normal((tokens, inner))
    y = torch.empty((tokens, outputs), dtype=torch.bfloat16, device=device)
    seconds = event_time(torch, lambda i: _kernels.matmul(x, copies[i % 5].t(), out=y), 10, 60)
    found["bf16_linear_256_tokens_8192x8192"] = {
        "us": round(seconds * 1e6, 1), "tflops": round(2.0 * tokens * outputs * inner / seconds / 1e12, 1),
        "roofline": roofline_of("hbm", outputs * inner * 2 + tokens * (inner + outputs) * 2, seconds),
        "plan": _native.plan_describe(2, "T", "N", outputs, tokens, inner, inner, inner, outputs)[1],
    }
    # x @ W with a row-major W [inner, outputs] ('N','N') and 16 tokens: the kernel that streams W as it lies
    tokens = 16
    x = normal((tokens, inner))
    y = torch.empty((tokens, outputs), dtype=torch.bfloat16, device=device)
    seconds = event_time(torch, lambda i: _kernels.matmul(x, copies[i % 5], out=y), 10, 60)
    found["bf16_x_at_w_row_major_16_tokens_8192x8192"] = {
        "us": round(seconds * 1e6, 1),
        "roofline": roofline_of("hbm", outputs * inner * 2 + tokens * (inner + outputs) * 2, seconds),
        "plan": _native.plan_describe(2, "N", "N", outputs, tokens, inner, outputs, inner, outputs)[1],
    }
    del copies, x, y
    # decode batches between the streaming kernel's two- and four-tile forms, on the widest and on a narrow
    # projection of the layer (three weight copies rotate)
    mid = {}
    for outputs, inner in ((28672, 8192), (8192, 8192)):
        copies = [normal((outputs, inner), 0.02) for _ in range(3)]
        for tokens in (48, 64):
            x = normal((tokens, inner))
            y = torch.empty((tokens, outputs), dtype=torch.bfloat16, device=device)
            seconds = event_time(torch, lambda i: _kernels.matmul(x, copies[i % 3].t(), out=y), 10, 60)
            mid["%dx%d_%d_tokens" % (outputs, inner, tokens)] = {
                "us": round(seconds * 1e6, 1),
                "roofline": roofline_of("hbm", outputs * inner * 2 + tokens * (inner + outputs) * 2, seconds),
                "plan": _native.plan_describe(2, "T", "N", outputs, tokens, inner, inner, inner, outputs)[1],
            }
        del copies, x, y
    found["bf16_linear_48_and_64_tokens"] = mid
    # FP8 block-scaled linear; the decode sizes rotate three weight copies (396 MB) so that the
    # weights come from HBM rather than from the 256 MB last-level cache
    outputs, inner = 18432, 7168
    copies = [torch.randint(0, 0x7E, (outputs, inner), device=device, dtype=torch.uint8)
              .view(torch.float8_e4m3fn) for _ in range(3)]
    w_scale = torch.rand((outputs // 128, inner // 128), device=device) * 0.1 + 1e-4
    fp8 = {}
    for tokens in (1, 16, 256, 4096):
        a = torch.randint(0, 0x7E, (tokens, inner), device=device, dtype=torch.uint8)
        a = a.view(torch.float8_e4m3fn)
        a_scale = torch.rand((tokens, inner // 128), device=device) * 0.1 + 1e-4
        out = torch.empty((tokens, outputs), dtype=torch.bfloat16, device=device)
        rotate = 3 if tokens <= 256 else 1
        seconds = event_time(
            torch, lambda i: _kernels.fp8_block_matmul(a, a_scale, copies[i % rotate], w_scale,
                                                       out=out), *((50, 100) if tokens >= 4096 else (20, 60)))
        flops = 2.0 * tokens * outputs * inner
        traffic = outputs * inner + w_scale.numel() * 4 + tokens * (inner + inner // 128 * 4 + outputs * 2)
        # few tokens stream the weights once (HBM roofline); 4096 tokens are matrix-core work
        bound = ("mfma fp8", flops) if flops / FP8_PEAK > traffic / HBM_PEAK else ("hbm", traffic)
        plan_text = _native.plan_describe(3, "T", "N", outputs, tokens, inner, inner, inner, outputs)[1]
        instruction = "e4m3_scaled_16x16x128" if "fp8dma16" in plan_text else "e4m3_scaled_32x32x64"
        fp8[str(tokens)] = {
            "us": round(seconds * 1e6, 1), "tflops": round(flops / seconds / 1e12, 1),
            "gbps": round(traffic / seconds / 1e9, 1),
            "roofline": roofline_of(*bound, seconds, instruction if bound[0] != "hbm" else None),
        }
    found["fp8_block_linear_18432x7168"] = fp8
    # single-token block-32 product of the reference header (FP32 scales per 32 x 32 block)
    token = torch.randint(0, 0x7E, (1, inner), device=device, dtype=torch.uint8).view(torch.float8_e4m3fn)
    token_scale = torch.rand((1, inner // 32), device=device) * 0.1 + 1e-4
    block_scale = torch.rand((outputs // 32, inner // 32), device=device) * 0.1 + 1e-4
    seconds = event_time(
        torch, lambda i: _kernels.fp8_decode(token, token_scale, copies[i % 3], block_scale), 10, 20)
    traffic = outputs * inner + block_scale.numel() * 4 + inner + inner // 32 * 4 + outputs * 2
    found["fp8_block32_decode_18432x7168"] = {
        "us": round(seconds * 1e6, 1), "gbps": round(traffic / seconds / 1e9, 1),
        "roofline": roofline_of("hbm", traffic, seconds),
    }
    # E8M0 block-scaled (microscaling) decode products of the reference header: E4M3 and packed E2M1
    # weights [18432, 7168], 16 tokens, rotating weight copies
    mx = {}
    tokens = 16
    a = torch.randint(0, 0x7E, (tokens, inner), device=device, dtype=torch.uint8).view(torch.float8_e4m3fn)
    a_scale = torch.randint(120, 130, (tokens, inner // 32), device=device, dtype=torch.uint8)
    for name, packed in (("e4m3", False), ("e2m1", True)):
        if packed:
            # six copies: three of them (198 MB) would fit the 256 MB last-level cache
            weights = [torch.randint(0, 256, (outputs, inner // 2), device=device, dtype=torch.uint8)
                       for _ in range(6)]
            scale = torch.randint(120, 130, (outputs, inner // 32), device=device, dtype=torch.uint8)
        else:
            weights = copies
            scale = torch.randint(120, 130, (outputs // 32, inner // 32), device=device, dtype=torch.uint8)
        seconds = event_time(
            torch, lambda i: _kernels.quantized_matmul(a, a_scale, weights[i % len(weights)], scale),
            10, 20)
        traffic = weights[0].numel() + scale.numel() + tokens * (inner + inner // 32 + outputs * 2)
        mx[name] = {"us": round(seconds * 1e6, 1), "gbps": round(traffic / seconds / 1e9, 1),
                    "roofline": roofline_of("hbm", traffic, seconds)}
    found["mx_quantized_matmul_m16_18432x7168"] = mx
    # the same products at 4096 tokens (tiled kernel, hardware-scaled matrix instructions)
    mx = {}
    for name, packed in (("e4m3", False), ("e2m1", True)):
        w, scale, a, a_scale = mx_operands(torch, device, packed, 4096, outputs, inner)
        seconds = event_time(torch, lambda i: _kernels.quantized_matmul(a, a_scale, w, scale), 50, 100)
        flops = 2.0 * 4096 * outputs * inner
        mx[name] = {"us": round(seconds * 1e6, 1), "tflops": round(flops / seconds / 1e12, 1),
                    "roofline": roofline_of("mfma fp8", flops, seconds, "e2m1_x_e4m3_scaled_32x32x64" if packed
                                            else "e4m3_scaled_32x32x64")}
        del w, scale, a, a_scale
    found["mx_quantized_matmul_m4096_18432x7168"] = mx
    # a narrow projection with a long K at 128 rows (56 tiles of 128 x 128 for 256 compute units: K is
    # divided over workgroups); five weight copies rotate so that the weights come from HBM
    mx = {}
    for name, packed in (("e4m3", False), ("e2m1", True)):
        parts = [mx_operands(torch, device, packed, 128, 7168, 18432) for _ in range(5 if not packed else 8)]
        a, a_scale = parts[0][2], parts[0][3]
        seconds = event_time(
            torch, lambda i: _kernels.quantized_matmul(a, a_scale, parts[i % len(parts)][0], parts[i % len(parts)][1]), 10, 60)
        traffic = parts[0][0].numel() + parts[0][1].numel() + 128 * (18432 + 18432 // 32 + 7168 * 2)
        mx[name] = {"us": round(seconds * 1e6, 1), "roofline": roofline_of("hbm", traffic, seconds)}
        del parts, a, a_scale
    found["mx_quantized_matmul_m128_7168x18432"] = mx
    # the grouped form as an MoE prefill meets it: 32 experts of [4096, 7168] with a capacity of 1024
    # rows each, every expert a quarter full (the rest of the capacity comes back as zeros)
    experts, capacity, features, inner = 32, 1024, 4096, 7168
    grouped = {}
    for name, packed in (("e4m3_weights", False), ("e2m1_weights", True)):
        parts = [mx_operands(torch, device, packed, 1, features, inner)[:2] for _ in range(experts)]
        table = torch.tensor([[w.data_ptr(), scale.data_ptr()] for w, scale in parts], dtype=torch.int64,
                             device=device)
        tokens = torch.randint(0, 0x7E, (experts, capacity, inner), device=device,
                               dtype=torch.uint8).view(torch.float8_e4m3fn)
        token_scale = torch.randint(120, 130, (experts, capacity, inner // 32), device=device, dtype=torch.uint8)
        order = torch.arange(experts, dtype=torch.int32, device=device)
        for label, fill in (("full", capacity), ("quarter_full", capacity // 4)):
            counts = torch.full((experts,), fill, dtype=torch.int32, device=device)
            seconds = event_time(
                torch, lambda i: _kernels.grouped_quantized_matmul(tokens, token_scale, table, order, counts,
                                                                   outputs=features, packed=packed), 10, 30)
            grouped[name + "_" + label] = {
                "us": round(seconds * 1e6, 1),
                "roofline": roofline_of("mfma fp8", 2.0 * experts * fill * features * inner, seconds)}
        del parts, table, tokens, token_scale
    found["mx_grouped_32_experts_4096x7168_capacity_1024"] = grouped
    # decode attention when the cache is larger than the sequences: 32 sequences of 512 positions in a
    # cache of 8192 (64 query heads, 8 KV heads of 128)
    cache_k = normal((32, 8192, 8, 128))
    cache_v = normal((32, 8192, 8, 128))
    query = normal((32, 64, 128))
    live = torch.full((32,), 512, dtype=torch.int32, device=device)
    seconds = event_time(torch, lambda i: _kernels.gqa_decode_attention(query, cache_k, cache_v, live), 20, 60)
    found["gqa_decode_512_live_of_8192"] = {
        "us": round(seconds * 1e6, 1), "roofline": roofline_of("hbm", 2 * 32 * 512 * 8 * 128 * 2, seconds)}
    del cache_k, cache_v, query
    del copies, w_scale
    # FP32 SGEMM 2048^3 (plumbing)
    size = 2048
    a32 = torch.rand((size, size), device=device) * 2 - 1
    b32 = torch.rand((size, size), device=device) * 2 - 1
    c32 = torch.empty((size, size), device=device)
    seconds = event_time(torch, lambda i: _kernels.matmul(a32, b32, out=c32), 20, 60)
    found["fp32_sgemm_2048"] = {"us": round(seconds * 1e6, 1),
                                "roofline": roofline_of("mfma fp32", 2.0 * size**3, seconds, "fp32_32x32x2")}
    # single-token FP8 expert step (9 of 289 experts, rotating sets)
    experts, hidden, width, choices = MOE_SHAPE
    step = moe_step(torch, _kernels, device, normal)
    seconds = event_time(torch, step, 10, 40)
    traffic = choices * (2 * width * hidden + hidden * width)
    found["fp8_moe_decode_9_of_289_experts"] = {
        "us": round(seconds * 1e6, 1), "roofline": roofline_of("hbm", traffic, seconds),
        "note": "two launches; bound by launch and latency, not bandwidth"}
    del step
    import ctypes as ct

    native = _native.context(device)
    # FP64 DGEMM 4096^3 (plumbing), through the C entry point

    size = 4096
    a64 = torch.rand((size, size), device=device, dtype=torch.float64) * 2 - 1
    b64 = torch.rand((size, size), device=device, dtype=torch.float64) * 2 - 1
    c64 = torch.empty((size, size), device=device, dtype=torch.float64)
    seconds = event_time(
        torch, lambda i: native.call("dgemm", b"N", b"N", size, size, size, ct.c_double(1.0),
                                     ct.c_void_p(a64.data_ptr()), size, ct.c_void_p(b64.data_ptr()), size,
                                     ct.c_double(0.0), ct.c_void_p(c64.data_ptr()), size), 2, 5)
    found["fp64_dgemm_4096"] = {"us": round(seconds * 1e6, 1),
                                "roofline": roofline_of("mfma fp64", 2.0 * size**3, seconds)}
    del a64, b64, c64
    # FP32 SGEMM 8192^3: the ordinary kernel and the default policy (two Strassen levels from 8192;
    # its time includes the guard's stream synchronisation), flops counted as 2 n^3 for both
    size = 8192
    a32 = torch.rand((size, size), device=device, dtype=torch.float32) * 2 - 1
    b32 = torch.rand((size, size), device=device, dtype=torch.float32) * 2 - 1
    c32 = torch.empty((size, size), device=device, dtype=torch.float32)
    entry = {}
    for policy in ("classical", "auto"):
        with _native.algorithm(policy):
            policy_context = _native.context(device)
            seconds = event_time(
                torch, lambda i: policy_context.call(
                    "sgemm", b"N", b"N", size, size, size, ct.c_float(1.0), ct.c_void_p(a32.data_ptr()), size,
                    ct.c_void_p(b32.data_ptr()), size, ct.c_float(0.0), ct.c_void_p(c32.data_ptr()), size), 1, 3)
        entry[policy] = {"ms": round(seconds * 1e3, 2),
                         "roofline": roofline_of("mfma fp32", 2.0 * size**3, seconds)}
    _native.context(device)  # back to the thread's policy
    found["fp32_sgemm_8192"] = entry
    del a32, b32, c32
    # decoder-layer decode step (Llama-3.1-70B shapes, batch 32, KV context 2048)
    step, attention = layer_step(torch, _kernels, device, normal)

    def layer(i):
        return step()

    eager = event_time(torch, layer, 10, 50)
    fused_norms = event_time(torch, lambda i: step.fused(), 10, 50)
    # the same step replayed from a captured graph (capture on a side stream after a warm-up there)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer(0)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        layer(0)
    replayed = event_time(torch, lambda i: graph.replay(), 20, 100)
    # a model replays all of its layers from one graph: eight steps in one graph show how much of a
    # replay is paid per launch of a graph rather than per kernel in it
    layers = 8
    stack = torch.cuda.CUDAGraph()
    with torch.cuda.graph(stack, stream=side):
        for _ in range(layers):
            layer(0)
    stacked = event_time(torch, lambda i: stack.replay(), 5, 20) / layers
    traffic = LAYER_BYTES
    seconds = event_time(torch, lambda i: attention(), 20, 60)
    found["gqa_decode_attention_b32_ctx2048"] = {
        "us": round(seconds * 1e6, 1), "roofline": roofline_of("hbm", KV_BYTES, seconds),
    }
    found["llama70b_layer_decode_b32_ctx2048"] = {
        "eager_us": round(eager * 1e6, 1), "graph_us": round(replayed * 1e6, 1),
        "graph_of_8_steps_us_per_step": round(stacked * 1e6, 1),
        "fused_norms_eager_us": round(fused_norms * 1e6, 1),
        "roofline": roofline_of("hbm", traffic, min(eager, replayed, stacked)),
        "note": "one layer, 8 launches (rotary embedding and cache append run inside the attention's first "
                "kernel); rate from the fastest of stream launches, a one-step graph and an eight-step graph "
                "(all device-bound); weights not rotated (1.7 GB per layer, beyond the 256 MB last-level "
                "cache). fused_norms: the 6-launch form with both residual-add + RMSNorm steps inside the "
                "linears around them, which pays up to 16 tokens and costs time at 32 (every workgroup "
                "normalises all tokens)",
    }
    return found


if __name__ == "__main__":
    main()
