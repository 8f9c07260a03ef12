"""ctypes loader for libcamblas_hip.so and per-(thread, device, stream) contexts.

Host-side mirror of the reference's private loader (camblas/_native.py): the same environment
contract (CAMBLAS_CUDA_LIBRARY selects the core library, the tensor binding
`_camblas_cuda_torch*.so` is looked up beside it), the same algorithm names and counter names, the
same rules about stream capture and fork. There is no CPU fallback: a missing library raises.
"""

import atexit
import ctypes as ct
import importlib.util
import os
import threading
from contextlib import contextmanager
from functools import lru_cache
from pathlib import Path

import torch

PACKAGE = Path(__file__).resolve().parent
DEFAULT_LIBRARY = PACKAGE / "lib" / "libcamblas_hip.so"

# ref: camblas/_native.py:17-36
ALGORITHMS = {
    "auto": 0,
    "classical": 1,
    "strassen": 2,
    "lt": 3,
    "symmetric": 4,
    "strassen2": 5,
    "strassen3": 6,
    "strassen4": 7,
}
_ALGORITHMS = ALGORITHMS
COUNTERS = ("classical", "strassen", "gram", "affine", "lt", "guard_fallback", "attention", "backward")

_P, _I, _F, _D, _C = ct.c_void_p, ct.c_int, ct.c_float, ct.c_double, ct.c_char
_U64, _SZ = ct.c_uint64, ct.c_size_t


def _gemm(scalar):
    return [_P, _C, _C, _I, _I, _I, scalar, _P, _I, _P, _I, scalar, _P, _I]


# name -> (argtypes, restype); names are looked up as "camblas_cuda_" + name unless they start
# with "hip_" (extensions under the camblas_hip_ prefix). Signatures: include/camblas_hip.h.
SIGNATURES = {
    "create": ([_I, _P, ct.POINTER(_P)], _I),
    "destroy": ([_P], _I),
    "error": ([_P], ct.c_char_p),
    "set_algorithm": ([_P, _I], _I),
    "stats": ([_P, ct.POINTER(_U64), _I], _I),
    "reset_stats": ([_P], _I),
    "sgemm": (_gemm(_F), _I),
    "dgemm": (_gemm(_D), _I),
    "bgemm": (_gemm(_F), _I),
    "bgemm_add": ([_P, _C, _C, _I, _I, _I, _F, _P, _I, _P, _I, _F, _P, _I, _P, _I], _I),
    "affine": ([_P, _I, _I, _I, _I, _P, _P, _P, _I, _P], _I),
    "mlp": ([_P, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P], _I),
    "attention": ([_P, _I, _I, _I, _I, _I, _D, _P, _P, _P, _P], _I),
    "mlp_backward": ([_P, _I, _I, _I, _I, _I] + [_P] * 11, _I),
    "silu_multiply": ([_P, _I, _U64, _P, _P, _P], _I),
    "swiglu": ([_P, _I, _U64, _I, _F, _P, _P, _P, _P], _I),
    "rms_norm": ([_P, _I, _I, _I, _F, _P, _P, _P], _I),
    "rms_norm_decode": ([_P, _I, _I, _I, _F, _I, _I, _P, _P, _P], _I),
    "add_rms_norm": ([_P, _I, _I, _F, _P, _P, _P, _P, _P], _I),
    "bfloat16_square": ([_P, _U64, _P, _P], _I),
    "rms_scale": ([_P, _I, _U64, _I, _F, _P, _P, _P, _P], _I),
    "quantized_matmul": ([_P, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P], _I),
    "route_groups": ([_P, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P], _I),
    "reduce_groups": ([_P, _I, _I, _I, _I, _P, _P, _P, _P], _I),
    "grouped_quantized_matmul": ([_P, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P], _I),
    "fp8_decode_supported": ([_P], _I),
    "fp8_decode": ([_P, _I, _I, _P, _P, _P, _P, _I, _I, _I, _P, _SZ, _P], _I),
    "fp8_workspace_size": ([_I, _I, _I], _SZ),
    "fp8_linear": ([_P, _I, _I, _P, _P, _P, _I, _I, _P, _SZ, _P], _I),
    "fp8_block_matmul": ([_P, _I, _I, _I, _P, _P, _P, _P, _P], _I),
    "fp8_quantise_1x128": ([_P, _I, _I, _P, _P, _P], _I),
    "fp8_block_workspace_size": ([_I, _I], _SZ),
    "fp8_block_linear": ([_P, _I, _I, _I, _P, _P, _P, _P, _SZ, _P], _I),
    "add_rms_norm_rows": ([_P, _I, _I, _I, _I, _F, _I, _P, _P, _P, _P, _P], _I),
    "rope": ([_P, _I, _I, _I, _I, _F, _P, _P], _I),
    "kv_append": ([_P, _I, _I, _I, _I, _P, _P, _P, _I, _P, _P], _I),
    "rope_kv_append": ([_P, _I, _I, _I, _I, _I, _F, _P, _P, _I, _P, _P], _I),
    "gqa_decode_attention": ([_P, _I, _I, _I, _I, _I, _P, _F, _P, _I, _P, _P, _P], _I),
    "gqa_decode_attention_noalloc": ([_P, _I, _I, _I, _I, _I, _P, _F, _P, _I, _P, _P, _P], _I),
    "gqa_decode_attention_noalloc_limit": ([], _SZ),
    "bf16_gated_linear": ([_P, _I, _I, _I, _P, _I, _P, _P, _I, _P, _I], _I),
    "rope_append_gqa_decode_attention": ([_P, _I, _I, _I, _I, _I, _P, _F, _F, _P, _I, _P, _P, _P, _P], _I),
    "rope_angles": ([_P, _I, _I, _F, _P, _P], _I),
    "bf16_linear_residual": ([_P, _I, _I, _I, _P, _I, _P, _I, _P, _I, _P, _I, _P, _I, _I, ct.POINTER(_I)], _I),
    "bf16_rms_linear": ([_P, _I, _I, _I, _P, _I, _P, _I, _I, _P, _F, _P, _I, _P, _I], _I),
    "bf16_rms_gated_linear": ([_P, _I, _I, _I, _P, _I, _P, _I, _I, _P, _F, _P, _P, _I, _P, _I], _I),
    "add_residual_squares": ([_P, _I, _I, _P, _P, _P, _P], _I),
    "fp8_moe_decode": ([_P, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _F, _P], _I),
    "hip_plan_describe": ([_I, _I, _C, _C, _I, _I, _I, _I, _I, _I, _I, ct.c_char_p, _SZ], _I),
    "hip_set_plan_override": ([_P, _I, _I], _I),
    "hip_kernel_count": ([_I], _I),
}


def symbol_name(name):
    return "camblas_" + name if name.startswith("hip_") else "camblas_cuda_" + name


def library_path():
    return Path(os.environ.get("CAMBLAS_CUDA_LIBRARY") or DEFAULT_LIBRARY)


@lru_cache(maxsize=1)
def library():
    """Load libcamblas_hip.so once and declare every entry point. Raises when it is missing."""
    path = library_path()
    if not path.is_file():
        raise RuntimeError(
            f"libcamblas_hip.so not found at {path}: build it with `python -m camblas_amd._build`"
        )
    lib = ct.CDLL(str(path))
    for name, (arguments, result) in SIGNATURES.items():
        function = getattr(lib, symbol_name(name))
        function.argtypes = arguments
        function.restype = result
    return lib


@lru_cache(maxsize=1)
def tensor_module():
    """Import the ATen tensor binding that sits beside the core library, or None if not built."""
    core = library_path()
    candidates = sorted(core.parent.glob("_camblas_cuda_torch*.so"))
    if not candidates:
        return None
    # the binding resolves camblas_cuda_* from the already-loaded core (ref: _native.py:57-61)
    ct.CDLL(str(core), mode=ct.RTLD_GLOBAL)
    spec = importlib.util.spec_from_file_location("_camblas_cuda_torch", candidates[0])
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def check(status, handle):
    """Raise RuntimeError with the library's message when a call failed."""
    if status:
        message = library().camblas_cuda_error(handle)
        raise RuntimeError(message.decode() if message else f"camblas status {status}")


_LOCAL = threading.local()
_LIVE = []
_LIVE_LOCK = threading.Lock()


class Context:
    """One native context: one device, one raw HIP stream, one host thread."""

    def __init__(self, device, stream):
        self.pid = os.getpid()
        self.device = device
        self.stream = stream
        self.handle = _P()
        check(library().camblas_cuda_create(device, stream, ct.byref(self.handle)), None)
        self.algorithm = "auto"
        with _LIVE_LOCK:
            _LIVE.append(self)

    def set_algorithm(self, name):
        if name != self.algorithm:
            check(library().camblas_cuda_set_algorithm(self.handle, ALGORITHMS[name]), self.handle)
            self.algorithm = name

    def call(self, name, *arguments):
        """Invoke camblas_cuda_<name>(handle, ...) and raise on a non-zero status."""
        function = getattr(library(), symbol_name(name))
        check(function(self.handle, *arguments), self.handle)


def context(device=None):
    """The calling thread's context for `device` and its current torch stream.

    Creation is refused while that stream is capturing; reuse after fork is refused
    (ref: camblas/_native.py:247-275).
    """
    if device is None:
        device = torch.cuda.current_device()
    elif not isinstance(device, int):
        index = torch.device(device).index
        device = torch.cuda.current_device() if index is None else index
    table = _LOCAL.__dict__.setdefault("contexts", {})
    stream = torch.cuda.current_stream(device).cuda_stream
    native = table.get((device, stream))
    if native is None or not native.handle:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("Warm up CAMBLAS on this stream before graph capture")
        native = table[(device, stream)] = Context(device, stream)
    if native.pid != os.getpid():
        raise RuntimeError("GPU contexts cannot be reused after fork; use spawn")
    native.set_algorithm(getattr(_LOCAL, "algorithm", "auto"))
    return native


def close():
    """Destroy every context created by this process (each waits for its stream)."""
    if tensor_module.cache_info().currsize:
        module = tensor_module()
        if module is not None and hasattr(module, "close"):
            module.close()
    if not library.cache_info().currsize:
        return
    with _LIVE_LOCK:
        for native in _LIVE:
            if native.handle and native.pid == os.getpid():
                library().camblas_cuda_destroy(native.handle)
                native.handle = _P()
        _LIVE.clear()
    if hasattr(_LOCAL, "contexts"):
        _LOCAL.contexts.clear()


atexit.register(close)


def _validate(name):
    if name not in ALGORITHMS:
        raise ValueError(f"Unknown algorithm {name!r}; choose {tuple(ALGORITHMS)}")


def set_algorithm(name):
    """Select the multiplication policy of the calling host thread."""
    _validate(name)
    module = tensor_module()
    if module is not None:
        module.set_default_algorithm(ALGORITHMS[name])
    _LOCAL.algorithm = name


@contextmanager
def algorithm(name):
    """Temporarily select a multiplication policy for the calling host thread."""
    previous = getattr(_LOCAL, "algorithm", "auto")
    set_algorithm(name)
    try:
        yield
    finally:
        set_algorithm(previous)


def stats(device=None, reset=False, all_threads=False):
    """Launch counters of the current device/stream context as a dict (ref: _native.py:360-414)."""
    if device is None:
        device = torch.cuda.current_device()
    elif not isinstance(device, int):
        index = torch.device(device).index
        device = torch.cuda.current_device() if index is None else index
    lib = library()

    def read(native):
        counts = (_U64 * 8)()
        check(lib.camblas_cuda_stats(native.handle, counts, 8), native.handle)
        if reset:
            check(lib.camblas_cuda_reset_stats(native.handle), native.handle)
        return list(counts)

    module = tensor_module()
    totals = dict.fromkeys(COUNTERS, 0)
    if all_threads:
        with _LIVE_LOCK:
            selected = [n for n in _LIVE if n.device == device and n.pid == os.getpid() and n.handle]
    else:
        selected = [context(device)]
    for native in selected:
        for name, count in zip(COUNTERS, read(native)):
            totals[name] += count
    if module is not None:
        extra = (
            module.stats_all(device, reset)
            if all_threads
            else module.stats(device, reset, ALGORITHMS[getattr(_LOCAL, "algorithm", "auto")])
        )
        for name in COUNTERS:
            totals[name] += int(extra.get(name, 0))
    return totals


def plan_describe(dtype, trans_a, trans_b, m, n, k, lda, ldb, ldc, aligned16=True, algorithm="auto"):
    """Planner introspection without a device: returns (kernel id, description)."""
    text = ct.create_string_buffer(128)
    code = library().camblas_hip_plan_describe(
        dtype, ALGORITHMS[algorithm], trans_a.encode(), trans_b.encode(), m, n, k, lda, ldb, ldc,
        int(aligned16), text, 128,
    )
    return code, text.value.decode()
