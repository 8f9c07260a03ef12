"""What the library does when hipMalloc fails (ref: tests/test_cuda.py:124-226 with its
tests/cuda_fail_alloc.c, and the fallback logic of src/cuda/backend.cu:470-485).

A preloaded interposer (tests/support/fail_next_hipmalloc.c, compiled by the build step or here with cc) makes exactly
one hipMalloc return hipErrorOutOfMemory on demand. It runs in a child process of its own; no
kernel misbehaves, an API call returns an error code. Routes covered:
  * scratch growth of an entry point that cannot do without it (dense attention): status -2, the
    text names the operation, the context stays usable;
  * split-K partials of a BF16 product: the product runs unsplit, counter `guard_fallback`;
  * Strassen scratch under `strassen`: the ordinary kernel, counters guard_fallback + classical;
    under `strassen3`: one level fewer, counters guard_fallback + strassen.
"""

import os
import shutil
import subprocess
import sys
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]

CHILD = r"""
import ctypes as ct
import torch
from camblas_amd import _kernels, _native

injector = ct.CDLL(None)
injector.camblas_test_fail_next_allocation.restype = None
injector.camblas_test_allocation_pending.restype = ct.c_int
device = torch.device("cuda:0")
lib = _native.library()
P = lambda t: ct.c_void_p(t.data_ptr())

# ---- an entry point that needs its scratch: dense attention
native = _native.context(device)
q = torch.randn(64, 32, device=device); k = torch.randn(96, 32, device=device); v = torch.randn(96, 16, device=device)
out = torch.empty(64, 16, device=device)
args = (native.handle, 0, 64, 96, 32, 16, ct.c_double(0.25), P(q), P(k), P(v), P(out))
injector.camblas_test_fail_next_allocation()
status = lib.camblas_cuda_attention(*args)
assert status == -2, status
assert injector.camblas_test_allocation_pending() == 0
assert b"attention scratch failed (status 2)" in lib.camblas_cuda_error(native.handle)
assert lib.camblas_cuda_attention(*args) == 0          # the context is still usable
torch.cuda.synchronize()
want = torch.softmax(0.25 * q.double() @ k.double().t(), -1) @ v.double()
assert ((out.double() - want).norm() / want.norm()).item() <= 1e-5

# ---- split-K partials of a BF16 product: unsplit instead, counted
_native.close()
native = _native.context(device)
x = torch.randn(48, 4096, device=device, dtype=torch.bfloat16)
w = (torch.randn(512, 4096, device=device) / 64).to(torch.bfloat16)
native.call("hip_set_plan_override", 1, 4)              # a register-staged tile variant, four K partitions
native.call("reset_stats")
injector.camblas_test_fail_next_allocation()
y = _kernels.linear(x, w)
torch.cuda.synchronize()
native.call("hip_set_plan_override", -1, 0)
assert injector.camblas_test_allocation_pending() == 0
counts = _native.stats(device)
assert counts["guard_fallback"] == 1 and counts["lt"] == 1, counts
want = x.double() @ w.double().t()
assert ((y.double() - want).norm() / want.norm()).item() <= 1e-2

# ---- Strassen scratch (ref: tests/test_cuda.py:124-196)
for dtype in (torch.float32, torch.float64):
    _native.close()
    a = torch.randn((512, 512), device=device, dtype=dtype) / 512**0.5
    b = torch.randn_like(a) / 512**0.5
    output = torch.empty_like(a)
    with _native.algorithm("classical"):
        _kernels.matmul(a, b, out=output)
    reference = output.clone()
    torch.cuda.synchronize()
    _native.stats(device, reset=True)
    injector.camblas_test_fail_next_allocation()
    with _native.algorithm("strassen"):
        _kernels.matmul(a, b, out=output)
    torch.cuda.synchronize()
    assert injector.camblas_test_allocation_pending() == 0
    counts = _native.stats(device)
    assert counts["guard_fallback"] == 1 and counts["classical"] == 1 and counts["strassen"] == 0, counts
    torch.testing.assert_close(output, reference)
    with _native.algorithm("strassen"):                  # usable afterwards, error state clean
        _kernels.matmul(a, b, out=output)
    torch.testing.assert_close(output, reference, rtol=1e-5, atol=2e-6)
    _native.close()
    with _native.algorithm("classical"):
        _kernels.matmul(a, b, out=output)
    _native.stats(device, reset=True)
    injector.camblas_test_fail_next_allocation()
    with _native.algorithm("strassen3"):
        _kernels.matmul(a, b, out=output)
    torch.cuda.synchronize()
    assert injector.camblas_test_allocation_pending() == 0
    counts = _native.stats(device)
    assert counts["guard_fallback"] == 1 and counts["strassen"] == 1 and counts["classical"] == 0, counts
    torch.testing.assert_close(output, reference, rtol=1e-5, atol=2e-6)
_native.close()
print("allocation failure routes ok")
"""


def test_allocation_failure_routes(tmp_path):
    # the build step leaves the interposer beside its source; without that it is compiled here
    shim = ROOT / "tests/support/fail_next_hipmalloc.so"
    if not shim.is_file():
        compiler = shutil.which("cc") or shutil.which("gcc")
        if not compiler:
            pytest.skip("no C compiler for the interposer")
        shim = tmp_path / "fail_next_hipmalloc.so"
        subprocess.run([compiler, "-shared", "-fPIC", str(ROOT / "tests/support/fail_next_hipmalloc.c"), "-ldl",
                        "-o", str(shim)], check=True, capture_output=True, text=True)
    environment = dict(os.environ)
    # ours goes in front of whatever is preloaded already; nothing is removed
    existing = environment.get("LD_PRELOAD", "")
    environment["LD_PRELOAD"] = str(shim) + (":" + existing if existing else "")
    result = subprocess.run([sys.executable, "-c", CHILD], cwd=ROOT, env=environment, capture_output=True,
                            text=True, timeout=240)
    assert result.returncode == 0 and "allocation failure routes ok" in result.stdout, result.stdout + result.stderr
