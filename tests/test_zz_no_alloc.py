"""The allocation-free decode-attention entry point against the ordinary one.

`camblas_cuda_gqa_decode_attention_noalloc` keeps its split partials in a fixed device array inside
the library instead of context scratch. Both entry points launch the same kernels, so the bar is
bit equality of the BF16 outputs, on two calls in a row that share the array (the second smaller,
so stale partials of the first call lie behind and beside the ones it reads), plus the oracle's
tolerance bar on the first call and a loud refusal beyond the array's size.
"""

import ctypes as ct

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _native
from helpers import bf16_values, from_device_bf16, ptr, rel_frobenius, to_device_bf16

pytestmark = pytest.mark.gpu

Q_HEADS, KV_HEADS, DIM = 16, 4, 128


def attend(native, name, q, k_cache, v_cache, lengths):
    batch, context_length = k_cache.shape[:2]
    out = torch.full((batch, Q_HEADS, DIM), float("nan"), dtype=torch.bfloat16, device=q.device)
    native.call(name, batch, Q_HEADS, KV_HEADS, DIM, context_length, ptr(lengths),
                ct.c_float(DIM**-0.5), ptr(q), q.stride(0), ptr(k_cache), ptr(v_cache), ptr(out))
    torch.cuda.synchronize()
    return out


def case(device, seed, batch, context_length, lengths):
    q = oracle.fill_normal_bf16(seed, (batch, Q_HEADS, DIM))
    k = oracle.fill_normal_bf16(seed + 1, (batch, context_length, KV_HEADS, DIM))
    v = oracle.fill_normal_bf16(seed + 2, (batch, context_length, KV_HEADS, DIM))
    lengths = np.asarray(lengths, np.int32)
    return (q, k, v, lengths), (to_device_bf16(q, device), to_device_bf16(k, device),
                                to_device_bf16(v, device), torch.from_numpy(lengths).to(device))


def test_two_calls_in_a_row_equal_the_allocating_entry_point(device):
    native = _native.context(device)
    host_a, dev_a = case(device, 9100, 6, 1500, [1500, 1, 257, 1024, 700, 1499])
    host_b, dev_b = case(device, 9200, 3, 520, [300, 520, 17])  # fewer sequences, fewer partitions
    for host, dev in ((host_a, dev_a), (host_b, dev_b)):
        resident = attend(native, "gqa_decode_attention_noalloc", *dev)
        allocating = attend(native, "gqa_decode_attention", *dev)
        assert np.array_equal(from_device_bf16(resident), from_device_bf16(allocating))
        want = oracle.gqa_decode(host[0], host[1], host[2], host[3], DIM**-0.5)
        assert rel_frobenius(bf16_values(resident), oracle.bf16_to_f32(want)) <= 1e-2


def test_sizes_beyond_the_fixed_array_are_refused(device):
    native = _native.context(device)
    limit = _native.library().camblas_cuda_gqa_decode_attention_noalloc_limit()
    assert limit == 16 << 20
    # partials: batch * q_heads * ceil(context / 256) * 520 bytes; nothing is read before the refusal
    batch, context_length = 64, 256 * 40
    assert batch * Q_HEADS * 40 * 520 > limit
    q = torch.zeros((batch, Q_HEADS, DIM), dtype=torch.bfloat16, device=device)
    cache = torch.zeros((16,), dtype=torch.bfloat16, device=device)  # never dereferenced
    out = torch.zeros_like(q)
    with pytest.raises(RuntimeError, match="allocation-free entry point holds"):
        native.call("gqa_decode_attention_noalloc", batch, Q_HEADS, KV_HEADS, DIM, context_length,
                    None, ct.c_float(1.0), ptr(q), q.stride(0), ptr(cache), ptr(cache[8:]), ptr(out))
    torch.cuda.synchronize()
    assert not out.any()


CHILD = r"""
import ctypes as ct
import torch
from camblas_amd import _native

injector = ct.CDLL(None)
injector.camblas_test_fail_next_allocation.restype = None
injector.camblas_test_allocation_pending.restype = ct.c_int
device = torch.device("cuda:0")
lib = _native.library()
P = lambda t: ct.c_void_p(t.data_ptr())
Q, KV, D, batch, length = 16, 4, 128, 5, 1300
torch.manual_seed(9300)
q = torch.randn((batch, Q, D), device=device).to(torch.bfloat16)
k = torch.randn((batch, length, KV, D), device=device).to(torch.bfloat16)
v = torch.randn((batch, length, KV, D), device=device).to(torch.bfloat16)
lengths = torch.tensor([1300, 1, 700, 257, 1299], dtype=torch.int32, device=device)
resident = torch.full((batch, Q, D), float("nan"), dtype=torch.bfloat16, device=device)
allocating = torch.full_like(resident, float("nan"))
torch.cuda.synchronize()
native = _native.context(device)                      # a context that has never grown its scratch
def arguments(out):
    return (native.handle, batch, Q, KV, D, length, P(lengths), ct.c_float(D ** -0.5), P(q), q.stride(0),
            P(k), P(v), P(out))
injector.camblas_test_fail_next_allocation()           # any hipMalloc from here on would fail
assert lib.camblas_cuda_gqa_decode_attention_noalloc(*arguments(resident)) == 0
assert injector.camblas_test_allocation_pending() == 1, "the allocation-free entry point allocated"
# the allocating entry point on the same fresh context does ask for memory: it takes the armed failure
assert lib.camblas_cuda_gqa_decode_attention(*arguments(allocating)) == -2
assert injector.camblas_test_allocation_pending() == 0
assert lib.camblas_cuda_gqa_decode_attention(*arguments(allocating)) == 0
torch.cuda.synchronize()
assert torch.equal(resident.view(torch.int16), allocating.view(torch.int16))
assert not torch.isnan(resident.float()).any()
_native.close()
print("no allocation ok")
"""


def test_the_entry_point_allocates_nothing_on_a_fresh_context(tmp_path):
    # A child process with the hipMalloc interposer of the allocation-failure tests preloaded: the
    # call must succeed with a failure armed and leave it armed.
    import os
    import shutil
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    shim = root / "tests/support/fail_next_hipmalloc.so"
    if not shim.is_file():
        compiler = shutil.which("cc") or shutil.which("gcc")
        if not compiler:
            pytest.skip("no C compiler for the interposer")
        shim = tmp_path / "fail_next_hipmalloc.so"
        subprocess.run([compiler, "-shared", "-fPIC", str(root / "tests/support/fail_next_hipmalloc.c"), "-ldl",
                        "-o", str(shim)], check=True, capture_output=True, text=True)
    environment = dict(os.environ)
    existing = environment.get("LD_PRELOAD", "")
    environment["LD_PRELOAD"] = str(shim) + (":" + existing if existing else "")
    result = subprocess.run([sys.executable, "-c", CHILD], cwd=root, env=environment, capture_output=True,
                            text=True, timeout=240)
    assert result.returncode == 0 and "no allocation ok" in result.stdout, result.stdout + result.stderr
