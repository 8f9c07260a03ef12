"""PyTorch's own plugin discovery, end to end, in fresh processes.

`import torch` walks the `torch.backends` entry-point group and calls what it finds
(torch/__init__.py `_import_device_backends`; the reference registers `camblas = camblas:_autoload`,
/root/reference pyproject.toml:12-16 and camblas/__init__.py:6-29). This package registers
`camblas = camblas_amd:_autoload` through `pyproject.toml` and, for boxes where nothing can be
installed, through the hand-written `camblas_amd-0.2.0.dist-info/` at the repository root, which
importlib.metadata finds on the module search path.

The child processes below contain nothing but ordinary PyTorch code. With CAMBLAS_ENABLE=1 a BF16
`F.linear`, a `torch.mm` and a `torch.addmm` must be counted by the library's contexts and agree
with an FP64 product; without it the library must not even be mapped into the process.
"""

import json
import os
import subprocess
import sys
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]

CHILD = r"""
import json, torch
import torch.nn.functional as F

def mapped():
    return any("libcamblas_hip.so" in line for line in open("/proc/self/maps"))

report = {"mapped_after_import_torch": mapped()}
torch.manual_seed(3)
device = torch.device("cuda:0")
x = torch.randn(24, 512, device=device, dtype=torch.bfloat16)
w = torch.randn(384, 512, device=device, dtype=torch.bfloat16) / 16
bias = torch.randn(384, device=device, dtype=torch.bfloat16)
y = F.linear(x, w)
z = torch.mm(x.float(), w.float().t())
u = torch.addmm(bias, x, w.t())
torch.cuda.synchronize()
want = x.double() @ w.double().t()
report["linear_error"] = ((y.double() - want).norm() / want.norm()).item()
report["mm_error"] = ((z.double() - want).norm() / want.norm()).item()
report["addmm_error"] = ((u.double() - (want + bias.double())).norm() / want.norm()).item()
report["mapped_after_products"] = mapped()
if report["mapped_after_products"]:
    from camblas_amd import _native
    report["launches"] = sum(_native.tensor_module().stats_all(0, False).values())
else:
    report["launches"] = 0
print("REPORT " + json.dumps(report))
"""


def run_child(enable):
    environment = {key: value for key, value in os.environ.items() if not key.startswith("CAMBLAS_")}
    environment.pop("TORCH_DEVICE_BACKEND_AUTOLOAD", None)
    if enable:
        environment["CAMBLAS_ENABLE"] = "1"
    # the repository root is the child's working directory, so it is on the module search path of
    # `python -c` and the dist-info beside the package is what importlib.metadata sees
    result = subprocess.run([sys.executable, "-c", CHILD], cwd=ROOT, env=environment, capture_output=True,
                            text=True, timeout=240)
    assert result.returncode == 0, result.stdout + result.stderr
    line = [text for text in result.stdout.splitlines() if text.startswith("REPORT ")][-1]
    return json.loads(line[len("REPORT "):])


def test_enabled_process_runs_plain_torch_code_in_the_library():
    report = run_child(enable=True)
    assert report["mapped_after_import_torch"], "import torch did not load the backend"
    assert report["launches"] >= 3, report
    assert report["linear_error"] <= 1e-2 and report["addmm_error"] <= 1e-2 and report["mm_error"] <= 1e-5


def test_disabled_process_never_touches_the_library():
    report = run_child(enable=False)
    assert not report["mapped_after_import_torch"] and not report["mapped_after_products"]
    assert report["launches"] == 0
    assert report["linear_error"] <= 1e-2
