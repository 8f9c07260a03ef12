"""camblas_amd: MI355X (gfx950) backend for the CAMBLAS GPU linear path.

Importing the package touches neither the GPU nor the native library. PyTorch discovers
`_autoload` through the `torch.backends` entry-point group and calls it once its own import is
complete; the function does nothing unless the process has opted in
(ref: camblas/__init__.py:6-29 for the environment contract).

    CAMBLAS_ENABLE=1            route torch.mm / addmm / matmul / F.linear to the HIP kernels
    CAMBLAS_CUDA_ALGORITHM      GEMM policy name; falls back to CAMBLAS_SGLANG_ALGORITHM, then "lt"
"""

import os

__all__ = ["_autoload"]

_POLICY_VARIABLES = ("CAMBLAS_CUDA_ALGORITHM", "CAMBLAS_SGLANG_ALGORITHM")


def _requested_policy(environment):
    for variable in _POLICY_VARIABLES:
        if variable in environment:
            return environment[variable]
    return "lt"


def _autoload():
    """Entry point of the `torch.backends` group: install the dispatcher overrides when enabled."""
    environment = os.environ
    if environment.get("CAMBLAS_ENABLE", "0") != "1":
        return  # nothing is loaded, no device is touched

    from . import _native

    # (a missing binding is reported before an unknown policy name, as in the reference)
    installer = getattr(_native.tensor_module(), "install_torch_backend", None)
    if installer is None:
        raise RuntimeError("Build the tensor binding with `python camblas_amd/_build.py` first")
    policy = _requested_policy(environment)
    if policy not in _native.ALGORITHMS:
        raise ValueError(f"Unknown CAMBLAS CUDA algorithm: {policy}")
    installer(_native.ALGORITHMS[policy])
