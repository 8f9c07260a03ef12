"""camblas_amd: MI355X (gfx950) backend for the CAMBLAS GPU linear path.

Importing the package touches neither the GPU nor the native library. `_autoload` is the
torch.backends entry point: it registers the native mm/addmm kernels when CAMBLAS_ENABLE=1
(ref: camblas/__init__.py:6-29).
"""

import os

__all__ = ["_autoload"]


def _autoload():
    """Register the HIP kernels behind torch.mm/addmm/matmul/F.linear when the process opts in."""
    if os.environ.get("CAMBLAS_ENABLE", "0") != "1":
        return
    from ._native import ALGORITHMS, tensor_module

    module = tensor_module()
    if module is None or not hasattr(module, "install_torch_backend"):
        raise RuntimeError(
            "Build the tensor binding with `python camblas_amd/_build.py` first"
        )
    name = os.environ.get(
        "CAMBLAS_CUDA_ALGORITHM", os.environ.get("CAMBLAS_SGLANG_ALGORITHM", "lt")
    )
    if name not in ALGORITHMS:
        raise ValueError(f"Unknown CAMBLAS CUDA algorithm: {name}")
    module.install_torch_backend(ALGORITHMS[name])
