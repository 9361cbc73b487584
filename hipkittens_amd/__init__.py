"""hipkittens_amd — MI355X (gfx950) quantized-contraction kernels behind a C ABI.

`tk_kernel` mirrors the reference's per-kernel pybind module convention
(`tk_kernel.dispatch_*(inputs..., outputs...)`, in-place, asynchronous);
`quant` prepares quantized operands on the tensors' own device.
"""
from . import quant, tk_kernel  # noqa: F401
from ._lib import lib_path, load_library  # noqa: F401

__all__ = ["tk_kernel", "quant", "load_library", "lib_path"]
