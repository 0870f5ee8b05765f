"""tinytensor_amd — MI355X (gfx950) GEMM backend for tinytensor: Python mirror of the host interface.

The product is libttamd.so (HIP kernels behind the C ABI of include/ttamd.h).  This package is the
thin host-side mirror of tinytensor's Tensor/backend interface for the GEMM path, used by the parity
tests and the benchmark: same names, argument meaning and error behaviour as the reference's C++ API.
"""
from .tensor import (  # noqa: F401
    BackendAMD, Conv2d, Device, Generator, Linear, Tensor, TTException, calc_fan_in_out, default_generator, kaiming_uniform_,
    set_default_generator_seed, broadcast_tensors, linear_backward, linear_init, linear_relu, linear_mse_head, mse_loss, normal, uniform_real, conv2d, conv2d_backward, full, get_backend, kAMD, linear,
    matmul, matmul_backward, where, max_pool2d, min_pool2d, avg_pool2d, pool2d_backward,
)
from . import _capi  # noqa: F401
from . import graph  # noqa: F401  (HIP streams and graphs; loads the HIP runtime on first use)
