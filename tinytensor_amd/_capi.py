"""ctypes binding of libttamd.so (the C ABI declared in include/ttamd.h).

There is no CPU fallback: if the HIP library has not been built the import fails with
instructions, and every call that needs a GPU reports the library's own error text.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libttamd.so")

OK, ERR_INVALID_ARGUMENT, ERR_INVALID_DEVICE, ERR_UNSUPPORTED_DTYPE, ERR_OUT_OF_MEMORY, ERR_LAUNCH = range(6)
BOOL, U8, I16, I32, I64, F32, F64 = range(7)
BIN = {"add": 0, "sub": 1, "mul": 2, "div": 3, "pow": 4, "maximum": 5, "minimum": 6, "lt": 7, "le": 8, "gt": 9, "ge": 10,
       "eq": 11, "ne": 12}
POOL = {"max": 0, "min": 1, "avg": 2}
UN = {"relu": 0, "negate": 1, "abs": 2, "sqrt": 3, "exp": 4, "log": 5, "sigmoid": 6, "tanh": 7}


class View3(C.Structure):
    _fields_ = [("data", C.c_void_p), ("offset", C.c_int64), ("stride", C.c_int64 * 3)]


class View4(C.Structure):
    _fields_ = [("data", C.c_void_p), ("offset", C.c_int64), ("stride", C.c_int64 * 4)]


class Epilogue(C.Structure):
    _fields_ = [("bias", C.c_void_p), ("bias_mode", C.c_int32), ("relu", C.c_int32), ("accumulate", C.c_int32),
                ("reserved", C.c_int32), ("relu_out", C.c_void_p), ("relu_grad_input", C.c_void_p), ("colsum_out", C.c_void_p),
                ("rhs_colsum_out", C.c_void_p)]


class Product(C.Structure):
    _fields_ = [("B", C.c_int), ("N", C.c_int), ("K", C.c_int), ("M", C.c_int), ("lhs", C.POINTER(View3)),
                ("rhs", C.POINTER(View3)), ("out", C.c_void_p), ("epilogue", C.POINTER(Epilogue))]


def _bind(lib: C.CDLL) -> None:
    i, vp, sz = C.c_int, C.c_void_p, C.c_size_t
    sig = {
        "ttamd_device_count": (i, [C.POINTER(i)]),
        "ttamd_last_error_string": (C.c_char_p, []),
        "ttamd_target_arch": (C.c_char_p, []),
        "ttamd_malloc": (i, [i, sz, C.POINTER(vp)]),
        "ttamd_free": (i, [i, vp, sz]),
        "ttamd_malloc_on_stream": (i, [i, sz, vp, C.POINTER(vp)]),
        "ttamd_free_on_stream": (i, [i, vp, sz, vp]),
        "ttamd_stream_release": (i, [i, vp]),
        "ttamd_memory_allocated": (i, [i, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
        "ttamd_empty_cache": (i, [i]),
        "ttamd_memory_cached": (i, [i, C.POINTER(C.c_uint64)]),
        "ttamd_memcpy_h2d": (i, [i, vp, vp, sz]),
        "ttamd_memcpy_d2h": (i, [i, vp, vp, sz]),
        "ttamd_memset_zero": (i, [i, vp, sz, vp]),
        "ttamd_device_synchronize": (i, [i]),
        "ttamd_contiguous": (i, [i, i, i, C.POINTER(C.c_int64), C.POINTER(C.c_int64), vp, C.c_int64, vp, vp]),
        "ttamd_binary": (i, [i, i, i, i, C.POINTER(C.c_int64), vp, C.c_int64, C.POINTER(C.c_int64), vp, C.c_int64,
                             C.POINTER(C.c_int64), vp, vp]),
        "ttamd_unary": (i, [i, i, i, i, C.POINTER(C.c_int64), vp, C.c_int64, C.POINTER(C.c_int64), vp, vp]),
        "ttamd_cast": (i, [i, i, i, i, C.POINTER(C.c_int64), vp, C.c_int64, C.POINTER(C.c_int64), vp, vp]),
        "ttamd_assign": (i, [i, i, i, C.POINTER(C.c_int64), vp, C.c_int64, C.POINTER(C.c_int64), vp, C.c_int64,
                             C.POINTER(C.c_int64), vp]),
        "ttamd_where": (i, [i, i, i, C.POINTER(C.c_int64), vp, C.c_int64, C.POINTER(C.c_int64), vp, C.c_int64,
                            C.POINTER(C.c_int64), vp, C.c_int64, C.POINTER(C.c_int64), vp, vp]),
        "ttamd_sum": (i, [i, i, i, C.POINTER(C.c_int64), vp, C.c_int64, C.POINTER(C.c_int64), i, vp, vp]),
        "ttamd_full": (i, [i, i, vp, C.c_int64, vp, vp]),
        "ttamd_random_fill": (i, [i, i, i, C.c_double, C.c_double, C.POINTER(C.c_uint64), C.c_int64, vp, vp]),
        "ttamd_mse_loss": (i, [i, i, C.c_int64, C.c_int64, vp, vp, vp, vp, vp, vp]),
        "ttamd_linear_mse_head": (i, [i, i, C.c_int64, C.c_int64, C.c_int64, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp]),
        "ttamd_random_fill_view": (i, [i, i, i, C.c_double, C.c_double, C.POINTER(C.c_uint64), i, C.POINTER(C.c_int64),
                                       C.POINTER(C.c_int64), vp, C.c_int64, vp]),
        "ttamd_random_fill_states": (i, [i, i, i, C.c_double, C.c_double, C.POINTER(C.c_uint64), i, C.POINTER(C.c_int64),
                                         C.POINTER(C.c_int64), vp, C.c_int64, vp]),
        "ttamd_random_fill_states_params": (i, [i, i, i, vp, C.c_int64, C.POINTER(C.c_int64), vp, C.c_int64, C.POINTER(C.c_int64),
                                                C.POINTER(C.c_uint64), i, C.POINTER(C.c_int64), C.POINTER(C.c_int64), vp,
                                                C.c_int64, vp]),
        "ttamd_batched_matmul": (i, [i, i, i, i, i, i, C.POINTER(View3), C.POINTER(View3), vp, C.POINTER(Epilogue), vp]),
        "ttamd_batched_matmul_pair": (i, [i, i, C.POINTER(Product), C.POINTER(Product), vp]),
        "ttamd_batched_matmul_noalloc": (i, [i, i, i, i, i, i, C.POINTER(View3), C.POINTER(View3), vp, C.POINTER(Epilogue), vp]),
        "ttamd_batched_matmul_variant": (C.c_char_p, [i, i, i, i, i, C.POINTER(View3), C.POINTER(View3)]),
        "ttamd_conv2d_forward": (i, [i, i, C.POINTER(View4), C.POINTER(View4), vp, vp] + [i] * 8 + [vp]),
        "ttamd_conv2d_backward_workspace": (i, [i] + [i] * 8 + [C.POINTER(sz)]),
        "ttamd_conv2d_last_kernel": (i, [i]),
        "ttamd_conv2d_backward": (i, [i, i, vp, C.POINTER(View4), C.POINTER(View4), vp, vp, vp] + [i] * 8 + [vp, sz, vp]),
        "ttamd_pool2d_forward": (i, [i, i, i, C.POINTER(View4), vp] + [i] * 7 + [vp]),
        "ttamd_pool2d_backward": (i, [i, i, i, vp, C.POINTER(View4), vp, vp] + [i] * 7 + [vp]),
        "ttamd_event_create": (i, [i, C.POINTER(vp)]),
        "ttamd_event_destroy": (i, [vp]),
        "ttamd_event_record": (i, [vp, vp]),
        "ttamd_event_elapsed_ms": (i, [vp, vp, C.POINTER(C.c_float)]),
    }
    missing = [name for name in sig if not hasattr(lib, name)]
    if missing:
        raise ImportError(f"{LIB_PATH} lacks {missing}: rebuild it (make -C tinytensor_amd/csrc)")
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args


def load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build the HIP library first "
            "(python -c 'import __graft_entry__ as g; g.build()' or make -C tinytensor_amd/csrc). "
            "tinytensor_amd has no CPU fallback.")
    lib = C.CDLL(LIB_PATH)
    _bind(lib)
    return lib


lib = load()


def last_error() -> str:
    return lib.ttamd_last_error_string().decode()
