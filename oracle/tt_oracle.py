"""ctypes/numpy front end of the CPU oracle (oracle/tt_oracle.c).

TEST INFRASTRUCTURE ONLY.  Importable from tests/, from __graft_entry__.smoke() and from
bench.py's cpu_baseline leg; never from the tinytensor_amd package.  It restates the
reference's CPU backend for the GEMM path; citations live in tt_oracle.h / tt_oracle.c.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

BOOL, U8, I16, I32, I64, F32, F64 = range(7)
NP_DTYPE = {U8: np.uint8, I16: np.int16, I32: np.int32, I64: np.int64, F32: np.float32, F64: np.float64}
CODE_OF = {np.dtype(v): k for k, v in NP_DTYPE.items()}
SUFFIX = {U8: "u8", I16: "i16", I32: "i32", I64: "i64", F32: "f32", F64: "f64"}


def build() -> None:
    """Compile the three flavours of the oracle in place (gcc only)."""
    subprocess.run(["make", "-C", _HERE, "-B", "all"], check=True, capture_output=True)


def _cpu_has(flag: str) -> bool:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    return flag in line.split()
    except OSError:
        pass
    return False


def _load(flavour: str) -> C.CDLL:
    name = {"fma": "libtt_oracle.so", "fma_v4": "libtt_oracle_v4.so", "nofma": "libtt_oracle_nofma.so"}[flavour]
    path = os.path.join(_HERE, name)
    if not os.path.exists(path):
        build()
    lib = C.CDLL(path)
    vp, ip, i32, i64, u64p = C.c_void_p, C.POINTER(C.c_int), C.c_int, C.c_int64, C.POINTER(C.c_uint64)
    lib.tto_splitmix64.restype = C.c_uint64
    lib.tto_splitmix64.argtypes = [C.c_uint64]
    lib.tto_xorshift64.restype = C.c_uint64
    lib.tto_xorshift64.argtypes = [u64p]
    lib.tto_generator_seed.restype = C.c_uint64
    lib.tto_generator_seed.argtypes = [C.c_uint64]
    lib.tto_uniform_real_f32.argtypes = [u64p, C.c_float, C.c_float, vp, i64]
    lib.tto_uniform_real_f64.argtypes = [u64p, C.c_double, C.c_double, vp, i64]
    lib.tto_normal_f32.argtypes = [u64p, C.c_float, C.c_float, vp, i64]
    lib.tto_normal_f64.argtypes = [u64p, C.c_double, C.c_double, vp, i64]
    lib.tto_uniform_real_view_f32.argtypes = [u64p, C.c_float, C.c_float, vp, i32, ip, ip, i32]
    lib.tto_uniform_real_view_f64.argtypes = [u64p, C.c_double, C.c_double, vp, i32, ip, ip, i32]
    lib.tto_draw_params_f32.argtypes = [u64p, i32, vp, vp, vp, i32, ip, ip, i32]
    lib.tto_draw_params_f64.argtypes = [u64p, i32, vp, vp, vp, i32, ip, ip, i32]
    lib.tto_draw_params_f32.restype = None
    lib.tto_draw_params_f64.restype = None
    for f in ("tto_uniform_real_f32", "tto_uniform_real_f64", "tto_normal_f32", "tto_normal_f64", "tto_uniform_real_view_f32",
              "tto_uniform_real_view_f64"):
        getattr(lib, f).restype = None
    lib.tto_contiguous.restype = None
    lib.tto_contiguous.argtypes = [vp, vp, i32, i32, ip, ip, i32]
    for suf in SUFFIX.values():
        for stem in ("tto_matmul_kernel_", "tto_matmul_blocked_scalar_", "tto_matmul_naive_"):
            fn = getattr(lib, stem + suf)
            fn.restype = None
            fn.argtypes = [vp, vp, vp, i32, i32, i32]
    lib.tto_batched_matmul.restype = i32
    lib.tto_batched_matmul.argtypes = [i32, i32, i32, i32, i32, vp, i32, ip, vp, i32, ip, vp]
    lib.tto_conv2d_forward.restype = i32
    lib.tto_conv2d_forward.argtypes = [i32, vp, vp, vp, vp] + [i32] * 8
    lib.tto_conv2d_backward.restype = i32
    lib.tto_conv2d_backward.argtypes = [i32, vp, vp, vp, vp, vp, vp] + [i32] * 8
    lib.tto_pool2d_forward.restype = i32
    lib.tto_pool2d_forward.argtypes = [i32, i32, vp, vp] + [i32] * 7
    lib.tto_pool2d_backward.restype = i32
    lib.tto_pool2d_backward.argtypes = [i32, i32, vp, vp, vp, vp] + [i32] * 7
    lib.tto_conv2d_naive.restype = i32
    lib.tto_conv2d_naive.argtypes = [i32, vp, vp, vp] + [i32] * 8
    for f in ("tto_unroll_f64", "tto_unroll_transpose_f64", "tto_col2im_f64"):
        getattr(lib, f).restype = None
        getattr(lib, f).argtypes = [vp, vp] + [i32] * 7
    lib.tto_uses_fma.restype = i32
    return lib


_LIBS: dict[str, C.CDLL] = {}


def lib(flavour: str = "fma") -> C.CDLL:
    """flavour: 'fma' (g++ build of the reference), 'nofma' (clang build), 'fast' (fma arithmetic,
    AVX-512VL encodings when the host has them; bit-identical to 'fma')."""
    if flavour == "fast":
        flavour = "fma_v4" if _cpu_has("avx512vl") else "fma"
    if flavour not in _LIBS:
        _LIBS[flavour] = _load(flavour)
    return _LIBS[flavour]


def _ptr(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


def _ints(v) -> "C.Array[C.c_int]":
    return (C.c_int * len(v))(*[int(x) for x in v])


# ----------------------------------------------------------------------------- RNG
class Generator:
    """tinytensor::Generator (tensor/random.cpp:46-63): state = splitmix64(seed), xorshift64 steps."""

    def __init__(self, seed: int = 0):
        self._state = C.c_uint64(lib().tto_generator_seed(seed))

    @property
    def state(self) -> int:
        return self._state.value

    def __call__(self) -> int:
        return lib().tto_xorshift64(C.byref(self._state))

    def uniform_real(self, low: float, high: float, shape, dtype=np.float32) -> np.ndarray:
        out = np.empty(int(np.prod(shape)), dtype=dtype)
        fn = lib().tto_uniform_real_f32 if out.dtype == np.float32 else lib().tto_uniform_real_f64
        fn(C.byref(self._state), low, high, _ptr(out), out.size)
        return out.reshape(shape)

    def uniform_real_(self, view: np.ndarray, low: float, high: float) -> None:
        """Tensor::uniform_real_ on a strided view, in place (cpu/distribution.cpp:96-139): `view` is any numpy view
        with non-negative strides; its elements are drawn in the view's own row-major order."""
        base, offset = view_base(view)
        fn = lib().tto_uniform_real_view_f32 if view.dtype == np.float32 else lib().tto_uniform_real_view_f64
        fn(C.byref(self._state), low, high, _ptr(base), view.ndim, _ints(view.shape), _ints(elem_strides(view)), offset)

    def draw_params_(self, view: np.ndarray, dist: int, p0: np.ndarray, p1: np.ndarray) -> None:
        """uniform_real_ (dist 0) / normal_ (dist 1) with parameter tensors, in place through `view`
        (cpu/distribution.cpp:96-139): p0 / p1 are broadcast to the view's shape and made contiguous, element i of
        the view (row-major rank) reads p0[i], p1[i]."""
        base, offset = view_base(view)
        a = np.ascontiguousarray(np.broadcast_to(p0, view.shape), dtype=view.dtype)
        b = np.ascontiguousarray(np.broadcast_to(p1, view.shape), dtype=view.dtype)
        fn = lib().tto_draw_params_f32 if view.dtype == np.float32 else lib().tto_draw_params_f64
        fn(C.byref(self._state), dist, _ptr(a), _ptr(b), _ptr(base), view.ndim, _ints(view.shape), _ints(elem_strides(view)), offset)

    def normal(self, mu: float, std: float, shape, dtype=np.float32) -> np.ndarray:
        out = np.empty(int(np.prod(shape)), dtype=dtype)
        fn = lib().tto_normal_f32 if out.dtype == np.float32 else lib().tto_normal_f64
        fn(C.byref(self._state), mu, std, _ptr(out), out.size)
        return out.reshape(shape)


# ----------------------------------------------------------------------------- views
def elem_strides(a: np.ndarray) -> list[int]:
    return [s // a.itemsize for s in a.strides]


def view_base(a: np.ndarray) -> tuple[np.ndarray, int]:
    """Underlying storage (1-D owner array) and element offset of a numpy view."""
    base = a
    while isinstance(base.base, np.ndarray):
        base = base.base
    off = (a.ctypes.data - base.ctypes.data) // a.itemsize
    return base, off


def contiguous(a: np.ndarray, flavour: str = "fma") -> np.ndarray:
    base, off = view_base(a)
    out = np.empty(a.shape, dtype=a.dtype)
    lib(flavour).tto_contiguous(_ptr(base), _ptr(out), a.itemsize, a.ndim, _ints(a.shape), _ints(elem_strides(a)), off)
    return out


# ----------------------------------------------------------------------------- GEMM
def _gemm(stem: str, A: np.ndarray, B: np.ndarray, flavour: str) -> np.ndarray:
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    assert A.dtype == B.dtype and A.ndim == 2 and B.ndim == 2 and A.shape[1] == B.shape[0]
    N, K = A.shape
    M = B.shape[1]
    out = np.zeros((N, M), dtype=A.dtype)
    getattr(lib(flavour), stem + SUFFIX[CODE_OF[A.dtype]])(_ptr(A), _ptr(B), _ptr(out), N, K, M)
    return out


def matmul_kernel(A, B, flavour="fma"):
    return _gemm("tto_matmul_kernel_", A, B, flavour)


def matmul_blocked_scalar(A, B, flavour="fma"):
    return _gemm("tto_matmul_blocked_scalar_", A, B, flavour)


def matmul_naive(A, B, flavour="fma"):
    return _gemm("tto_matmul_naive_", A, B, flavour)


def batched_matmul(lhs: np.ndarray, rhs: np.ndarray, flavour: str = "fma") -> np.ndarray:
    """BackendBase::batched_matmul on the CPU device for 3-D (possibly strided) numpy views."""
    assert lhs.ndim == 3 and rhs.ndim == 3 and lhs.dtype == rhs.dtype
    Bn, N, K = lhs.shape
    assert rhs.shape[0] == Bn and rhs.shape[1] == K
    M = rhs.shape[2]
    lb, lo = view_base(lhs)
    rb, ro = view_base(rhs)
    out = np.zeros((Bn, N, M), dtype=lhs.dtype)
    rc = lib(flavour).tto_batched_matmul(
        CODE_OF[lhs.dtype], Bn, N, K, M, _ptr(lb), lo, _ints(elem_strides(lhs)), _ptr(rb), ro,
        _ints(elem_strides(rhs)), _ptr(out))
    if rc != 0:
        raise TypeError("unsupported dtype")
    return out


def matmul(lhs: np.ndarray, rhs: np.ndarray, flavour: str = "fma") -> np.ndarray:
    """tinytensor::matmul rank dispatch (tensor/tensor.cpp:2390-2484) over the CPU backend."""
    if lhs.dtype == np.bool_ and rhs.dtype == np.bool_:
        raise TypeError("matmul does not support boolean tensors")
    if lhs.ndim == 1 and rhs.ndim == 1:
        return batched_matmul(lhs.reshape(1, 1, -1), rhs.reshape(1, -1, 1), flavour).reshape(-1)
    if lhs.ndim == 1 and rhs.ndim == 2:
        return batched_matmul(lhs.reshape(1, 1, -1), rhs[None], flavour).reshape(-1)
    if lhs.ndim == 2 and rhs.ndim == 1:
        return batched_matmul(lhs[None], rhs.reshape(1, -1, 1), flavour).reshape(-1)
    if lhs.ndim == 2 and rhs.ndim == 2:
        return batched_matmul(lhs[None], rhs[None], flavour)[0]
    if lhs.ndim == 3 and rhs.ndim == 3:
        return batched_matmul(lhs, rhs, flavour)
    raise ValueError("Unsupported sizes")


def matmul_backward(lhs: np.ndarray, rhs: np.ndarray, grad: np.ndarray, flavour: str = "fma"):
    """TensorBatchedMatmul::backward (autograd/binary_ops.cpp:173-179): both grads via permuted views."""
    return (matmul(grad, rhs.transpose(0, 2, 1), flavour), matmul(lhs.transpose(0, 2, 1), grad, flavour))


# ----------------------------------------------------------------------------- conv2d
def conv2d_forward(x, w, bias=None, stride=1, padding=0, flavour="fma"):
    x = np.ascontiguousarray(x)
    w = np.ascontiguousarray(w)
    Bn, Cc, H, W = x.shape
    O, _, k, _ = w.shape
    Ho = (H + 2 * padding - k) // stride + 1
    Wo = (W + 2 * padding - k) // stride + 1
    out = np.zeros((Bn, O, Ho, Wo), dtype=x.dtype)
    b = None if bias is None else np.ascontiguousarray(bias)
    rc = lib(flavour).tto_conv2d_forward(CODE_OF[x.dtype], _ptr(x), _ptr(w), None if b is None else _ptr(b),
                                         _ptr(out), Bn, Cc, H, W, O, k, stride, padding)
    assert rc == 0
    return out


def conv2d_backward(gout, x, w, has_bias=False, stride=1, padding=0, flavour="fma"):
    gout = np.ascontiguousarray(gout)
    x = np.ascontiguousarray(x)
    w = np.ascontiguousarray(w)
    Bn, Cc, H, W = x.shape
    O, _, k, _ = w.shape
    gx = np.zeros_like(x)
    gw = np.zeros_like(w)
    gb = np.zeros(O, dtype=x.dtype) if has_bias else None
    rc = lib(flavour).tto_conv2d_backward(CODE_OF[x.dtype], _ptr(gout), _ptr(x), _ptr(w), _ptr(gx), _ptr(gw),
                                          None if gb is None else _ptr(gb), Bn, Cc, H, W, O, k, stride, padding)
    assert rc == 0
    return gx, gw, gb


def conv2d_naive(x, w, stride=1, padding=0, flavour="fma"):
    x = np.ascontiguousarray(x)
    w = np.ascontiguousarray(w)
    Bn, Cc, H, W = x.shape
    O, _, k, _ = w.shape
    Ho = (H + 2 * padding - k) // stride + 1
    Wo = (W + 2 * padding - k) // stride + 1
    out = np.zeros((Bn, O, Ho, Wo), dtype=x.dtype)
    rc = lib(flavour).tto_conv2d_naive(CODE_OF[x.dtype], _ptr(x), _ptr(w), _ptr(out), Bn, Cc, H, W, O, k, stride,
                                       padding)
    assert rc == 0
    return out


# ----------------------------------------------------------------------------- pooling
POOL_OPS = {"max": 0, "min": 1, "avg": 2}


def pool2d_forward(x, op: str, kernel_size: int, stride: int, padding: int):
    """max_pool2d / min_pool2d / avg_pool2d on the CPU device (cpu/conv.cpp:296-349, kernel conv.hpp:121-161).
    avg of an integer input yields float32 (common/reduce.h:63-69)."""
    x = np.ascontiguousarray(x)
    Bn, Cc, H, W = x.shape
    Ho = (H + 2 * padding - kernel_size) // stride + 1
    Wo = (W + 2 * padding - kernel_size) // stride + 1
    rdtype = np.float32 if (op == "avg" and x.dtype.kind != "f") else x.dtype
    out = np.zeros((Bn, Cc, Ho, Wo), dtype=rdtype)
    rc = lib().tto_pool2d_forward(CODE_OF[x.dtype], POOL_OPS[op], _ptr(x), _ptr(out), Bn, Cc, H, W, kernel_size, stride,
                                  padding)
    assert rc == 0
    return out


def pool2d_backward(gout, x, result, op: str, kernel_size: int, stride: int, padding: int):
    """*_pool2d_backward (cpu/conv.cpp:351-426, kernels conv.hpp:171-275); float dtypes."""
    x = np.ascontiguousarray(x)
    gout = np.ascontiguousarray(gout, dtype=x.dtype)
    result = np.ascontiguousarray(result, dtype=x.dtype)
    Bn, Cc, H, W = x.shape
    gx = np.zeros_like(x)
    rc = lib().tto_pool2d_backward(CODE_OF[x.dtype], POOL_OPS[op], _ptr(gout), _ptr(x), _ptr(result), _ptr(gx), Bn, Cc, H,
                                   W, kernel_size, stride, padding)
    assert rc == 0
    return gx


# ----------------------------------------------------------------------------- nn::Linear / MLP step
def linear_init(gen: Generator, in_features: int, out_features: int, dtype=np.float32):
    """nn::Linear default init (nn/linear.cpp:20-40, nn/init.cpp:30-52,106-112): weight [in,out]
    ~ U(+-sqrt(3)/sqrt(fan)), bias ~ U(+-1/sqrt(fan)), fan = weight.size(0) = in_features."""
    fan = float(in_features)
    bound_w = np.sqrt(3.0) * (1.0 / np.sqrt(fan))
    W = gen.uniform_real(-bound_w, bound_w, (in_features, out_features), dtype)
    bound_b = 1.0 / np.sqrt(fan)
    b = gen.uniform_real(-bound_b, bound_b, (out_features,), dtype)
    return W, b


def conv2d_init(gen: Generator, in_channels: int, out_channels: int, kernel_size: int, bias: bool = True, dtype=np.float32):
    """nn::Conv2d default init (nn/conv2d.cpp:20-66): weight [O,C,k,k] drawn IN PLACE through the view
    weight.permute(1,0,2,3) by kaiming_uniform_ (fan = view.size(0)*k*k = C*k*k, nn/init.cpp:30-52,106-112), then bias
    ~ U(+-1/sqrt(fan)) with fan = calc_fan_in_out(weight) = O*k*k."""
    k = kernel_size
    W = np.zeros((out_channels, in_channels, k, k), dtype=dtype)
    bound_w = np.sqrt(3.0) * (1.0 / np.sqrt(float(in_channels * k * k)))
    gen.uniform_real_(W.transpose(1, 0, 2, 3), -bound_w, bound_w)
    b = None
    if bias:
        bound_b = 1.0 / np.sqrt(float(out_channels * k * k))
        b = gen.uniform_real(-bound_b, bound_b, (out_channels,), dtype)
    return W, b
