"""Host-side mirror of tinytensor's Tensor / BackendBase interface for the GEMM path.

Only what the hot path needs: strided views over device storage (shape, stride, offset in
elements, exactly what tinytensor::Tensor carries, include/tt/tensor.h:245-255), the `matmul`
frontend (tinytensor/tensor/tensor.cpp:2390-2484), the autograd call pattern of the backward GEMMs
(tinytensor/autograd/binary_ops.cpp:165-179), nn::Linear's forward (tinytensor/nn/linear.cpp:42-50),
conv2d / conv2d_backward (tinytensor/tensor/backend_base.h:269-284) and the storage interop
(from_vec / to_vec, backend_base.h:35-60).  All arithmetic happens in libttamd.so; nothing here
computes on the host.
"""
from __future__ import annotations

import contextlib
import ctypes as C
import math
from dataclasses import dataclass

import numpy as np

from . import _capi
from ._capi import lib

_NP_OF = {_capi.BOOL: np.bool_, _capi.U8: np.uint8, _capi.I16: np.int16, _capi.I32: np.int32, _capi.I64: np.int64,
          _capi.F32: np.float32, _capi.F64: np.float64}
_CODE_OF = {np.dtype(v): k for k, v in _NP_OF.items()}
# promotion follows the ScalarType order bool < u8 < i16 < i32 < i64 < f32 < f64 (include/tt/scalar.h:21-29)


class TTException(Exception):
    """tinytensor::TTException (include/tt/exception.h:15-25)."""


@dataclass(frozen=True)
class Device:
    backend: str
    id: int = 0

    def __str__(self) -> str:
        return f"{self.backend}:{self.id}"


kAMD = Device("amd", 0)


def _check(status: int) -> None:
    """Status -> exception mapping documented in include/ttamd.h."""
    if status == _capi.OK:
        return
    msg = _capi.last_error()
    if status == _capi.ERR_LAUNCH:
        # The reference prints and exits (TT_ERROR, include/tt/exception.h:28-36); a Python host raises.
        raise RuntimeError(f"unrecoverable device error: {msg}")
    raise TTException(msg)


_PINNED = None  # while a HIP graph is being captured: the list that keeps every storage allocated meanwhile alive


class _Storage:
    """Owning device allocation (peer of DeviceMemory<T>, cuda/data_types.cuh:28-101).  The block is requested for the
    stream that launches go to at that moment and returned for the one current at its release, so that the library's
    block cache never hands it to another stream while kernels of those two may still use it."""

    def __init__(self, nbytes: int, device: Device):
        self.nbytes = int(nbytes)
        self.device = device
        p = C.c_void_p()
        _check(lib.ttamd_malloc_on_stream(device.id, self.nbytes, _stream_arg(), C.byref(p)))
        self.ptr = p.value or 0
        if _PINNED is not None:
            _PINNED.append(self)

    def __del__(self):
        if getattr(self, "ptr", 0):
            lib.ttamd_free_on_stream(self.device.id, C.c_void_p(self.ptr), self.nbytes, _stream_arg())
            self.ptr = 0


def _dense_strides(shape) -> tuple:
    st, acc = [], 1
    for s in reversed(shape):
        st.append(acc)
        acc *= s
    return tuple(reversed(st))


class Tensor:
    """Strided view over device storage."""

    def __init__(self, storage: _Storage, dtype: int, shape, stride=None, offset: int = 0):
        self.storage = storage
        self.dtype = dtype
        self.shape = tuple(int(s) for s in shape)
        self.stride = tuple(int(s) for s in (stride if stride is not None else _dense_strides(self.shape)))
        self.offset = int(offset)

    # ---- construction / readback -------------------------------------------------------------
    @staticmethod
    def from_numpy(a: np.ndarray, device: Device = kAMD) -> "Tensor":
        """Tensor(std::vector<T>, shape, device) -> BackendBase::from_vec (backend_base.h:35-48)."""
        a = np.ascontiguousarray(a)
        if a.dtype not in _CODE_OF:
            raise TTException(f"unsupported dtype {a.dtype}")
        st = _Storage(max(a.nbytes, 1), device)
        if a.nbytes:
            _check(lib.ttamd_memcpy_h2d(device.id, C.c_void_p(st.ptr), C.c_void_p(a.ctypes.data), a.nbytes))
        return Tensor(st, _CODE_OF[a.dtype], a.shape)

    @staticmethod
    def empty(shape, dtype: int, device: Device = kAMD) -> "Tensor":
        n = int(np.prod(shape)) if len(shape) else 1
        st = _Storage(max(n * np.dtype(_NP_OF[dtype]).itemsize, 1), device)
        return Tensor(st, dtype, shape)

    def storage_to_numpy(self) -> np.ndarray:
        """BackendBase::to_vec: the WHOLE storage as a flat host array (backend_base.h:55-60)."""
        npdt = np.dtype(_NP_OF[self.dtype])
        out = np.empty(self.storage.nbytes // npdt.itemsize, dtype=npdt)
        if out.nbytes:
            _check(lib.ttamd_memcpy_d2h(self.device.id, C.c_void_p(out.ctypes.data), C.c_void_p(self.storage.ptr),
                                        out.nbytes))
        return out

    def to_numpy(self) -> np.ndarray:
        """Host copy of this view (Tensor::to_vec applies the view after the download)."""
        flat = self.storage_to_numpy()
        isz = flat.itemsize
        v = np.lib.stride_tricks.as_strided(flat[self.offset:], shape=self.shape,
                                            strides=tuple(s * isz for s in self.stride), writeable=False)
        return np.array(v)

    # ---- properties ----------------------------------------------------------------------------
    @property
    def device(self) -> Device:
        return self.storage.device

    def dim(self) -> int:
        return len(self.shape)

    def size(self, i: int) -> int:
        return self.shape[i]

    def numel(self) -> int:
        return int(np.prod(self.shape)) if self.shape else 1

    def is_contiguous(self) -> bool:
        return self.stride == _dense_strides(self.shape)

    @property
    def itemsize(self) -> int:
        return np.dtype(_NP_OF[self.dtype]).itemsize

    # ---- views (tinytensor/autograd/shape_ops.cpp:24-146: only shape/stride/offset change) -------
    def permute(self, *dims) -> "Tensor":
        if len(dims) == 1 and isinstance(dims[0], (tuple, list)):
            dims = tuple(dims[0])
        if sorted(dims) != list(range(self.dim())):
            raise TTException(f"Invalid permutation {dims} for {self.dim()} dimensions")
        return Tensor(self.storage, self.dtype, [self.shape[d] for d in dims], [self.stride[d] for d in dims],
                      self.offset)

    def unsqueeze(self, dim: int) -> "Tensor":
        if dim < 0:
            dim += self.dim() + 1
        shape = list(self.shape)
        stride = list(self.stride)
        shape.insert(dim, 1)
        stride.insert(dim, 0)  # a size-1 dimension is never stepped over; no copy is needed
        return Tensor(self.storage, self.dtype, shape, stride, self.offset)

    def squeeze(self, dim: int) -> "Tensor":
        if self.shape[dim] != 1:
            return self
        shape = list(self.shape)
        stride = list(self.stride)
        del shape[dim], stride[dim]
        return Tensor(self.storage, self.dtype, shape, stride, self.offset)

    def expand(self, shape) -> "Tensor":
        shape = tuple(shape)
        if len(shape) != self.dim():
            raise TTException("expand: rank mismatch")
        stride = []
        for have, want, st in zip(self.shape, shape, self.stride):
            if have == want:
                stride.append(st)
            elif have == 1:
                stride.append(0)
            else:
                raise TTException(f"expand: cannot expand {self.shape} to {shape}")
        return Tensor(self.storage, self.dtype, shape, stride, self.offset)

    def contiguous(self) -> "Tensor":
        """Tensor::contiguous (tensor.cpp:583-591): self if dense, else the identity op into new storage."""
        return self if self.is_contiguous() else get_backend(self.device).identity(self)

    def reshape(self, shape) -> "Tensor":
        """Tensor::reshape (tensor.cpp:1371-1387): a view when dense, a clone otherwise."""
        shape = list(shape)
        if shape.count(-1) == 1:
            known = int(np.prod([s for s in shape if s != -1]))
            shape[shape.index(-1)] = self.numel() // max(known, 1)
        if int(np.prod(shape)) != self.numel():
            raise TTException(f"reshape: {self.shape} cannot be viewed as {tuple(shape)}")
        base = self.contiguous()
        return Tensor(base.storage, base.dtype, shape, None, base.offset)

    def flatten(self, start: int = 0, end: int = -1) -> "Tensor":
        n = self.dim()
        if n == 0:
            return self.reshape([1])
        start %= n
        end %= n
        merged = int(np.prod(self.shape[start:end + 1]))
        return self.reshape(list(self.shape[:start]) + [merged] + list(self.shape[end + 1:]))

    # ---- elementwise ops around the GEMMs (frontend broadcasting, then one backend call) ----------
    def _binary(self, other, op: str) -> "Tensor":
        if not isinstance(other, Tensor):
            other = _constant(self.shape, other, self.dtype, self.device)
        if other.dtype != self.dtype:  # operands are cast to promote_types(lhs, rhs) (tensor/tensor.cpp:2272-2274)
            dt = max(self.dtype, other.dtype)
            a, b = broadcast_tensors(self.to(dt), other.to(dt))
        else:
            a, b = broadcast_tensors(self, other)
        return get_backend(self.device).binary(a, b, op)

    def __add__(self, o): return self._binary(o, "add")
    def __sub__(self, o): return self._binary(o, "sub")
    def __mul__(self, o): return self._binary(o, "mul")
    def __truediv__(self, o): return self._binary(o, "div")
    def __lt__(self, o): return self._binary(o, "lt")
    def __gt__(self, o): return self._binary(o, "gt")
    def __rmul__(self, o): return self._binary(o, "mul")
    def pow(self, o): return self._binary(o, "pow")
    def relu(self): return get_backend(self.device).unary(self, "relu")

    def to(self, dtype: int) -> "Tensor":
        """Tensor::to(ScalarType) (tensor/tensor.cpp:534-540): the tensor itself when the dtype already matches."""
        return self if dtype == self.dtype else get_backend(self.device).to(self, dtype)

    def assign(self, rhs: "Tensor") -> "Tensor":
        get_backend(self.device).assign(self, rhs)
        return self
    def sum(self, dim: int | None = None): return get_backend(self.device).sum(self, dim)

    def mean(self):
        """Tensor::mean(): sum() / numel (tinytensor/tensor/tensor.cpp mean -> sum, then div by N)."""
        return self.sum() / float(self.numel())

    def item(self):
        return self.to_numpy().reshape(-1)[0]

    def uniform_real_(self, low, high, gen: "Generator") -> "Tensor":
        """Tensor::uniform_real_(low, high, gen) (tensor/tensor.cpp:1783-1801) -> BackendBase::uniform_real_: in place,
        through this tensor's view (element i of the view takes the i-th draw, cpu/kernel/distribution.hpp:28-32).
        `low` / `high` are two numbers, or two tensors of this tensor's shape and dtype (a pair per element)."""
        if self.dtype not in (_capi.F32, _capi.F64):
            raise TTException("uniform_real_ expects a floating point tensor")
        if isinstance(low, Tensor) or isinstance(high, Tensor):
            get_backend(self.device).random_fill_params_(self, 0, low, high, gen)
            return self
        if not low < high:
            raise TTException("Expected low < high. At least one element violates this.")
        get_backend(self.device).random_fill_(self, 0, low, high, gen)
        return self

    def normal_(self, mu, std, gen: "Generator") -> "Tensor":
        """Tensor::normal_(mu, std, gen) -> BackendBase::normal_, in place through this tensor's view; the parameters
        are two numbers or two tensors of this tensor's shape and dtype."""
        if self.dtype not in (_capi.F32, _capi.F64):
            raise TTException("normal_ expects a floating point tensor")
        if isinstance(mu, Tensor) or isinstance(std, Tensor):
            get_backend(self.device).random_fill_params_(self, 1, mu, std, gen)
            return self
        get_backend(self.device).random_fill_(self, 1, mu, std, gen)
        return self

    def view3(self) -> _capi.View3:
        v = _capi.View3()
        v.data = self.storage.ptr
        v.offset = self.offset
        for i in range(3):
            v.stride[i] = self.stride[i]
        return v

    def view4(self) -> _capi.View4:
        v = _capi.View4()
        v.data = self.storage.ptr
        v.offset = self.offset
        for i in range(4):
            v.stride[i] = self.stride[i]
        return v


# -------------------------------------------------------------------------------------------------
_STREAM = None  # hipStream_t (an integer handle) that every launch of this module goes to; None = default stream


def _stream_arg():
    return C.c_void_p(_STREAM) if _STREAM else None


@contextlib.contextmanager
def pin_allocations(keep: list):
    """Every storage allocated inside the block is appended to `keep`, which the caller holds for as long as the
    addresses must stay the allocation's own (a captured HIP graph replays with the addresses it was recorded with:
    a temporary that went back to the block cache could be handed to an unrelated tensor and overwritten by a replay)."""
    global _PINNED
    prev, _PINNED = _PINNED, keep
    try:
        yield keep
    finally:
        _PINNED = prev


class BackendAMD:
    """The methods of tinytensor::BackendBase (tensor/backend_base.h:23-322) that the GEMM path uses."""

    @contextlib.contextmanager
    def on_stream(self, stream: int | None):
        """Sends every kernel launched inside the block to `stream` (a hipStream_t handle, e.g. one under HIP graph
        capture).  No counterpart in the reference, whose CUDA backend always uses the default stream
        (cuda/kernel_launch.cuh:19-29); host copies (to_numpy, from_numpy) stay blocking default-stream copies."""
        global _STREAM
        prev, _STREAM = _STREAM, stream
        try:
            yield
        finally:
            _STREAM = prev

    def get_device_count(self) -> int:
        n = C.c_int()
        _check(lib.ttamd_device_count(C.byref(n)))
        return n.value

    def current_memory_allocated(self, device_id: int) -> int:
        cur, tot = C.c_uint64(), C.c_uint64()
        _check(lib.ttamd_memory_allocated(device_id, C.byref(cur), C.byref(tot)))
        return cur.value

    def total_memory_allocated(self, device_id: int) -> int:
        cur, tot = C.c_uint64(), C.c_uint64()
        _check(lib.ttamd_memory_allocated(device_id, C.byref(cur), C.byref(tot)))
        return tot.value

    def synchronize(self, device_id: int = 0) -> None:
        _check(lib.ttamd_device_synchronize(device_id))

    def identity(self, t: Tensor) -> Tensor:
        """BackendBase::identity on a view = clone into dense storage (cpu/unary.cpp:26-58)."""
        out = Tensor.empty(t.shape, t.dtype, t.device)
        nd = t.dim()
        shape = (C.c_int64 * max(nd, 1))(*t.shape)
        stride = (C.c_int64 * max(nd, 1))(*t.stride)
        _check(lib.ttamd_contiguous(t.device.id, t.dtype, nd, shape, stride, C.c_void_p(t.storage.ptr), t.offset,
                                    C.c_void_p(out.storage.ptr), _stream_arg()))
        return out

    @staticmethod
    def _i64(vals):
        return (C.c_int64 * max(len(vals), 1))(*vals)

    def binary(self, lhs: Tensor, rhs: Tensor, op: str) -> Tensor:
        """BackendBase::add/sub/mul/div/pow/maximum/minimum and the comparisons (backend_base.h:109-131)."""
        if lhs.shape != rhs.shape or lhs.dtype != rhs.dtype:
            raise TTException(f"binary op {op}: operands must share shape and dtype")
        code = _capi.BIN[op]
        out = Tensor.empty(lhs.shape, _capi.BOOL if code >= _capi.BIN["lt"] else lhs.dtype, lhs.device)
        _check(lib.ttamd_binary(lhs.device.id, lhs.dtype, code, lhs.dim(), self._i64(lhs.shape), C.c_void_p(lhs.storage.ptr),
                                lhs.offset, self._i64(lhs.stride), C.c_void_p(rhs.storage.ptr), rhs.offset,
                                self._i64(rhs.stride), C.c_void_p(out.storage.ptr), _stream_arg()))
        return out

    def unary(self, t: Tensor, op: str) -> Tensor:
        """BackendBase::relu / negate / abs / sqrt / exp / log / sigmoid / tanh (backend_base.h:136-260)."""
        out = Tensor.empty(t.shape, t.dtype, t.device)
        _check(lib.ttamd_unary(t.device.id, t.dtype, _capi.UN[op], t.dim(), self._i64(t.shape), C.c_void_p(t.storage.ptr),
                               t.offset, self._i64(t.stride), C.c_void_p(out.storage.ptr), _stream_arg()))
        return out

    def where(self, cond: Tensor, lhs: Tensor, rhs: Tensor) -> Tensor:
        """BackendBase::where (backend_base.h:263)."""
        if cond.dtype != _capi.BOOL or cond.shape != lhs.shape or lhs.shape != rhs.shape or lhs.dtype != rhs.dtype:
            raise TTException("where: cond must be bool and all operands must share one shape")
        out = Tensor.empty(lhs.shape, lhs.dtype, lhs.device)
        _check(lib.ttamd_where(lhs.device.id, lhs.dtype, lhs.dim(), self._i64(lhs.shape), C.c_void_p(cond.storage.ptr),
                               cond.offset, self._i64(cond.stride), C.c_void_p(lhs.storage.ptr), lhs.offset,
                               self._i64(lhs.stride), C.c_void_p(rhs.storage.ptr), rhs.offset, self._i64(rhs.stride),
                               C.c_void_p(out.storage.ptr), _stream_arg()))
        return out

    def sum(self, t: Tensor, dim: int | None = None) -> Tensor:
        """BackendBase::sum(tensor) / sum(tensor, dim) (backend_base.h:148-149).  bool and integer tensors are summed
        in 64 bits into an I64 result (common/reduce.h:56-61)."""
        rdtype = t.dtype if t.dtype in (_capi.F32, _capi.F64) else _capi.I64
        if dim is None:
            out = Tensor.empty((1,), rdtype, t.device)
            d = -1
        else:
            d = dim % t.dim()
            out = Tensor.empty(t.shape[:d] + t.shape[d + 1:], rdtype, t.device)
        _check(lib.ttamd_sum(t.device.id, t.dtype, t.dim(), self._i64(t.shape), C.c_void_p(t.storage.ptr), t.offset,
                             self._i64(t.stride), d, C.c_void_p(out.storage.ptr), _stream_arg()))
        return out

    def full(self, value, numel: int, dtype: int, device: Device) -> Tensor:
        """BackendBase::full (backend_base.h:51)."""
        out = Tensor.empty((numel,), dtype, device)
        host = np.array([value], dtype=_NP_OF[dtype])
        _check(lib.ttamd_full(device.id, dtype, C.c_void_p(host.ctypes.data), numel, C.c_void_p(out.storage.ptr), _stream_arg()))
        return out

    def random_fill_(self, t: Tensor, dist: int, p0: float, p1: float, gen: "Generator") -> None:
        """BackendBase::uniform_real_ / normal_ (backend_base.h:96-103) with scalar parameters, written through the
        view `t` in place; `gen` advances by t.numel() outputs."""
        _check(lib.ttamd_random_fill_view(t.device.id, t.dtype, dist, p0, p1, C.byref(gen.state), t.dim(), self._i64(t.shape),
                                          self._i64(t.stride), C.c_void_p(t.storage.ptr), t.offset, _stream_arg()))

    def random_fill_params_(self, t: Tensor, dist: int, a: Tensor, b: Tensor, gen: "Generator") -> None:
        """BackendBase::uniform_real_ / normal_ (backend_base.h:96-103) with parameter tensors: element i of `t` reads
        its pair at rank i of `a` and `b` (views over t's shape).  The states are drawn here, one per element, as
        create_gen_states does (cpu/distribution.cpp:31-38)."""
        if not (isinstance(a, Tensor) and isinstance(b, Tensor)) or a.shape != t.shape or b.shape != t.shape \
                or a.dtype != t.dtype or b.dtype != t.dtype:
            raise TTException("distribution parameters must be tensors of the result's shape and dtype")
        n = t.numel()
        states = (C.c_uint64 * max(n, 1))()
        x, m = gen.state.value, (1 << 64) - 1
        for i in range(n):
            x ^= (x << 13) & m
            x ^= x >> 7
            x ^= (x << 17) & m
            states[i] = x
        _check(lib.ttamd_random_fill_states_params(
            t.device.id, t.dtype, dist, C.c_void_p(a.storage.ptr), a.offset, self._i64(a.stride), C.c_void_p(b.storage.ptr),
            b.offset, self._i64(b.stride), states, t.dim(), self._i64(t.shape), self._i64(t.stride), C.c_void_p(t.storage.ptr),
            t.offset, _stream_arg()))
        gen.state = C.c_uint64(x)

    def to(self, t: Tensor, dtype: int) -> Tensor:
        """BackendBase::to(tensor, dtype) (backend_base.h:74): element-wise static_cast into dense storage."""
        out = Tensor.empty(t.shape, dtype, t.device)
        _check(lib.ttamd_cast(t.device.id, t.dtype, dtype, t.dim(), self._i64(t.shape), C.c_void_p(t.storage.ptr), t.offset,
                              self._i64(t.stride), C.c_void_p(out.storage.ptr), _stream_arg()))
        return out

    def assign(self, lhs: Tensor, rhs: Tensor) -> None:
        """BackendBase::assign(lhs, rhs) (backend_base.h:78): writes rhs's elements through lhs's view."""
        if lhs.shape != rhs.shape or lhs.dtype != rhs.dtype:
            raise TTException("assign: operands must share shape and dtype")
        _check(lib.ttamd_assign(lhs.device.id, lhs.dtype, lhs.dim(), self._i64(lhs.shape), C.c_void_p(lhs.storage.ptr),
                                lhs.offset, self._i64(lhs.stride), C.c_void_p(rhs.storage.ptr), rhs.offset,
                                self._i64(rhs.stride), _stream_arg()))

    def pool2d(self, input: Tensor, op: str, kernel_size: int, stride: int, padding: int) -> Tensor:
        """BackendBase::max_pool2d / min_pool2d / avg_pool2d (backend_base.h:286-311)."""
        B, Cc, H, W = input.shape
        Ho = (H + 2 * padding - kernel_size) // stride + 1
        Wo = (W + 2 * padding - kernel_size) // stride + 1
        rdtype = _capi.F32 if (op == "avg" and input.dtype not in (_capi.F32, _capi.F64)) else input.dtype
        out = Tensor.empty((B, Cc, Ho, Wo), rdtype, input.device)
        iv = input.view4()
        _check(lib.ttamd_pool2d_forward(input.device.id, input.dtype, _capi.POOL[op], C.byref(iv), C.c_void_p(out.storage.ptr),
                                        B, Cc, H, W, kernel_size, stride, padding, _stream_arg()))
        return out

    def pool2d_backward(self, grad_output: Tensor, input: Tensor, result: Tensor, op: str, kernel_size: int, stride: int,
                        padding: int) -> Tensor:
        """BackendBase::{max,min,avg}_pool2d_backward (backend_base.h:288-311)."""
        B, Cc, H, W = input.shape
        go, res = grad_output.contiguous(), result.contiguous()
        gx = Tensor.empty(input.shape, input.dtype, input.device)
        iv = input.view4()
        _check(lib.ttamd_pool2d_backward(
            input.device.id, input.dtype, _capi.POOL[op], C.c_void_p(go.storage.ptr + go.offset * go.itemsize), C.byref(iv),
            C.c_void_p(res.storage.ptr + res.offset * res.itemsize), C.c_void_p(gx.storage.ptr), B, Cc, H, W, kernel_size,
            stride, padding, _stream_arg()))
        return gx

    def batched_matmul(self, lhs: Tensor, rhs: Tensor, bias: Tensor | None = None, bias_mode: int = 0,
                       relu: bool = False, out: Tensor | None = None, accumulate: bool = False,
                       relu_out: Tensor | None = None, relu_grad_input: Tensor | None = None,
                       colsum_out: Tensor | None = None, rhs_colsum_out: Tensor | None = None) -> Tensor:
        """BackendBase::batched_matmul (backend_base.h:130).  The keyword arguments select the fused
        epilogue of ttamd_batched_matmul; with the defaults this is the reference call exactly.
        relu_out: dense [B,N,M] tensor that receives max(out, 0) while `out` keeps the value before the ReLU;
        relu_grad_input: dense [B,N,M] saved input z of a ReLU, out = result * (z < 0 ? 0 : 1);
        colsum_out: dense [B,M] tensor that receives out summed over its rows;
        rhs_colsum_out: dense [B,M] tensor that receives rhs (dense row-major) summed over its rows."""
        out, ep = self._product(lhs, rhs, out, bias=bias, bias_mode=bias_mode, relu=relu, accumulate=accumulate, relu_out=relu_out,
                                relu_grad_input=relu_grad_input, colsum_out=colsum_out, rhs_colsum_out=rhs_colsum_out)
        B, N, K = lhs.shape
        lv, rv = lhs.view3(), rhs.view3()
        _check(lib.ttamd_batched_matmul(lhs.device.id, lhs.dtype, B, N, K, rhs.size(2), C.byref(lv), C.byref(rv),
                                        C.c_void_p(out.storage.ptr), C.byref(ep) if ep is not None else None, _stream_arg()))
        return out

    @staticmethod
    def _product(lhs: Tensor, rhs: Tensor, out: Tensor | None, bias=None, bias_mode=0, relu=False, accumulate=False,
                 relu_out=None, relu_grad_input=None, colsum_out=None, rhs_colsum_out=None):
        """The result tensor and the ttamd_epilogue (or None) of one product; checks the epilogue's tensors."""
        assert lhs.dim() == 3 and rhs.dim() == 3 and lhs.size(2) == rhs.size(1)
        B, N, K = lhs.shape
        M = rhs.size(2)
        if out is None:
            out = Tensor.empty((B, N, M), lhs.dtype, lhs.device)
        ep = None
        if (bias is not None or relu or accumulate or relu_out is not None or relu_grad_input is not None or colsum_out is not None
                or rhs_colsum_out is not None):
            ep = _capi.Epilogue()
            ep.bias = (bias.storage.ptr + bias.offset * bias.itemsize) if bias is not None else None
            ep.bias_mode = bias_mode if bias is not None else 0
            ep.relu = int(relu)
            ep.accumulate = int(accumulate)
            for name, t in (("relu_out", relu_out), ("relu_grad_input", relu_grad_input), ("colsum_out", colsum_out),
                            ("rhs_colsum_out", rhs_colsum_out)):
                if t is None:
                    continue
                want = (B, M) if name in ("colsum_out", "rhs_colsum_out") else (B, N, M)
                dense = all(n == 1 or st == d for n, st, d in zip(t.shape, t.stride, _dense_strides(t.shape)))
                if not dense or t.numel() != int(np.prod(want)) or t.dtype != lhs.dtype:
                    raise TTException(f"batched_matmul: {name} must be a dense tensor of {want} elements of the operands' dtype")
                setattr(ep, name, t.storage.ptr + t.offset * t.itemsize)
        return out, ep

    def batched_matmul_pair(self, first: tuple, second: tuple) -> tuple:
        """Two independent products in one call (ttamd_batched_matmul_pair): what TensorBatchedMatmul::backward
        (autograd/binary_ops.cpp:173-179) asks of the backend.  Each argument is (lhs, rhs) or (lhs, rhs, kwargs) with
        batched_matmul's keyword arguments; returns the two results."""
        prods, keep = [], []
        for spec in (first, second):
            lhs, rhs = spec[0], spec[1]
            kw = dict(spec[2]) if len(spec) > 2 else {}
            out, ep = self._product(lhs, rhs, kw.pop("out", None), **kw)
            lv, rv = lhs.view3(), rhs.view3()
            B, N, K = lhs.shape
            pr = _capi.Product(B, N, K, rhs.size(2), C.pointer(lv), C.pointer(rv), C.c_void_p(out.storage.ptr),
                               C.pointer(ep) if ep is not None else None)
            prods.append(pr)
            keep.append((lv, rv, ep, out))
        if keep[0][3].dtype != keep[1][3].dtype or first[0].device != second[0].device:
            raise TTException("batched_matmul_pair: both products must have one dtype and device")
        _check(lib.ttamd_batched_matmul_pair(first[0].device.id, first[0].dtype, C.byref(prods[0]), C.byref(prods[1]), _stream_arg()))
        return keep[0][3], keep[1][3]

    def batched_matmul_variant(self, lhs: Tensor, rhs: Tensor) -> str:
        B, N, K = lhs.shape
        lv, rv = lhs.view3(), rhs.view3()
        return lib.ttamd_batched_matmul_variant(lhs.dtype, B, N, K, rhs.size(2), C.byref(lv), C.byref(rv)).decode()

    def conv2d(self, input: Tensor, weight: Tensor, bias: Tensor | None, stride: int, padding: int,
               out: Tensor | None = None) -> Tensor:
        """BackendBase::conv2d (backend_base.h:269-275).  `out`: reuse a result tensor (benchmarks)."""
        B, Cc, H, W = input.shape
        O, _, k, _ = weight.shape
        Ho = (H + 2 * padding - k) // stride + 1
        Wo = (W + 2 * padding - k) // stride + 1
        if out is None:
            out = Tensor.empty((B, O, Ho, Wo), input.dtype, input.device)
        weight = weight.contiguous()  # used as the matrix [O, C*k*k], as cpu/conv.cpp:69 reshapes it
        iv, wv = input.view4(), weight.view4()
        bptr = None
        if bias is not None:
            bias = bias.contiguous()
            bptr = C.c_void_p(bias.storage.ptr + bias.offset * bias.itemsize)
        _check(lib.ttamd_conv2d_forward(input.device.id, input.dtype, C.byref(iv), C.byref(wv), bptr,
                                        C.c_void_p(out.storage.ptr), B, Cc, H, W, O, k, stride, padding, _stream_arg()))
        return out

    def conv2d_backward(self, grad_output: Tensor, input: Tensor, weight: Tensor, bias: Tensor | None, stride: int,
                        padding: int, buffers=None, return_buffers: bool = False):
        """BackendBase::conv2d_backward (backend_base.h:277-284) -> (grad_input, grad_weight, grad_bias|None).
        `return_buffers`: return (gx, gw, gb, workspace_storage) instead, a tuple that a later call takes as `buffers`
        to write into the same results and workspace (benchmarks: no allocation inside a timed loop)."""
        B, Cc, H, W = input.shape
        O, _, k, _ = weight.shape
        go = grad_output.contiguous()
        weight = weight.contiguous()
        if buffers is not None:
            gx, gw, gb, ws = buffers
        else:
            gx = Tensor.empty(input.shape, input.dtype, input.device)
            gw = Tensor.empty(weight.shape, input.dtype, input.device)
            gb = Tensor.empty((O,), input.dtype, input.device) if bias is not None else None
            ws_bytes = C.c_size_t()
            _check(lib.ttamd_conv2d_backward_workspace(input.dtype, B, Cc, H, W, O, k, stride, padding,
                                                       C.byref(ws_bytes)))
            ws = _Storage(max(ws_bytes.value, 1), input.device)
        iv, wv = input.view4(), weight.view4()
        _check(lib.ttamd_conv2d_backward(
            input.device.id, input.dtype, C.c_void_p(go.storage.ptr + go.offset * go.itemsize), C.byref(iv),
            C.byref(wv), C.c_void_p(gx.storage.ptr), C.c_void_p(gw.storage.ptr),
            C.c_void_p(gb.storage.ptr) if gb is not None else None, B, Cc, H, W, O, k, stride, padding,
            C.c_void_p(ws.ptr), ws.nbytes, _stream_arg()))
        if return_buffers:
            return gx, gw, gb, ws
        # (no wait for the kernels: like every other temporary, the workspace goes back to the allocator in stream order)
        return gx, gw, gb


_BACKEND = BackendAMD()


def get_backend(device: Device) -> BackendAMD:
    """get_backend(Device) (tinytensor/tensor/backend_register.cpp:19-38)."""
    if device.backend != "amd":
        raise TTException(f"Unknown device type {device.backend}")
    return _BACKEND


class Generator:
    """tinytensor::Generator (tensor/random.cpp:46-63): state = splitmix64(seed); xorshift64 steps."""

    def __init__(self, seed: int = 0):
        m = (1 << 64) - 1
        r = (seed + 0x9E3779B97F4A7C15) & m
        r = ((r ^ (r >> 30)) * 0xBF58476D1CE4E5B9) & m
        r = ((r ^ (r >> 27)) * 0x94D049BB133111EB) & m
        self.state = C.c_uint64(r ^ (r >> 31))


_DEFAULT_GENERATOR = Generator(0)


def default_generator() -> Generator:
    """get_default_generator() (tensor/random.cpp:69-90): the generator that draws without an explicit one use."""
    return _DEFAULT_GENERATOR


def set_default_generator_seed(seed: int) -> None:
    """set_default_generator_seed (tensor/random.cpp:84-86)."""
    _DEFAULT_GENERATOR.state = Generator(seed).state


def _random_fill(shape, dtype, dist, p0, p1, gen: Generator, device: Device) -> Tensor:
    out = Tensor.empty(shape, dtype, device)
    _check(lib.ttamd_random_fill(device.id, dtype, dist, p0, p1, C.byref(gen.state), out.numel(),
                                 C.c_void_p(out.storage.ptr), _stream_arg()))
    return out


def uniform_real(low: float, high: float, shape, gen: Generator, dtype: int = _capi.F32, device: Device = kAMD) -> Tensor:
    """tinytensor::uniform_real(low, high, shape, options, gen) (tensor/tensor.cpp:1773-1781)."""
    if not low < high:
        raise TTException("Expected low < high. At least one element violates this.")
    return _random_fill(shape, dtype, 0, low, high, gen, device)


def normal(mu: float, std: float, shape, gen: Generator, dtype: int = _capi.F32, device: Device = kAMD) -> Tensor:
    return _random_fill(shape, dtype, 1, mu, std, gen, device)


def linear_init(in_features: int, out_features: int, gen: Generator, dtype: int = _capi.F32, device: Device = kAMD):
    """nn::Linear's constructor (nn/linear.cpp:20-40): weight [in,out] by kaiming_uniform_ (gain 1, fan = size(0)),
    then bias ~ U(+-1/sqrt(fan)); both drawn from `gen` in that order."""
    fan = float(in_features)
    bound_w = (3.0 ** 0.5) * (1.0 / fan ** 0.5)
    W = uniform_real(-bound_w, bound_w, (in_features, out_features), gen, dtype, device)
    bound_b = 1.0 / fan ** 0.5
    b = uniform_real(-bound_b, bound_b, (out_features,), gen, dtype, device)
    return W, b


def calc_fan_in_out(t: Tensor):
    """nn::calc_fan_in_out (nn/init.cpp:30-52): BOTH fans are size(0) times the receptive field (sizes beyond dim 1)."""
    if t.dim() < 2:
        raise TTException(f"Unable to calculate fan in and fan out for tensors with dimensions fewer than 2. Given tensor "
                          f"with {t.dim()} dimensions")
    field = 1
    for d in range(2, t.dim()):
        field *= t.size(d)
    return float(t.size(0) * field), float(t.size(0) * field)


def kaiming_uniform_(t: Tensor, gen: Generator, gain: float = 1.0) -> None:
    """nn::kaiming_uniform_ (nn/init.cpp:106-112), fan_in mode: U(+-sqrt(3) * gain / sqrt(fan)) drawn in place."""
    fan, _ = calc_fan_in_out(t)
    bound = math.sqrt(3.0) * (gain / math.sqrt(fan))
    t.uniform_real_(-bound, bound, gen)


class Conv2d:
    """nn::Conv2d (nn/conv2d.cpp:20-81, include/tt/nn/conv2d.h:35-44).  weight [out,in,k,k] is initialised through the
    view weight.permute(1,0,2,3) (conv2d.cpp:56): the draws run over [in,out,k,k] in row-major order of that view and
    its fan is in_channels*k*k; the bias bound comes from calc_fan_in_out(weight) = out_channels*k*k (conv2d.cpp:60-62).
    Both are drawn from `gen` (the reference uses the thread's default generator) in that order."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size: int, stride: int, padding: int, bias: bool = True,
                 dtype: int = _capi.F32, device: Device = kAMD, gen: Generator | None = None):
        for name, v, ok in (("in_channels", in_channels, in_channels > 0), ("out_channels", out_channels, out_channels > 0),
                            ("kernel_size", kernel_size, kernel_size > 0), ("stride", stride, stride > 0)):
            if not ok:
                raise TTException(f"Expected {name} > 0, given {name}={v}")
        if padding < 0:
            raise TTException(f"Expected padding >= 0, given padding={padding}")
        gen = gen if gen is not None else default_generator()
        self.stride, self.padding = stride, padding
        self.weight = Tensor.empty((out_channels, in_channels, kernel_size, kernel_size), dtype, device)
        kaiming_uniform_(self.weight.permute(1, 0, 2, 3), gen)
        self.bias = None
        if bias:
            self.bias = Tensor.empty((out_channels,), dtype, device)
            fan_in, _ = calc_fan_in_out(self.weight)
            bound = 1.0 / math.sqrt(fan_in)
            self.bias.uniform_real_(-bound, bound, gen)

    def parameters(self):
        return [self.weight] + ([self.bias] if self.bias is not None else [])

    def forward(self, input: Tensor) -> Tensor:
        if input.dim() == 4 and input.size(1) != self.weight.size(1):
            raise TTException(f"Input channels {input.size(1)} does not match layer input channels {self.weight.size(1)}")
        return conv2d(input, self.weight, self.bias, self.stride, self.padding)

    __call__ = forward


class Linear:
    """nn::Linear (nn/linear.cpp:20-50): weight [in,out] by kaiming_uniform_, bias ~ U(+-1/sqrt(in)), forward
    matmul(input, weight) + bias with the bias add fused into the GEMM's epilogue."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, dtype: int = _capi.F32, device: Device = kAMD,
                 gen: Generator | None = None):
        gen = gen if gen is not None else default_generator()
        self.weight = Tensor.empty((in_features, out_features), dtype, device)
        kaiming_uniform_(self.weight, gen)
        self.bias = None
        if bias:
            self.bias = Tensor.empty((out_features,), dtype, device)
            fan_in, _ = calc_fan_in_out(self.weight)
            bound = 1.0 / math.sqrt(fan_in)
            self.bias.uniform_real_(-bound, bound, gen)

    def parameters(self):
        return [self.weight] + ([self.bias] if self.bias is not None else [])

    def forward(self, input: Tensor) -> Tensor:
        return linear(input, self.weight, self.bias)

    __call__ = forward


def full(shape, value, dtype: int = _capi.F32, device: Device = kAMD) -> Tensor:
    """tinytensor::full: a one-element storage expanded to `shape` (stride 0), like Tensor(Scalar).expand()."""
    shape = tuple(shape)
    one = get_backend(device).full(value, 1, dtype, device)
    return Tensor(one.storage, dtype, shape, (0,) * len(shape), 0)


_CONSTANTS: dict = {}  # (bytes of the value in its dtype, dtype, device id) -> one-element tensor


def _constant(shape, value, dtype: int, device: Device) -> Tensor:
    """A scalar operand of an element-wise call (`t * 2.0`, `where(c, 0.0, 1.0)`) as a stride-0 view of a one-element
    tensor that is kept for the next call with the same value: such operands are only ever read, so one launch fills
    the element the first time and later calls launch nothing (a training step written op by op issues ten of these
    fills).  The element is filled on the current stream and the device synchronised before it goes into the table, so
    that any stream may read it afterwards; a first use inside a stream capture cannot wait and stays a one-off
    (the warm-up runs that precede a capture have normally met the value already).  `full()` itself never shares."""
    shape = tuple(shape)
    key = (np.array(value).astype(_NP_OF[dtype]).tobytes(), dtype, device.id)
    one = _CONSTANTS.get(key)
    if one is None:
        one = get_backend(device).full(value, 1, dtype, device)
        from .graph import stream_is_capturing
        if not stream_is_capturing(_STREAM):
            get_backend(device).synchronize(device.id)
            if len(_CONSTANTS) >= 256:
                _CONSTANTS.pop(next(iter(_CONSTANTS)))
            _CONSTANTS[key] = one
    elif _PINNED is not None:
        # a cached constant read inside a capture: the graph replays with this address, so the storage must outlive
        # its eviction from the cache (otherwise the block could go to another tensor between replays)
        _PINNED.append(one.storage)
    return Tensor(one.storage, dtype, shape, (0,) * len(shape), 0)


def broadcast_tensors(a: Tensor, b: Tensor):
    """Right-aligned broadcasting through unsqueeze + expand views (no data movement)."""
    while a.dim() < b.dim():
        a = a.unsqueeze(0)
    while b.dim() < a.dim():
        b = b.unsqueeze(0)
    shape = []
    for x, y in zip(a.shape, b.shape):
        if x != y and x != 1 and y != 1:
            raise TTException(f"Shapes {a.shape} and {b.shape} cannot be broadcast")
        shape.append(max(x, y) if 0 not in (x, y) else 0)
    return a.expand(shape), b.expand(shape)


def where(cond: Tensor, lhs, rhs) -> Tensor:
    """tinytensor::where with scalar or tensor branches."""
    if not isinstance(lhs, Tensor):
        lhs = _constant(cond.shape, lhs, rhs.dtype if isinstance(rhs, Tensor) else _capi.F32, cond.device)
    if not isinstance(rhs, Tensor):
        rhs = _constant(cond.shape, rhs, lhs.dtype, cond.device)
    lhs, rhs = broadcast_tensors(lhs, rhs)
    cond, lhs = broadcast_tensors(cond, lhs)
    cond, rhs = broadcast_tensors(cond, rhs)
    return get_backend(cond.device).where(cond, lhs, rhs)


# -------------------------------------------------------------------------------------------------
def _promote(lhs: Tensor, rhs: Tensor):
    if lhs.device != rhs.device:
        raise TTException(f"Expected tensors on the same device, given {lhs.device} and {rhs.device}")
    dt = max(lhs.dtype, rhs.dtype)
    if dt == _capi.BOOL:
        raise TTException("matmul does not support boolean tensors")
    # check_promote (tensor/tensor.cpp:2398-2399): operands are cast to promote_types(lhs, rhs), which orders the
    # dtypes bool < u8 < i16 < i32 < i64 < f32 < f64 (common/scalar.cpp:17-26)
    return lhs.to(dt), rhs.to(dt)


def matmul(lhs: Tensor, rhs: Tensor) -> Tensor:
    """tinytensor::matmul (tensor/tensor.cpp:2390-2484): rank dispatch onto batched_matmul."""
    lhs, rhs = _promote(lhs, rhs)
    be = get_backend(lhs.device)
    ls, rs = lhs.shape, rhs.shape
    if lhs.dim() == 1 and rhs.dim() == 1:
        if ls[0] != rs[0]:
            raise TTException(f"Invalid shapes for dot product. LHS={ls} and RHS={rs}")
        return be.batched_matmul(lhs.reshape([1, 1, ls[0]]), rhs.reshape([1, rs[0], 1])).flatten()
    if lhs.dim() == 1 and rhs.dim() == 2:
        if ls[0] != rs[0]:
            raise TTException(f"Invalid shape for matrix multiplication. LHS={ls} and RHS={rs}")
        return be.batched_matmul(lhs.reshape([1, 1, ls[0]]), rhs.unsqueeze(0)).flatten()
    if lhs.dim() == 2 and rhs.dim() == 1:
        if ls[1] != rs[0]:
            raise TTException(f"Invalid shape for matrix multiplication. LHS={ls} and RHS={rs}")
        return be.batched_matmul(lhs.unsqueeze(0), rhs.reshape([1, rs[0], 1])).flatten()
    if lhs.dim() == 2 and rhs.dim() == 2:
        if ls[1] != rs[0]:
            raise TTException(f"Invalid shape for matrix multiplication. LHS={ls} and RHS={rs}")
        return be.batched_matmul(lhs.unsqueeze(0), rhs.unsqueeze(0)).squeeze(0)
    if lhs.dim() == 3 and rhs.dim() == 3:
        if ls[2] != rs[1] or ls[0] != rs[0]:
            raise TTException(f"Invalid shape for batched matrix multiplication. LHS={ls} and RHS={rs}")
        return be.batched_matmul(lhs, rhs)
    raise TTException("Unsupported sizes. Try reshaping or broadcasting.")


def matmul_backward(lhs: Tensor, rhs: Tensor, grad_output: Tensor):
    """TensorBatchedMatmul::backward (autograd/binary_ops.cpp:173-179): dA = dC.B^T, dB = A^T.dC, both
    on permute({0,2,1}) VIEWS.  Both gradients are always computed, as in the reference."""
    if (lhs.dim() == 3 and rhs.dim() == 3 and grad_output.dim() == 3 and lhs.dtype == rhs.dtype == grad_output.dtype
            and lhs.dtype != _capi.BOOL and lhs.device == rhs.device == grad_output.device
            and grad_output.shape == (lhs.size(0), lhs.size(1), rhs.size(2)) and lhs.size(2) == rhs.size(1) and lhs.size(0) == rhs.size(0)):
        # what forward stored: 3-D operands of one dtype -- both products in one backend call (one grid where that pays)
        return get_backend(lhs.device).batched_matmul_pair((grad_output, rhs.permute(0, 2, 1)), (lhs.permute(0, 2, 1), grad_output))
    return matmul(grad_output, rhs.permute(0, 2, 1)), matmul(lhs.permute(0, 2, 1), grad_output)


def linear(input: Tensor, weight: Tensor, bias: Tensor | None = None, relu: bool = False) -> Tensor:
    """nn::Linear::forward (nn/linear.cpp:42-50): matmul(input.flatten(0,-2), weight) + bias, weight
    [in,out].  The bias add (and an optional ReLU that follows it) is fused into the GEMM epilogue."""
    x2 = input.flatten(0, -2) if input.dim() != 2 else input
    if x2.size(1) != weight.size(0):
        raise TTException(f"Invalid shape for matrix multiplication. LHS={x2.shape} and RHS={weight.shape}")
    x2, weight = _promote(x2, weight)
    if bias is not None:
        bias = bias.to(x2.dtype)
    out = get_backend(input.device).batched_matmul(x2.unsqueeze(0), weight.unsqueeze(0), bias=bias, bias_mode=1,
                                                   relu=relu)
    return out.reshape(list(input.shape[:-1]) + [weight.size(1)])


def linear_relu(input: Tensor, weight: Tensor, bias: Tensor | None = None):
    """nn::Linear::forward followed by relu() in one launch -> (z, a): z = input . weight + bias is what autograd saves
    as the ReLU's input (autograd/unary_ops.cpp:562-567), a = max(z, 0) what the next layer reads."""
    x2 = input.flatten(0, -2) if input.dim() != 2 else input
    if x2.size(1) != weight.size(0):
        raise TTException(f"Invalid shape for matrix multiplication. LHS={x2.shape} and RHS={weight.shape}")
    x2, weight = _promote(x2, weight)
    if bias is not None:
        bias = bias.to(x2.dtype)
    a = Tensor.empty((1, x2.size(0), weight.size(1)), x2.dtype, x2.device)
    z = get_backend(input.device).batched_matmul(x2.unsqueeze(0), weight.unsqueeze(0), bias=bias, bias_mode=1, relu_out=a)
    shape = list(input.shape[:-1]) + [weight.size(1)]
    return z.reshape(shape), a.reshape(shape)


def linear_backward(grad_output: Tensor, input: Tensor, weight: Tensor, relu_input: Tensor | None = None,
                    bias_grad: bool | str = True):
    """Backward of y = x . W (+ b) for 2-D operands dy = grad_output [n, out], x = input [n, in], W = weight [in, out],
    as autograd emits it (TensorBatchedMatmul::backward on permute views, autograd/binary_ops.cpp:173-179) with the
    element-wise steps that follow dx fused into its GEMM:
        dx = dy . W^T;
        when x = relu(relu_input): dx *= where(relu_input < 0, 0, 1)   (TensorRelu::backward, unary_ops.cpp:568-573);
        when bias_grad is True: db_prev = dx.sum(0), the bias gradient of the Linear layer that produced relu_input,
            from the store of dx's GEMM;
        dW = x^T . dy;
        when bias_grad == "own": db = dy.sum(0), this layer's own bias gradient, from the vectors of dy that dW's GEMM
            stages (dy must be dense).
    Returns (dx, dW, db_prev | db | None)."""
    be = get_backend(grad_output.device)
    n, fin = input.shape
    own = bias_grad == "own"
    fout = grad_output.size(1)
    db = Tensor.empty((1, fout if own else fin), grad_output.dtype, grad_output.device) if bias_grad else None
    dx, dW = be.batched_matmul_pair(
        (grad_output.unsqueeze(0), weight.unsqueeze(0).permute(0, 2, 1),
         dict(relu_grad_input=relu_input.unsqueeze(0) if relu_input is not None else None, colsum_out=None if own else db)),
        (input.unsqueeze(0).permute(0, 2, 1), grad_output.unsqueeze(0), dict(rhs_colsum_out=db if own else None)))
    return dx.squeeze(0), dW.squeeze(0), (db.reshape([fout if own else fin]) if db is not None else None)


def mse_loss(input: Tensor, target: Tensor, grad: bool = True, bias_grad: bool = False):
    """nn::mse_loss(input, target) with mean reduction (nn/loss.cpp:69-72) and, when `grad`, its backward in the same
    pass -> (loss [1], grad_input | None, grad_input.sum(0) | None).  2-D dense operands of one float dtype."""
    if input.shape != target.shape or input.dtype != target.dtype or input.dim() != 2:
        raise TTException("mse_loss: input and target must be 2-D tensors of one shape and dtype")
    input, target = input.contiguous(), target.contiguous()
    rows, cols = input.shape
    loss = Tensor.empty((1,), input.dtype, input.device)
    g = Tensor.empty(input.shape, input.dtype, input.device) if grad else None
    cs = Tensor.empty((cols,), input.dtype, input.device) if (grad and bias_grad) else None
    ptr = lambda t: C.c_void_p(t.storage.ptr + t.offset * t.itemsize) if t is not None else None
    _check(lib.ttamd_mse_loss(input.device.id, input.dtype, rows, cols, ptr(input), ptr(target), ptr(loss), ptr(g), ptr(cs),
                              _stream_arg()))
    return loss, g, cs


def linear_mse_head(input: Tensor, weight: Tensor, bias: Tensor | None, target: Tensor, relu_input: Tensor | None = None):
    """A network's last Linear layer with the loss behind it, forward and backward in one call:
    y = nn::Linear::forward(input) (nn/linear.cpp:42-50), loss = nn::mse_loss(y, target) (nn/loss.cpp:69-72) and what
    autograd makes of them -- dy = (1 / numel) * 2 * (y - target) (reduce_ops.cpp:195-205, binary_ops.cpp:153-159),
    dx = (dy . W^T) * where(relu_input < 0, 0, 1), dW = x^T . dy (binary_ops.cpp:173-179, unary_ops.cpp:568-573),
    db = dy.sum(0).  2-D operands of one float dtype, at most 64 outputs.
    Returns (y, loss [1], dx, dW, db | None)."""
    if input.dim() != 2 or weight.dim() != 2 or target.dim() != 2:
        raise TTException("linear_mse_head: input, weight and target must be 2-D")
    rows, fin = input.shape
    fout = weight.size(1)
    if weight.size(0) != fin:
        raise TTException(f"Invalid shape for matrix multiplication. LHS={input.shape} and RHS={weight.shape}")
    if tuple(target.shape) != (rows, fout) or (relu_input is not None and tuple(relu_input.shape) != (rows, fin)):
        raise TTException("linear_mse_head: target must be [rows, out_features] and relu_input [rows, in_features]")
    if bias is not None and bias.numel() != fout:
        raise TTException("linear_mse_head: bias must hold out_features elements")
    others = [t for t in (weight, bias, target, relu_input) if t is not None]
    if any(t.dtype != input.dtype for t in others) or input.dtype not in (_capi.F32, _capi.F64):
        raise TTException("linear_mse_head: operands of one floating point dtype")
    if rows < 1 or fin < 1 or fout < 1 or fout > 64:
        raise TTException("linear_mse_head: at least one row, input and output; at most 64 outputs")
    input, weight, target = input.contiguous(), weight.contiguous(), target.contiguous()
    bias = bias.contiguous() if bias is not None else None
    relu_input = relu_input.contiguous() if relu_input is not None else None
    new = lambda *shape: Tensor.empty(shape, input.dtype, input.device)
    y, loss, dy, dx, dW = new(rows, fout), new(1), new(rows, fout), new(rows, fin), new(fin, fout)
    db = new(fout) if bias is not None else None
    ptr = lambda t: C.c_void_p(t.storage.ptr + t.offset * t.itemsize) if t is not None else None
    _check(lib.ttamd_linear_mse_head(input.device.id, input.dtype, rows, fin, fout, ptr(input), ptr(weight), ptr(bias), ptr(target),
                                     ptr(relu_input), ptr(y), ptr(loss), ptr(dy), ptr(dx), ptr(dW), ptr(db), _stream_arg()))
    return y, loss, dx, dW, db


def conv2d(input: Tensor, weight: Tensor, bias: Tensor | None = None, stride: int = 1, padding: int = 0) -> Tensor:
    """tinytensor::conv2d argument checks (tensor/tensor.cpp:3089-3167) then BackendBase::conv2d."""
    if input.dim() != 4 or weight.dim() != 4:
        raise TTException("conv2d expects 4-D input [B,C,H,W] and weight [O,C,k,k]")
    if input.size(1) != weight.size(1):
        raise TTException("conv2d: input channels do not match weight channels")
    if weight.size(2) != weight.size(3):
        raise TTException("conv2d: only square kernels are supported")
    if stride <= 0 or padding < 0:
        raise TTException("conv2d: stride must be > 0 and padding >= 0")
    if bias is not None and (bias.dim() != 1 or bias.size(0) != weight.size(0)):
        raise TTException("conv2d: bias must have one entry per output channel")
    if input.dtype != weight.dtype or input.dtype == _capi.BOOL:
        raise TTException("conv2d: operands must share one non-bool dtype")
    return get_backend(input.device).conv2d(input, weight, bias, stride, padding)


def conv2d_backward(grad_output: Tensor, input: Tensor, weight: Tensor, bias: Tensor | None = None, stride: int = 1,
                    padding: int = 0):
    """TensorConv2d::backward (autograd/conv_ops.cpp:55-80) -> BackendBase::conv2d_backward."""
    return get_backend(input.device).conv2d_backward(grad_output, input, weight, bias, stride, padding)


def _pool2d(input: Tensor, op: str, kernel_size: int, stride: int, padding: int) -> Tensor:
    # argument checks of tinytensor::{max,min,avg}_pool2d (tensor/tensor.cpp:3169-3198)
    if input.dtype == _capi.BOOL:
        raise TTException(f"{op}_pool2d: bool tensors are not supported")
    if input.dim() != 4:
        raise TTException(f"Input shape {input.shape} expected to have 4 dimensions.")
    if stride <= 0:
        raise TTException(f"Stide of {stride} is expected to be positive.")
    if padding < 0:
        raise TTException(f"Padding of {padding} is expected to be non-negative.")
    if input.size(2) + padding < kernel_size or input.size(3) + padding < kernel_size:
        raise TTException(f"Kernel size {kernel_size} cannot be greater than input size ({input.size(2)}, {input.size(3)}) "
                          f"+ padding {padding}")
    return get_backend(input.device).pool2d(input, op, kernel_size, stride, padding)


def max_pool2d(input: Tensor, kernel_size: int, stride: int, padding: int) -> Tensor:
    return _pool2d(input, "max", kernel_size, stride, padding)


def min_pool2d(input: Tensor, kernel_size: int, stride: int, padding: int) -> Tensor:
    return _pool2d(input, "min", kernel_size, stride, padding)


def avg_pool2d(input: Tensor, kernel_size: int, stride: int, padding: int) -> Tensor:
    return _pool2d(input, "avg", kernel_size, stride, padding)


def pool2d_backward(grad_output: Tensor, input: Tensor, result: Tensor, op: str, kernel_size: int, stride: int,
                    padding: int) -> Tensor:
    """Tensor{Max,Min,Avg}Pool2d::backward (autograd/conv_ops.cpp:100-190) -> BackendBase::*_pool2d_backward."""
    return get_backend(input.device).pool2d_backward(grad_output, input, result, op, kernel_size, stride, padding)
