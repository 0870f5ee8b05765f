"""GPU tests for ttamd_cast (BackendBase::to) and ttamd_assign (BackendBase::assign) through the C ABI.
The expected values are numpy's: astype is C's static_cast for in-range values (cpu/cast.cpp:27-34), and view
assignment is the element loop of cpu/kernel/assign.hpp:15-21.  Bit-exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

DTYPES = [np.bool_, np.uint8, np.int16, np.int32, np.int64, np.float32, np.float64]


def dev(tt, a):
    return tt.Tensor.from_numpy(a)


@pytest.mark.parametrize("src", DTYPES)
@pytest.mark.parametrize("dst", DTYPES)
def test_cast_every_pair(tt, src, dst):
    rng = np.random.default_rng(7)
    if src == np.bool_:
        a = rng.integers(0, 2, (5, 7, 3)).astype(src)
    elif np.dtype(src).kind == "f":
        a = (rng.integers(0, 200, (5, 7, 3)) / 4.0).astype(src)   # fractional, in range of every target, non-negative
        a[0, 0, 0] = 0.0
    else:
        a = rng.integers(0, 120, (5, 7, 3)).astype(src)
    t = dev(tt, a)
    code = tt.Tensor.from_numpy(np.zeros(1, dst)).dtype
    got = t.to(code).to_numpy()
    assert got.dtype == np.dtype(dst) and np.array_equal(got, a.astype(dst))
    # a permuted view is read through its strides; signed values keep their sign where the target has one
    if np.dtype(src).kind in "if" and np.dtype(dst).kind in "if":
        b = -a
        assert np.array_equal(dev(tt, b).permute(2, 0, 1).to(code).to_numpy(), b.transpose(2, 0, 1).astype(dst))
    if dst == src:
        assert t.to(code) is t   # Tensor::to returns the tensor itself (tensor/tensor.cpp:536-538)


@pytest.mark.parametrize("dtype", DTYPES)
def test_assign_through_views(tt, dtype):
    rng = np.random.default_rng(9)
    base = rng.integers(0, 100, (6, 10)).astype(dtype)
    rhs = rng.integers(0, 100, (4, 3)).astype(dtype)
    tb = dev(tt, base)
    # lhs = base[1:5, 2:8:2] as an explicit (offset, stride) view; rhs read through a transposed view
    lhs = tt.Tensor(tb.storage, tb.dtype, (4, 3), (10, 2), 12)
    lhs.assign(dev(tt, np.ascontiguousarray(rhs.T)).permute(1, 0))
    want = base.copy()
    want[1:5, 2:8:2] = rhs
    assert np.array_equal(tb.to_numpy(), want)
    with pytest.raises(tt.TTException):
        lhs.assign(dev(tt, rhs[:2]))                     # shape mismatch
