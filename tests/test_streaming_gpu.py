"""GPU tests for the dense 16-byte-vector forms and the tiled transposing copy of the streaming kernels
(elementwise binary / unary / where / cast / sum / contiguous).  Sizes are chosen so that the vector body, the
element-wise tail and the unaligned fall-back all run; expected values are numpy's on the same inputs (the
operations are single IEEE operations or integer arithmetic, so the comparison is bit-exact; sum is
tolerance-based because the reduction order differs from numpy's)."""
import numpy as np
import pytest

from helpers import ALL_NON_BOOL

pytestmark = pytest.mark.gpu


def dev(tt, a):
    return tt.Tensor.from_numpy(a)


@pytest.mark.parametrize("dtype", ALL_NON_BOOL)
@pytest.mark.parametrize("n", [1, 15, 16, 1000, 4099, 70001])
def test_dense_binary_unary_where_with_tails_and_offsets(tt, dtype, n):
    rng = np.random.default_rng(n)
    a = rng.integers(1, 9, n + 3).astype(dtype)
    b = rng.integers(1, 9, n + 3).astype(dtype)
    ta, tb = dev(tt, a), dev(tt, b)
    be = tt.get_backend(tt.kAMD)
    for off in (0, 1):  # offset 1: the view is dense but not 16-byte aligned
        va = tt.Tensor(ta.storage, ta.dtype, (n,), (1,), off)
        vb = tt.Tensor(tb.storage, tb.dtype, (n,), (1,), off)
        x, y = a[off:off + n], b[off:off + n]
        assert np.array_equal((va + vb).to_numpy(), x + y)
        assert np.array_equal((va * vb).to_numpy(), x * y)
        assert np.array_equal((va / vb).to_numpy(), (x / y).astype(dtype) if np.dtype(dtype).kind == "f" else x // y)
        lt = va < vb
        assert np.array_equal(lt.to_numpy(), x < y)
        assert np.array_equal(be.unary(va, "negate").to_numpy(), (0 - x).astype(dtype))
        assert np.array_equal(tt.where(lt, va, vb).to_numpy(), np.where(x < y, x, y))
        assert np.array_equal(va.to(tt._capi.F64).to_numpy(), x.astype(np.float64))
        assert np.array_equal(va.to(tt._capi.U8).to_numpy(), x.astype(np.uint8))
        assert np.array_equal(va.contiguous().to_numpy(), x)
        assert np.array_equal(be.identity(va).to_numpy(), x)


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.float32, np.float64])
@pytest.mark.parametrize("shape,perm", [
    ((70, 130), (1, 0)),            # 2-D transpose, ragged 64x64 tiles
    ((3, 65, 100), (0, 2, 1)),      # batched transpose (the backward GEMM views)
    ((2, 20, 24, 33), (0, 3, 1, 2)),  # NHWC storage viewed as NCHW
    ((5, 17, 40), (2, 0, 1)),       # unit-stride dimension moved to the front
    ((4, 8, 9), (0, 2, 1)),         # too small for tiles: element-wise gather
    ((16, 1, 48), (2, 1, 0)),
])
def test_contiguous_of_permuted_views(tt, dtype, shape, perm):
    rng = np.random.default_rng(sum(shape))
    a = rng.integers(0, 100, shape).astype(dtype)
    t = dev(tt, a).permute(*perm)
    assert not t.is_contiguous()
    got = t.contiguous()
    assert got.is_contiguous() and np.array_equal(got.to_numpy(), a.transpose(perm))
    # a window of the permuted view (offset, larger strides) goes the same way
    if len(shape) == 2:
        big = rng.integers(0, 100, (shape[0] + 5, shape[1] + 7)).astype(dtype)
        tb = dev(tt, big)
        view = tt.Tensor(tb.storage, tb.dtype, (shape[1], shape[0]), (1, shape[1] + 7), 2 * (shape[1] + 7) + 3)
        assert np.array_equal(view.contiguous().to_numpy(), big[2:2 + shape[0], 3:3 + shape[1]].T)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32])
def test_sum_large_dense_and_strided(tt, dtype):
    rng = np.random.default_rng(0)
    a = rng.integers(-8, 9, (2051, 4099)).astype(dtype)   # 8.4 M elements: the two-stage, 16-byte-load form
    t = dev(tt, a)
    exact = int(a.astype(np.int64).sum())
    assert float(t.sum().item()) == exact                   # small integers: exact in every order
    assert float(t.permute(1, 0).sum().item()) == exact     # strided view
    assert np.array_equal(t.sum(0).to_numpy(), a.sum(0).astype(dtype))
    if np.dtype(dtype).kind == "f":
        b = rng.normal(size=(1500, 3001)).astype(dtype)
        got = float(dev(tt, b).sum().item())
        want = float(b.astype(np.float64).sum())
        assert abs(got - want) <= (1e-3 if dtype == np.float32 else 1e-9) * np.abs(b).sum()
