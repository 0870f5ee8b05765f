"""GPU parity tests for ttamd_pool2d_forward / ttamd_pool2d_backward through the C ABI, against the CPU oracle
(oracle/tt_oracle_pool.c).  The kernels fold each window in the reference's order with its arithmetic, so the
comparison is bit-exact for every dtype, forward and backward, ties and padding included.
"""
import numpy as np
import pytest

from helpers import ALL_NON_BOOL

pytestmark = pytest.mark.gpu

OPS = ["max", "min", "avg"]


def dev(tt, a):
    return tt.Tensor.from_numpy(a)


def forward(tt, op, t, k, S, P):
    return {"max": tt.max_pool2d, "min": tt.min_pool2d, "avg": tt.avg_pool2d}[op](t, k, S, P)


@pytest.mark.parametrize("op", OPS)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_reference_shape_forward_backward_exact(tt, oracle, op, dtype):
    # tests/test_conv.cpp:186-278 and tests/test_conv_autograd.cpp:109-230: B4 C128 68x28, k3 s2 p1, random data
    rng = np.random.default_rng(1)
    x = rng.normal(size=(4, 128, 68, 28)).astype(dtype)
    tx = dev(tt, x)
    out = forward(tt, op, tx, 3, 2, 1)
    want = oracle.pool2d_forward(x, op, 3, 2, 1)
    assert out.shape == want.shape == (4, 128, 34, 14)
    assert np.array_equal(out.to_numpy(), want)
    g = rng.normal(size=want.shape).astype(dtype)
    gx = tt.pool2d_backward(dev(tt, g), tx, out, op, 3, 2, 1)
    assert np.array_equal(gx.to_numpy(), oracle.pool2d_backward(g, x, want, op, 3, 2, 1))


@pytest.mark.parametrize("op", OPS)
@pytest.mark.parametrize("dtype", ALL_NON_BOOL)
@pytest.mark.parametrize("geom", [(2, 3, 9, 8, 2, 2, 0), (1, 2, 7, 7, 3, 1, 1), (2, 2, 6, 9, 3, 3, 2), (1, 1, 5, 5, 5, 1, 2), (3, 1, 1, 1, 1, 1, 0),
                                  # non-overlapping windows: odd width (no pair accesses), rows / columns no window reaches
                                  (2, 3, 9, 7, 2, 2, 0), (1, 2, 10, 11, 3, 3, 0), (2, 2, 8, 8, 4, 4, 0), (1, 3, 64, 66, 2, 2, 0),
                                  # overlapping windows on rows of 4n elements (four elements per lane in backward): three,
                                  # four and five covering output columns, a single group per row, padding wider than 1
                                  (2, 3, 9, 8, 3, 2, 1), (1, 2, 7, 12, 2, 1, 0), (2, 2, 10, 16, 4, 2, 1), (1, 2, 6, 8, 2, 1, 1),
                                  (1, 1, 5, 4, 3, 2, 0), (2, 1, 11, 20, 6, 3, 2), (1, 2, 9, 24, 5, 4, 2),
                                  # rows longer than a wave's 64 groups of four, and rows that end inside a wave
                                  (1, 2, 9, 520, 3, 2, 1), (2, 1, 7, 44, 3, 2, 1), (1, 1, 6, 256, 3, 2, 1), (1, 2, 5, 260, 2, 1, 0),
                                  # two and three input rows (every window hangs over an edge), a single group of four
                                  (1, 2, 2, 4, 3, 2, 1), (2, 1, 2, 8, 3, 2, 1), (1, 1, 3, 4, 3, 2, 1)])
def test_every_dtype_and_geometry_exact(tt, oracle, op, dtype, geom):
    Bn, Cc, H, W, k, S, P = geom
    rng = np.random.default_rng(sum(geom))
    lo = 0 if np.dtype(dtype).kind == "u" else -3
    x = rng.integers(lo, 4, (Bn, Cc, H, W)).astype(dtype)  # few distinct values: ties everywhere
    tx = dev(tt, x)
    out = forward(tt, op, tx, k, S, P)
    want = oracle.pool2d_forward(x, op, k, S, P)
    got = out.to_numpy()
    assert got.dtype == want.dtype and np.array_equal(got, want)
    if np.dtype(dtype).kind == "f":
        g = rng.integers(-4, 5, want.shape).astype(dtype)
        gx = tt.pool2d_backward(dev(tt, g), tx, out, op, k, S, P)
        assert np.array_equal(gx.to_numpy(), oracle.pool2d_backward(g, x, want, op, k, S, P))


def test_strided_input_view_empty_batch_and_errors(tt, oracle):
    rng = np.random.default_rng(2)
    xs = rng.normal(size=(2, 9, 8, 3)).astype(np.float32)   # stored NHWC
    x = np.ascontiguousarray(xs.transpose(0, 3, 1, 2))
    tx = dev(tt, xs).permute(0, 3, 1, 2)
    assert not tx.is_contiguous()
    for op in OPS:
        for k, S, P in ((3, 2, 1), (2, 2, 0)):
            out = forward(tt, op, tx, k, S, P)
            want = oracle.pool2d_forward(x, op, k, S, P)
            assert np.array_equal(out.to_numpy(), want)
            g = rng.normal(size=want.shape).astype(np.float32)
            gx = tt.pool2d_backward(dev(tt, g), tx, out, op, k, S, P)
            assert gx.is_contiguous() and np.array_equal(gx.to_numpy(), oracle.pool2d_backward(g, x, want, op, k, S, P))
    empty = tt.Tensor.empty((0, 3, 8, 8), tt._capi.F32)
    assert tt.max_pool2d(empty, 2, 2, 0).shape == (0, 3, 4, 4)
    with pytest.raises(tt.TTException):
        tt.max_pool2d(dev(tt, x.astype(bool)), 2, 2, 0)              # bool is rejected (DISABLE_BOOL)
    with pytest.raises(tt.TTException):
        tt.avg_pool2d(dev(tt, x[0]), 2, 2, 0)                        # 3-D input
    with pytest.raises(tt.TTException):
        tt.min_pool2d(dev(tt, x), 2, 0, 0)                           # stride 0
    with pytest.raises(tt.TTException):
        tt.min_pool2d(dev(tt, x), 2, 1, -1)                          # negative padding
    with pytest.raises(tt.TTException):
        tt.max_pool2d(dev(tt, x), 12, 1, 1)                          # window larger than input + padding
    with pytest.raises(tt.TTException):
        tt.pool2d_backward(dev(tt, np.zeros((2, 3, 4, 4), np.int32)), dev(tt, x.astype(np.int32)),
                           dev(tt, np.zeros((2, 3, 4, 4), np.int32)), "max", 3, 2, 1)   # integers have no gradient


def test_linearity_and_unit_mass_at_full_size(tt):
    # size-independent properties on a large tensor (64 x 64 x 112 x 112 f32, 205 MB)
    rng = np.random.default_rng(3)
    x = rng.normal(size=(64, 64, 112, 112)).astype(np.float32)
    tx = dev(tt, x)
    mx = tt.max_pool2d(tx, 2, 2, 0)
    mn = tt.min_pool2d(tx, 2, 2, 0)
    av = tt.avg_pool2d(tx, 2, 2, 0)
    xm = x.reshape(64, 64, 56, 2, 56, 2)
    assert np.array_equal(mx.to_numpy(), xm.max(axis=(3, 5)))
    assert np.array_equal(mn.to_numpy(), xm.min(axis=(3, 5)))
    assert np.allclose(av.to_numpy(), xm.mean(axis=(3, 5)), rtol=0, atol=1e-6)
    ones = tt.Tensor.from_numpy(np.ones(mx.shape, np.float32))
    gmax = tt.pool2d_backward(ones, tx, mx, "max", 2, 2, 0).to_numpy()
    assert gmax.sum(dtype=np.float64) == mx.numel()            # one unit of gradient per window
    assert np.array_equal(gmax != 0, x == np.repeat(np.repeat(mx.to_numpy(), 2, 2), 2, 3))
    gavg = tt.pool2d_backward(ones, tx, av, "avg", 2, 2, 0).to_numpy()
    assert np.array_equal(gavg, np.full_like(x, 0.25))
