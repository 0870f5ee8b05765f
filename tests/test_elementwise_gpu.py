"""GPU tests of the elementwise / reduction set around the GEMMs (ttamd_binary, ttamd_unary, ttamd_where, ttamd_sum,
ttamd_full) and of a whole MLP training step that never leaves the device between its GEMMs.

Oracles: numpy for the arithmetic (IEEE add/sub/mul/div and integer wrap-around are exact and identical), a
sequential sum for the reductions (the reference's reduce kernel order), the CPU oracle's GEMM for the MLP step.
Bars: exact for integer dtypes, for +,-,*,/ and comparisons on floats, relu, where, full; <= 1e-6 (f32) /
1e-14 (f64) relative for transcendental functions; <= 1e-5 relative for float sums (different association)."""
import numpy as np
import pytest

from helpers import ALL_NON_BOOL, max_rel_error, mlp_train_step

pytestmark = pytest.mark.gpu


def dev(tt, a):
    return tt.Tensor.from_numpy(a)


@pytest.mark.parametrize("dtype", ALL_NON_BOOL)
def test_binary_ops_exact(tt, dtype):
    rng = np.random.default_rng(1)
    if np.issubdtype(dtype, np.floating):
        a = rng.uniform(-4, 4, (7, 33, 5)).astype(dtype)
        b = rng.uniform(0.5, 4, (7, 33, 5)).astype(dtype)
    else:
        hi = 100 if dtype == np.uint8 else 1000
        a = rng.integers(0 if dtype == np.uint8 else -hi, hi, (7, 33, 5)).astype(dtype)
        b = rng.integers(1, 9, (7, 33, 5)).astype(dtype)
    ta, tb = dev(tt, a), dev(tt, b)
    be = tt.get_backend(tt.kAMD)
    with np.errstate(over="ignore"):
        assert np.array_equal((ta + tb).to_numpy(), (a + b).astype(dtype))
        assert np.array_equal((ta - tb).to_numpy(), (a - b).astype(dtype))
        assert np.array_equal((ta * tb).to_numpy(), (a * b).astype(dtype))   # integers wrap modulo 2^n on both sides
    if np.issubdtype(dtype, np.floating):
        assert np.array_equal((ta / tb).to_numpy(), a / b)
        assert np.array_equal(ta.pow(2.0).to_numpy(), a * a)
        assert max_rel_error(tb.pow(tb).to_numpy(), np.power(b, b)) <= (1e-6 if dtype == np.float32 else 1e-14)
    else:
        assert np.array_equal((ta / tb).to_numpy(), (a.astype(np.int64) // b.astype(np.int64) if dtype == np.uint8 else
                                                    np.trunc(a.astype(np.float64) / b).astype(np.int64)).astype(dtype))
    for op, fn in (("lt", np.less), ("le", np.less_equal), ("gt", np.greater), ("ge", np.greater_equal),
                   ("eq", np.equal), ("ne", np.not_equal), ("maximum", np.maximum), ("minimum", np.minimum)):
        got = be.binary(ta, tb, op).to_numpy()
        assert np.array_equal(got, fn(a, b))


def test_binary_on_strided_and_broadcast_views(tt):
    rng = np.random.default_rng(2)
    a = rng.uniform(-1, 1, (6, 8)).astype(np.float32)
    row = rng.uniform(-1, 1, (8,)).astype(np.float32)
    ta = dev(tt, a)
    assert np.array_equal((ta.permute(1, 0) + dev(tt, np.ascontiguousarray(a.T))).to_numpy(), a.T + a.T)
    assert np.array_equal((ta + dev(tt, row)).to_numpy(), a + row)            # bias-style broadcast (stride 0)
    assert np.array_equal((ta * 2.5).to_numpy(), a * np.float32(2.5))         # scalar operand
    assert np.array_equal((ta < 0.0).to_numpy(), a < 0)
    w = tt.where(ta < 0.0, 0.0, 1.0)                                          # relu-backward mask of the reference
    assert np.array_equal(w.to_numpy(), np.where(a < 0, np.float32(0), np.float32(1)))
    with pytest.raises(tt.TTException):
        ta + dev(tt, np.zeros((5,), np.float32))


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.uint8])
@pytest.mark.parametrize("shape", [(1024, 1024), (7, 13), (3,), (257, 5)])
def test_scalar_operands_take_the_splat_kernels(tt, dtype, shape):
    # tensor (op) scalar and where(mask, scalar, scalar | tensor): one operand is a single element with every stride 0;
    # sizes with and without a tail behind the 16-byte vectors
    rng = np.random.default_rng(sum(shape))
    a = rng.integers(0, 7, shape).astype(dtype)
    b = rng.integers(0, 7, shape).astype(dtype)
    ta, tb = dev(tt, a), dev(tt, b)
    two = dtype(2)
    assert np.array_equal((ta + 2).to_numpy(), a + two)
    assert np.array_equal((ta * 2).to_numpy(), a * two)
    assert np.array_equal((ta - 2).to_numpy(), (a - two).astype(dtype))
    assert np.array_equal((ta < 3).to_numpy(), a < 3)
    mask = ta < 3
    assert np.array_equal(tt.where(mask, 0, 1).to_numpy(), np.where(a < 3, dtype(0), dtype(1)))
    assert np.array_equal(tt.where(mask, tb, 5).to_numpy(), np.where(a < 3, b, dtype(5)))
    assert np.array_equal(tt.where(mask, 5, tb).to_numpy(), np.where(a < 3, dtype(5), b))
    # scalar on the left of a non-commutative op
    s = dev(tt, np.full((1,) * len(shape), 9, dtype=dtype)).expand(shape)
    assert np.array_equal((s - ta).to_numpy(), (dtype(9) - a).astype(dtype))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_unary_ops(tt, dtype):
    rng = np.random.default_rng(3)
    a = rng.uniform(-3, 3, (5, 77)).astype(dtype)
    ta, be = dev(tt, a), tt.get_backend(tt.kAMD)
    tol = 1e-6 if dtype == np.float32 else 1e-14
    assert np.array_equal(ta.relu().to_numpy(), np.maximum(a, 0))
    assert np.array_equal(be.unary(ta, "negate").to_numpy(), -a)
    assert np.array_equal(be.unary(ta, "abs").to_numpy(), np.abs(a))
    pos = dev(tt, np.abs(a) + dtype(0.1))
    assert np.array_equal(be.unary(pos, "sqrt").to_numpy(), np.sqrt(np.abs(a) + dtype(0.1)))  # correctly rounded
    assert max_rel_error(be.unary(ta, "exp").to_numpy(), np.exp(a)) <= tol
    assert max_rel_error(be.unary(pos, "log").to_numpy(), np.log(np.abs(a) + dtype(0.1))) <= tol
    assert max_rel_error(be.unary(ta, "tanh").to_numpy(), np.tanh(a)) <= tol
    assert max_rel_error(be.unary(ta, "sigmoid").to_numpy(), 1 / (1 + np.exp(-a))) <= tol
    # relu on a permuted view
    assert np.array_equal(ta.permute(1, 0).relu().to_numpy(), np.maximum(a.T, 0))


@pytest.mark.parametrize("dtype", [np.int32, np.float32, np.float64])
def test_sum_and_full(tt, dtype):
    rng = np.random.default_rng(4)
    a = rng.integers(-50, 50, (9, 130, 17)).astype(dtype)  # integer-valued: every order of summation is exact
    ta = dev(tt, a)
    for d in range(3):
        assert np.array_equal(ta.sum(d).to_numpy(), a.sum(axis=d, dtype=dtype))
    assert ta.sum().to_numpy()[0] == a.sum(dtype=dtype)
    assert np.array_equal(ta.permute(2, 0, 1).sum(1).to_numpy(), a.transpose(2, 0, 1).sum(axis=1, dtype=dtype))
    big = rng.integers(-5, 5, (300000,)).astype(dtype)     # two-stage path
    assert dev(tt, big).sum().to_numpy()[0] == big.sum(dtype=dtype)
    f = tt.full((3, 4), 7, tt._capi.I32 if dtype == np.int32 else (tt._capi.F32 if dtype == np.float32 else tt._capi.F64))
    assert f.stride == (0, 0) and np.array_equal(f.to_numpy(), np.full((3, 4), 7, dtype))
    if np.issubdtype(dtype, np.floating):
        x = rng.uniform(-1, 1, (100, 1000)).astype(dtype)
        seq = np.zeros(1000, dtype=dtype)
        for r in x:                                         # the reference's order: sequential over the reduced dim
            seq = seq + r
        got = dev(tt, x).sum(0).to_numpy()
        assert np.array_equal(got, seq)                     # short dimension: same order, same IEEE additions
        # long reduced dimension with few outputs: sliced / wavefront-parallel forms, fixed order but not sequential
        y = rng.uniform(-1, 1, (1024, 1000)).astype(dtype)
        tol = (1e-5 if dtype == np.float32 else 1e-13) * 1024
        assert np.max(np.abs(dev(tt, y).sum(0).to_numpy() - y.sum(0, dtype=np.float64))) <= tol
        assert np.max(np.abs(dev(tt, y).sum(1).to_numpy() - y.sum(1, dtype=np.float64))) <= tol
        assert np.max(np.abs(dev(tt, y).permute(1, 0).sum(0).to_numpy() - y.sum(1, dtype=np.float64))) <= tol
        yi = np.round(y * 8)                                 # multiples of 1/8: exact in any order
        assert np.array_equal(dev(tt, yi).sum(0).to_numpy(), yi.sum(0))
        assert np.array_equal(dev(tt, yi).sum(1).to_numpy(), yi.sum(1))
        assert np.array_equal(dev(tt, yi[:, :7]).sum(0).to_numpy(), yi[:, :7].sum(0))   # fewer outputs than one block
        assert abs(float(dev(tt, x).mean().to_numpy()[0]) - float(x.mean(dtype=np.float64))) <= 1e-5


def mlp_step_on_device(tt, X, T, params):
    """The training step of benchmark configuration 5 with every op on the device: fused Linear(+bias) GEMMs, relu, mse_loss
    as pow(y - t, 2).mean(), and the backward pass op for op as the reference's autograd emits it
    (autograd/unary_ops.cpp:568-573, binary_ops.cpp:173-179, reduce_ops.cpp:201-205; bias grads = sum over dim 0)."""
    d = lambda a: tt.Tensor.from_numpy(a)
    x, t = d(X), d(T)
    (W1, b1), (W2, b2), (W3, b3) = [(d(W), d(b)) for W, b in params]
    z1 = tt.linear(x, W1, b1)
    a1 = z1.relu()
    z2 = tt.linear(a1, W2, b2)
    a2 = z2.relu()
    y = tt.linear(a2, W3, b3)
    diff = y - t
    loss = diff.pow(2.0).mean()
    gy = tt.full(y.shape, 1.0 / y.numel() * 2.0, y.dtype) * diff          # ((1/N) * 2) * (y - t)
    out = {"y": y, "loss": loss, "db3": gy.sum(0)}
    da2, out["dW3"] = tt.matmul_backward(a2.unsqueeze(0), W3.unsqueeze(0), gy.unsqueeze(0))
    m2 = tt.where(z2 < 0.0, 0.0, 1.0)
    dz2 = da2.squeeze(0) * m2
    out["db2"] = dz2.sum(0)
    da1, out["dW2"] = tt.matmul_backward(a1.unsqueeze(0), W2.unsqueeze(0), dz2.unsqueeze(0))
    m1 = tt.where(z1 < 0.0, 0.0, 1.0)
    dz1 = da1.squeeze(0) * m1
    out["db1"] = dz1.sum(0)
    out["dX"], out["dW1"] = tt.matmul_backward(x.unsqueeze(0), W1.unsqueeze(0), dz1.unsqueeze(0))
    res = {k: v.to_numpy() for k, v in out.items()}
    for k in ("dW1", "dW2", "dW3", "dX"):
        res[k] = res[k][0]
    res["loss"] = res["loss"][0]
    res["masks"] = (m1.to_numpy(), m2.to_numpy())
    return res


def test_mlp_training_step_entirely_on_device(tt, oracle):
    X = oracle.Generator(0).uniform_real(0.0, 1.0, (1024, 784))
    T = oracle.Generator(1).uniform_real(0.0, 1.0, (1024, 10))
    g = oracle.Generator(0)
    params = [oracle.linear_init(g, a, b) for a, b in ((784, 1024), (1024, 1024), (1024, 10))]
    got = mlp_step_on_device(tt, X, T, params)
    cpu = lambda masks: mlp_train_step(X, T, params, lambda a, b: oracle.matmul(a, b),
                                       lambda a, b, gr: tuple(v[0] for v in oracle.matmul_backward(a[None], b[None], gr[None])),
                                       masks=masks)
    want = cpu(got["masks"])          # same ReLU masks on both sides (a step function of z; see helpers.mlp_train_step)
    own = cpu(None)
    assert sum(int(np.sum(a != b)) for a, b in zip(got["masks"], own["masks"])) <= 8
    for key in ("y", "dW1", "db1", "dW2", "db2", "dW3", "db3", "dX"):
        assert got[key].shape == want[key].shape
        assert max_rel_error(got[key], want[key]) <= 1e-4, key
    assert abs(float(got["loss"]) - float(want["loss"])) <= 1e-4 * abs(float(want["loss"]))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_seeded_draws_match_the_cpu_generator(tt, oracle, dtype):
    code = tt._capi.F32 if dtype == np.float32 else tt._capi.F64
    g_dev, g_cpu = tt.Generator(0), oracle.Generator(0)
    assert g_dev.state.value == g_cpu.state
    a = tt.uniform_real(-1.0, 1.0, (300, 17), g_dev, code).to_numpy()
    assert np.array_equal(a, g_cpu.uniform_real(-1.0, 1.0, (300, 17), dtype))       # integer bit construction + one fma: exact
    assert g_dev.state.value == g_cpu.state                                         # master generator advanced identically
    b = tt.normal(0.0, 0.1, (5000,), g_dev, code).to_numpy()
    want = g_cpu.normal(0.0, 0.1, (5000,), dtype)
    assert g_dev.state.value == g_cpu.state
    # Box-Muller goes through log1p / sqrt / sin of two different math libraries: tolerance, not bits
    assert np.max(np.abs(b - want)) <= (2e-6 if dtype == np.float32 else 1e-13)
    with pytest.raises(tt.TTException):
        tt.uniform_real(1.0, 1.0, (4,), g_dev, code)


def test_linear_default_init_on_device_equals_cpu_init(tt, oracle):
    g_dev, g_cpu = tt.Generator(0), oracle.Generator(0)
    for fan_in, fan_out in ((784, 1024), (1024, 10)):
        W, b = tt.linear_init(fan_in, fan_out, g_dev)
        Wc, bc = oracle.linear_init(g_cpu, fan_in, fan_out)
        assert np.array_equal(W.to_numpy(), Wc) and np.array_equal(b.to_numpy(), bc)


def test_binary_ops_promote_mixed_dtypes(tt):
    """Binary operators cast their operands to promote_types(lhs, rhs) (tensor/tensor.cpp:2272-2274): the ReLU mask
    where(z < 0, 0, 1) is f32 by default and multiplies an f64 gradient as f64."""
    z = np.array([[-1.5, 0.0, 2.25], [3.0, -0.5, 1.0]])
    tz = tt.Tensor.from_numpy(z)
    mask = tt.where(tz < 0.0, 0.0, 1.0)
    assert mask.dtype == tt._capi.F32
    prod = tz * mask
    assert prod.dtype == tt._capi.F64 and np.array_equal(prod.to_numpy(), z * (z >= 0))
    i = tt.Tensor.from_numpy(np.array([1, 2, 3], dtype=np.int32))
    f = tt.Tensor.from_numpy(np.array([0.5, 0.25, 2.0], dtype=np.float32))
    assert np.array_equal((i + f).to_numpy(), np.array([1.5, 2.25, 5.0], dtype=np.float32))
