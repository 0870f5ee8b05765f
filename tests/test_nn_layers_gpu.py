"""nn::Conv2d and nn::Linear on the device (nn/conv2d.cpp:20-81, nn/linear.cpp:20-50): default initialisation bit-equal
to the CPU oracle's, in-place draws through strided views, forward against the oracle."""
import numpy as np
import pytest

from helpers import max_rel_error

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_in_place_draws_through_views_match_the_cpu_generator(tt, oracle, dtype):
    code = tt._capi.F32 if dtype == np.float32 else tt._capi.F64
    base_h = np.full((5, 4, 3, 6), -7.0, dtype=dtype)
    base_d = tt.Tensor.from_numpy(base_h)
    # permuted, sliced through an offset: shape [3,5,3,6] of a [5,4,3,6] storage, first index of dim 1 skipped
    view_h = base_h.transpose(1, 0, 2, 3)[1:]
    view_d = tt.Tensor(base_d.storage, code, (3, 5, 3, 6), (18, 72, 6, 1), 18)
    g_dev, g_cpu = tt.Generator(3), oracle.Generator(3)
    view_d.uniform_real_(-0.5, 0.25, g_dev)
    g_cpu.uniform_real_(view_h, -0.5, 0.25)
    assert np.array_equal(base_d.to_numpy(), base_h)  # drawn elements and the untouched ones
    assert g_dev.state.value == g_cpu.state
    # normal_ through the same view: same elements touched, values within the two math libraries' rounding
    view_d.normal_(0.0, 0.1, g_dev)
    got = base_d.to_numpy()
    assert np.array_equal(got[:, 0], base_h[:, 0])
    want = oracle.Generator(3)
    want.uniform_real(-1, 1, (view_h.size,), dtype)  # skip what the uniform draw consumed
    z = want.normal(0.0, 0.1, view_h.shape, dtype)
    assert np.max(np.abs(got.transpose(1, 0, 2, 3)[1:] - z)) <= (2e-6 if dtype == np.float32 else 1e-13)
    with pytest.raises(tt.TTException):
        tt.Tensor.from_numpy(np.zeros(4, np.int32)).uniform_real_(0.0, 1.0, g_dev)
    with pytest.raises(tt.TTException):
        view_d.uniform_real_(1.0, 1.0, g_dev)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_draws_with_parameter_tensors_match_the_cpu_generator(tt, oracle, dtype):
    """uniform_real_ / normal_ with a parameter pair per element (backend_base.h:96-103, cuda/distribution.cu:32-99):
    non-constant `high` / `std`, parameters given as a dense tensor, as a permuted view and as a value expanded with
    stride 0, the result written through a permuted view with an offset."""
    code = tt._capi.F32 if dtype == np.float32 else tt._capi.F64
    rng = np.random.default_rng(8)
    base_h = np.full((4, 6, 5), -7.0, dtype=dtype)
    base_d = tt.Tensor.from_numpy(base_h)
    view_h = base_h.transpose(1, 0, 2)[1:, :, 1:4]                               # [5,4,3]
    view_d = tt.Tensor(base_d.storage, code, (5, 4, 3), (5, 30, 1), 6)
    low = rng.uniform(-2.0, 1.0, (5, 4, 3)).astype(dtype)
    high_src = (low.transpose(2, 0, 1) + rng.uniform(0.1, 3.0, (3, 5, 4))).astype(dtype)   # stored as [3,5,4]
    high = high_src.transpose(1, 2, 0)                                             # the [5,4,3] view of it
    t_low = tt.Tensor.from_numpy(low)
    t_high = tt.Tensor.from_numpy(np.ascontiguousarray(high_src)).permute(1, 2, 0)
    assert not t_high.is_contiguous()
    g_dev, g_cpu = tt.Generator(13), oracle.Generator(13)
    view_d.uniform_real_(t_low, t_high, g_dev)
    g_cpu.draw_params_(view_h, 0, low, high)
    assert np.array_equal(base_d.to_numpy(), base_h)                              # bit construction + one fma: exact
    assert g_dev.state.value == g_cpu.state
    # normal: mu one value expanded over the shape (stride 0), std per element
    std = rng.uniform(0.05, 2.0, (5, 4, 3)).astype(dtype)
    t_mu = tt.Tensor.from_numpy(np.array([[[0.25]]], dtype=dtype)).expand((5, 4, 3))
    view_d.normal_(t_mu, tt.Tensor.from_numpy(std), g_dev)
    g_cpu.draw_params_(view_h, 1, np.array(0.25, dtype=dtype), std)
    got = base_d.to_numpy()
    assert np.array_equal(got[:, 0], base_h[:, 0]) and np.array_equal(got[:, :, 0], base_h[:, :, 0])   # untouched elements
    assert np.max(np.abs(got - base_h)) <= (2e-5 if dtype == np.float32 else 1e-12)  # |z| <= ~6, std <= 2: libm rounding
    assert g_dev.state.value == g_cpu.state
    with pytest.raises(tt.TTException):
        view_d.uniform_real_(t_low, tt.Tensor.from_numpy(np.zeros((5, 4), dtype=dtype)), g_dev)   # shapes must agree


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_conv2d_default_init_equals_cpu_init(tt, oracle, dtype):
    code = tt._capi.F32 if dtype == np.float32 else tt._capi.F64
    g_dev, g_cpu = tt.Generator(0), oracle.Generator(0)
    for cin, cout, k, bias in ((32, 64, 3, True), (3, 8, 5, True), (1, 32, 3, False)):
        layer = tt.Conv2d(cin, cout, k, 1, 1, bias=bias, dtype=code, gen=g_dev)
        W, b = oracle.conv2d_init(g_cpu, cin, cout, k, bias=bias, dtype=dtype)
        assert layer.weight.shape == (cout, cin, k, k) and layer.weight.is_contiguous()
        assert np.array_equal(layer.weight.to_numpy(), W)
        if bias:
            assert np.array_equal(layer.bias.to_numpy(), b)
        else:
            assert layer.bias is None
        assert g_dev.state.value == g_cpu.state


def test_conv2d_layer_forward_on_config4_input(tt, oracle):
    # Conv2d(32, 64, 3, stride 1, padding 1) with its default init on the benchmark's input [64,32,28,28] ~ N(0, 0.1)
    tt.set_default_generator_seed(0)
    layer = tt.Conv2d(32, 64, 3, 1, 1)  # draws from the default generator, like the reference's constructor
    W, b = oracle.conv2d_init(oracle.Generator(0), 32, 64, 3)
    assert np.array_equal(layer.weight.to_numpy(), W) and np.array_equal(layer.bias.to_numpy(), b)
    x = oracle.Generator(5).normal(0.0, 0.1, (64, 32, 28, 28))
    got = layer(tt.Tensor.from_numpy(x)).to_numpy()
    want = oracle.conv2d_forward(x, W, b, 1, 1)
    assert got.shape == (64, 64, 28, 28)
    assert max_rel_error(got, want) <= 1e-4
    with pytest.raises(tt.TTException):
        layer(tt.Tensor.from_numpy(np.zeros((1, 31, 28, 28), np.float32)))
    for bad in ((0, 4, 3, 1, 0), (4, 0, 3, 1, 0), (4, 4, 0, 1, 0), (4, 4, 3, 0, 0), (4, 4, 3, 1, -1)):
        with pytest.raises(tt.TTException):
            tt.Conv2d(*bad)


def test_linear_layer_default_init_and_forward(tt, oracle):
    g_dev, g_cpu = tt.Generator(2), oracle.Generator(2)
    layer = tt.Linear(784, 96, gen=g_dev)
    W, b = oracle.linear_init(g_cpu, 784, 96)
    assert np.array_equal(layer.weight.to_numpy(), W) and np.array_equal(layer.bias.to_numpy(), b)
    x = oracle.Generator(8).uniform_real(0.0, 1.0, (50, 784))
    got = layer(tt.Tensor.from_numpy(x)).to_numpy()
    want = oracle.matmul(x, W) + b[None, :]
    assert max_rel_error(got, want) <= 1e-4


def test_integer_and_bool_sums_are_64_bit(tt):
    # common/reduce.h:56-61: sums of the integer dtypes (and bool) accumulate in int64 and return I64
    rng = np.random.default_rng(0)
    for np_dt in (np.uint8, np.int16, np.int32, np.int64):
        hi = min(np.iinfo(np_dt).max, 2**40)
        a = rng.integers(hi // 2, hi, (300, 257), dtype=np_dt)
        t = tt.Tensor.from_numpy(a)
        total = t.sum()
        assert total.dtype == tt._capi.I64
        assert int(total.to_numpy()[0]) == int(a.astype(np.int64).sum())          # far beyond the input type's range
        for dim in (0, 1):
            s = t.sum(dim)
            assert s.dtype == tt._capi.I64 and np.array_equal(s.to_numpy(), a.astype(np.int64).sum(axis=dim))
        big = tt.Tensor.from_numpy(rng.integers(0, min(hi, 200), (70000,), dtype=np_dt))  # two-stage path
        assert int(big.sum().to_numpy()[0]) == int(big.to_numpy().astype(np.int64).sum())
    m = rng.random((1000, 130)) < 0.3
    tm = tt.Tensor.from_numpy(m)
    assert tm.dtype == tt._capi.BOOL
    assert tm.sum().dtype == tt._capi.I64 and int(tm.sum().to_numpy()[0]) == int(m.sum())
    assert np.array_equal(tm.sum(0).to_numpy(), m.sum(axis=0).astype(np.int64))
    assert np.array_equal(tm.permute(1, 0).sum(0).to_numpy(), m.sum(axis=1).astype(np.int64))   # strided view
    f = tt.Tensor.from_numpy(np.ones((4, 5), np.float32))
    assert f.sum().dtype == tt._capi.F32 and f.sum(1).dtype == tt._capi.F32


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_draws_from_caller_supplied_states(tt, oracle, dtype):
    """ttamd_random_fill_states: the caller draws one generator state per element (cpu/distribution.cpp:31-38) and the
    device writes element i of the view from state i -- the same values as the call that draws the states itself."""
    import ctypes as C
    code = tt._capi.F32 if dtype == np.float32 else tt._capi.F64
    lib = tt._capi.lib
    shape, stride, offset = (3, 5, 2), (2, 6, 1), 1           # a permuted view with an offset into 31 stored elements
    n = int(np.prod(shape))
    for dist, p0, p1 in ((0, -0.5, 0.25), (1, 0.0, 0.1)):
        gen = oracle.Generator(11)
        states = (C.c_uint64 * n)(*[gen() for _ in range(n)])  # Generator::operator(), element order = the view's row-major order
        by_states = tt.Tensor.from_numpy(np.full(31, -7.0, dtype=dtype))
        rc = lib.ttamd_random_fill_states(0, code, dist, p0, p1, states, 3, (C.c_int64 * 3)(*shape), (C.c_int64 * 3)(*stride),
                                          C.c_void_p(by_states.storage.ptr), offset, None)
        assert rc == 0, tt._capi.last_error()
        by_master = tt.Tensor.from_numpy(np.full(31, -7.0, dtype=dtype))
        view = tt.Tensor(by_master.storage, code, shape, stride, offset)
        g_dev = tt.Generator(11)
        (view.uniform_real_ if dist == 0 else view.normal_)(p0, p1, g_dev)
        assert g_dev.state.value == gen.state                  # both consumed n outputs
        assert np.array_equal(by_states.to_numpy(), by_master.to_numpy())
        assert np.count_nonzero(by_states.to_numpy() != -7.0) == n
    if dtype == np.float32:
        rc = lib.ttamd_random_fill_states(0, tt._capi.I32, 0, 0.0, 1.0, states, 3, (C.c_int64 * 3)(*shape), (C.c_int64 * 3)(*stride),
                                          C.c_void_p(by_states.storage.ptr), offset, None)
        assert rc != 0                                          # floating point dtypes only
