"""The reference's own hot-path tests that need libtorch (TT_TORCH), at their own sizes, on the HIP path.

tests/test_matmul_autograd.cpp:43-261 (f64, data U(-5, 5) from mt19937(0): dot product of 2048, 379 . [379 x 635],
[379 x 635] . [635], [379 x 1147] . [1147 x 635] and the batch of 4 of those; forward and both gradients),
tests/test_conv.cpp:147-183 (f32 [4,3,68,28] * [128,3,3,3] + bias, stride 2, padding 1, integer data in [-5, 5]) and
tests/test_conv_autograd.cpp:43-106 (f64 [4,3,38,28] * [64,3,3,3] + bias, stride 2, padding 1, data U(-1, 1), all three
gradients).  The reference compares with torch; here the expected values come from the CPU oracle, which
tests/test_oracle_torch.py pins against torch's CPU operators on these same shapes.  Tolerances are the reference's:
allclose(atol, rtol 1e-5) with atol 1e-6 for the matmul gradients (1e-4 for the dot product), 1e-6 for the conv forward,
1e-4 for the conv gradients -- element-wise for all three, not only the mean difference the reference settles for on
grad_input."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def allclose(a, b, atol, rtol=1e-5):
    # include/tt/tensor.h:3396-3398: |a - b| <= atol + rtol * |b|
    return a.shape == b.shape and bool(np.all(np.abs(a - b) <= atol + rtol * np.abs(b)))


def rand_vec(gen, n, dtype, low=-5.0, high=5.0):
    """rand_vec of the reference tests: single-precision uniforms from a Mersenne twister, cast to T."""
    return gen.uniform(low, high, n).astype(np.float32).astype(dtype)


def lifted(a, b):
    """The 3-D operands tinytensor::matmul makes of 1-D / 2-D ones (tensor/tensor.cpp:2390-2484)."""
    a3 = a.reshape(1, 1, -1) if a.ndim == 1 else a.reshape((1,) + a.shape) if a.ndim == 2 else a
    b3 = b.reshape(1, -1, 1) if b.ndim == 1 else b.reshape((1,) + b.shape) if b.ndim == 2 else b
    return a3, b3


CASES = {
    "dot_2048": ((2048,), (2048,), 1e-4),
    "dot_12": ((12,), (12,), 1e-4),
    "vector_matrix": ((379,), (379, 635), 1e-6),
    "matrix_vector": ((379, 635), (635,), 1e-6),
    "matrix_matrix": ((379, 1147), (1147, 635), 1e-6),
    "batched": ((4, 379, 1147), (4, 1147, 635), 1e-6),
}


@pytest.mark.parametrize("case", list(CASES))
def test_matmul_autograd_cases_at_reference_size(tt, oracle, case):
    shape_l, shape_r, atol = CASES[case]
    gen = np.random.RandomState(0)                      # MT19937, seed 0
    lhs = rand_vec(gen, int(np.prod(shape_l)), np.float64).reshape(shape_l)
    rhs = rand_vec(gen, int(np.prod(shape_r)), np.float64).reshape(shape_r)
    l3, r3 = lifted(lhs, rhs)
    want = oracle.batched_matmul(l3, r3)
    grad = rand_vec(gen, want.size, np.float64).reshape(want.shape)
    want_l, want_r = oracle.matmul_backward(l3, r3, grad)
    t_l, t_r = tt.Tensor.from_numpy(lhs), tt.Tensor.from_numpy(rhs)
    out = tt.matmul(t_l, t_r)                           # the frontend's own rank lift
    assert allclose(out.to_numpy().reshape(want.shape), want, atol)
    # backward as autograd runs it: on the lifted operands, through permute views (autograd/binary_ops.cpp:173-179)
    got_l, got_r = tt.matmul_backward(tt.Tensor.from_numpy(l3), tt.Tensor.from_numpy(r3), tt.Tensor.from_numpy(grad))
    assert got_l.shape == l3.shape and got_r.shape == r3.shape
    assert allclose(got_l.to_numpy(), want_l, atol)
    assert allclose(got_r.to_numpy(), want_r, atol)
    # the north-star bar as well: K-scaled relative error <= 1e-12 in f64
    scale = np.abs(l3) @ np.abs(r3)
    assert np.max(np.abs(out.to_numpy().reshape(want.shape) - want) / scale) <= 1e-12


def test_conv_forward_with_bias_at_reference_size(tt, oracle):
    # tests/test_conv.cpp:147-183; its rand_vec draws integers in [-5, 5] (uniform_int_distribution), so f32 is exact
    gen = np.random.RandomState(0)
    B, C, O, H, W, k, S, P = 4, 3, 128, 68, 28, 3, 2, 1
    x = gen.randint(-5, 6, (B, C, H, W)).astype(np.float32)
    w = gen.randint(-5, 6, (O, C, k, k)).astype(np.float32)
    bias = gen.randint(-5, 6, O).astype(np.float32)
    want = oracle.conv2d_forward(x, w, bias, S, P)
    got = tt.conv2d(tt.Tensor.from_numpy(x), tt.Tensor.from_numpy(w), tt.Tensor.from_numpy(bias), S, P).to_numpy()
    assert got.shape == (B, O, 34, 14)
    assert allclose(got, want, 1e-6)
    assert np.array_equal(got, want)
    # and on real-valued data of the same shape
    xr, wr, br = (rand_vec(gen, a.size, np.float32).reshape(a.shape) for a in (x, w, bias))
    got = tt.conv2d(tt.Tensor.from_numpy(xr), tt.Tensor.from_numpy(wr), tt.Tensor.from_numpy(br), S, P).to_numpy()
    want = oracle.conv2d_forward(xr, wr, br, S, P)
    scale = oracle.conv2d_forward(np.abs(xr), np.abs(wr), np.abs(br), S, P)
    assert np.max(np.abs(got - want) / scale) <= 1e-4             # the f32 bar, K-scaled


def test_conv_autograd_at_reference_size(tt, oracle):
    # tests/test_conv_autograd.cpp:43-106
    gen = np.random.RandomState(0)
    B, C, O, H, W, k, S, P = 4, 3, 64, 38, 28, 3, 2, 1
    Ho, Wo = (H + 2 * P - k) // S + 1, (W + 2 * P - k) // S + 1
    x = rand_vec(gen, B * C * H * W, np.float64, -1.0, 1.0).reshape(B, C, H, W)
    w = rand_vec(gen, O * C * k * k, np.float64, -1.0, 1.0).reshape(O, C, k, k)
    bias = rand_vec(gen, O, np.float64, -1.0, 1.0)
    grad = rand_vec(gen, B * O * Ho * Wo, np.float64, -1.0, 1.0).reshape(B, O, Ho, Wo)
    t_x, t_w, t_b, t_g = (tt.Tensor.from_numpy(a) for a in (x, w, bias, grad))
    out = tt.conv2d(t_x, t_w, t_b, S, P)
    assert allclose(out.to_numpy(), oracle.conv2d_forward(x, w, bias, S, P), 1e-6)
    gx, gw, gb = tt.conv2d_backward(t_g, t_x, t_w, t_b, S, P)
    want_x, want_w, want_b = oracle.conv2d_backward(grad, x, w, True, S, P)
    assert float(np.abs(gx.to_numpy() - want_x).mean()) < 0.001   # the reference's own criterion for grad_input
    assert allclose(gx.to_numpy(), want_x, 1e-4)                   # ... and element-wise
    assert allclose(gw.to_numpy(), want_w, 1e-4)
    assert allclose(gb.to_numpy(), want_b, 1e-4)
    # f64 bar of this repository: 1e-12 of the K-scaled magnitude
    sx, sw, sb = oracle.conv2d_backward(np.abs(grad), np.abs(x), np.abs(w), True, S, P)
    assert np.max(np.abs(gx.to_numpy() - want_x) / np.maximum(sx, 1e-300)) <= 1e-12
    assert np.max(np.abs(gw.to_numpy() - want_w) / sw) <= 1e-12
    assert np.max(np.abs(gb.to_numpy() - want_b) / sb) <= 1e-12
