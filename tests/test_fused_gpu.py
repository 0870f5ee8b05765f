"""The fused forms around a Linear layer's GEMMs: second output max(out, 0) (Linear + ReLU), the ReLU-backward mask and
the bias gradient's column sums in the store of the GEMM that computes grad_output, mse_loss with its backward in one
pass, and the whole MLP training step of benchmark configuration 5 built from them.  Each piece is compared with numpy on
integer-valued data (exact in any summation order) for every kernel family that can carry it, then the whole step with
the CPU oracle at the benchmark's size."""
import ctypes as C

import numpy as np
import pytest

from helpers import max_rel_error, mlp_train_step

pytestmark = pytest.mark.gpu

# (B, N, K, M): small-tile plain, ragged with odd M (no paired stores), two halves of k, a small output, split k, 128 x 128, 192 x 192,
# 256 x 256 / 256 x 128 tiles, K = 10 (the skinny backward product of configuration 5), element-wise gathers
SHAPES = [(1, 200, 96, 136), (2, 130, 70, 151), (1, 1024, 1024, 1024), (1, 256, 512, 256), (1, 320, 512, 416), (1, 2048, 64, 2048),
          (1, 3072, 32, 3072), (1, 4096, 32, 4096), (1, 1024, 10, 1024), (3, 70, 50, 90),
          # reductions of at most 16 (their own kernel): ragged rows and columns, rows of 4n and of odd length, one to four
          # tiles per wave, several row blocks (the column sums then come from partial rows), batches, k = 1 and k = 16
          (2, 300, 7, 52), (1, 5000, 16, 36), (1, 77, 1, 131), (3, 260, 3, 16), (1, 2500, 10, 1024), (1, 513, 13, 70)]


def _variant(tt, a, b):
    return tt.get_backend(tt.kAMD).batched_matmul_variant(a, b)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", SHAPES)
def test_store_extensions_match_numpy(tt, dtype, shape):
    B, N, K, M = shape
    rng = np.random.default_rng(N + K + M)
    a = rng.integers(-3, 4, (B, N, K)).astype(dtype)
    b = rng.integers(-3, 4, (B, K, M)).astype(dtype)
    bias = rng.integers(-5, 6, (M,)).astype(dtype)
    z = rng.integers(-2, 3, (B, N, M)).astype(dtype)           # the saved input of a ReLU: negatives, zeros, positives
    be = tt.get_backend(tt.kAMD)
    ta, tb, tbias, tz = (tt.Tensor.from_numpy(v) for v in (a, b, bias, z))
    prod = np.matmul(a.astype(np.float64), b.astype(np.float64))
    # 1. Linear + ReLU: out keeps the value before the ReLU, relu_out its positive part
    act = tt.Tensor.empty((B, N, M), ta.dtype)
    out = be.batched_matmul(ta, tb, bias=tbias, bias_mode=1, relu_out=act)
    want = (prod + bias).astype(dtype)
    assert np.array_equal(out.to_numpy(), want), _variant(tt, ta, tb)
    assert np.array_equal(act.to_numpy(), np.maximum(want, 0))
    # 2. ReLU backward mask and column sums in one store
    cs = tt.Tensor.empty((B, M), ta.dtype)
    dz = be.batched_matmul(ta, tb, relu_grad_input=tz, colsum_out=cs)
    want_dz = (prod * np.where(z < 0, 0.0, 1.0)).astype(dtype)
    assert np.array_equal(dz.to_numpy(), want_dz)
    assert np.array_equal(cs.to_numpy(), want_dz.sum(axis=1).astype(dtype))
    # 3. column sums alone, on transposed views (the operands of a backward GEMM)
    at = tt.Tensor.from_numpy(np.ascontiguousarray(a.transpose(0, 2, 1))).permute(0, 2, 1)
    bt = tt.Tensor.from_numpy(np.ascontiguousarray(b.transpose(0, 2, 1))).permute(0, 2, 1)
    cs2 = tt.Tensor.empty((B, M), ta.dtype)
    out2 = be.batched_matmul(at, bt, colsum_out=cs2)
    assert np.array_equal(out2.to_numpy(), prod.astype(dtype))
    assert np.array_equal(cs2.to_numpy(), prod.sum(axis=1).astype(dtype))
    # the plain call is untouched by the extensions
    assert np.array_equal(be.batched_matmul(ta, tb).to_numpy(), prod.astype(dtype))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", [(1, 200, 96, 136), (1, 1024, 1024, 1024), (1, 320, 512, 416), (1, 1024, 10, 1024), (1, 300, 64, 10),
                                   (1, 4096, 32, 4096)])
def test_relu_backward_mask_multiplies_like_the_reference(tt, dtype, shape):
    """TensorRelu::backward is grad_output * where(input < 0, 0, 1) (autograd/unary_ops.cpp:568-573), a product: an
    infinite or NaN gradient under the mask gives NaN.  The fused store does the same (every kernel family: tiles, two
    halves, split k, short reduction, thin output, 256 x 256).  The sign of a masked zero is not kept: the reference
    leaves -0 under a negative gradient, the store's later additions of an absent operand (+0) turn it into +0; the
    two compare equal."""
    B, N, K, M = shape
    rng = np.random.default_rng(N * 3 + K + M)
    a = rng.integers(-3, 4, (B, N, K)).astype(dtype)
    b = rng.integers(-3, 4, (B, K, M)).astype(dtype)
    z = rng.integers(-2, 3, (B, N, M)).astype(dtype)
    a[0, 3, :] = 1
    a[0, 3, 0] = np.inf                                    # row 3 of the product: +-inf, or NaN where b[0, 0, m] is 0
    a[0, N - 1, K - 1] = np.nan                            # last row: NaN everywhere
    z[0, 3, : M // 2] = -1
    z[0, N - 1, ::2] = -1
    be = tt.get_backend(tt.kAMD)
    ta, tb, tz = (tt.Tensor.from_numpy(v) for v in (a, b, z))
    with np.errstate(invalid="ignore"):
        prod = np.matmul(a.astype(np.float64), b.astype(np.float64))
        want = (prod * np.where(z < 0, 0.0, 1.0)).astype(dtype)
    got = be.batched_matmul(ta, tb, relu_grad_input=tz).to_numpy()
    variant = _variant(tt, ta, tb)
    assert np.array_equal(np.isnan(got), np.isnan(want)), variant
    assert np.isnan(want[0, 3, : M // 2]).all() and np.isnan(got[0, N - 1]).all()
    finite = ~np.isnan(want)
    assert np.array_equal(got[finite], want[finite]), variant


def test_store_extension_argument_checks(tt):
    be = tt.get_backend(tt.kAMD)
    a = tt.Tensor.from_numpy(np.ones((1, 8, 8), np.float32))
    good = tt.Tensor.empty((1, 8, 8), tt._capi.F32)
    with pytest.raises(tt.TTException):
        be.batched_matmul(a, a, relu=True, relu_out=good)              # relu_out excludes relu
    with pytest.raises(tt.TTException):
        be.batched_matmul(a, a, accumulate=True, out=good, colsum_out=tt.Tensor.empty((1, 8), tt._capi.F32))
    with pytest.raises(tt.TTException):
        be.batched_matmul(a, a, relu_out=tt.Tensor.empty((1, 8, 4), tt._capi.F32))
    i = tt.Tensor.from_numpy(np.ones((1, 8, 8), np.int32))
    with pytest.raises(tt.TTException):
        be.batched_matmul(i, i, colsum_out=tt.Tensor.empty((1, 8), tt._capi.I32))
    # integer operands do carry the mask and the second output (vector-ALU kernel)
    zi = tt.Tensor.from_numpy(np.array([[[-1, 0, 1, 2, -3, 4, 5, -6]] * 8], np.int32))
    acti = tt.Tensor.empty((1, 8, 8), tt._capi.I32)
    got = be.batched_matmul(i, i, relu_grad_input=zi, relu_out=acti).to_numpy()
    assert np.array_equal(got[0], np.where(zi.to_numpy()[0] < 0, 0, 8)) and np.array_equal(acti.to_numpy(), got)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", [(1024, 10), (7, 3), (50000, 64), (300, 1000), (1, 1), (4096, 33),
                                   (16384, 1), (16385, 1), (256, 64), (257, 64), (1000, 5)])
def test_mse_loss_forward_and_backward(tt, dtype, shape):
    rng = np.random.default_rng(shape[0])
    y = rng.uniform(-1, 1, shape).astype(dtype)
    t = rng.uniform(-1, 1, shape).astype(dtype)
    narrow = shape[1] <= 64
    loss, g, cs = tt.mse_loss(tt.Tensor.from_numpy(y), tt.Tensor.from_numpy(t), grad=True, bias_grad=narrow)
    d = y.astype(np.float64) - t
    tol = 1e-5 if dtype == np.float32 else 1e-13
    assert abs(float(loss.to_numpy()[0]) - np.mean(d * d)) <= tol * np.mean(d * d)
    want_g = (dtype(1) / dtype(y.size) * dtype(2)) * (y - t)       # ((1/N) * 2) * (y - t), the reference's rounding
    assert np.array_equal(g.to_numpy(), want_g)
    if narrow:
        assert np.max(np.abs(cs.to_numpy() - want_g.astype(np.float64).sum(0))) <= tol * np.abs(want_g).sum(0).max()
    else:
        with pytest.raises(tt.TTException):
            tt.mse_loss(tt.Tensor.from_numpy(y), tt.Tensor.from_numpy(t), grad=True, bias_grad=True)
    only_loss, none_g, none_cs = tt.mse_loss(tt.Tensor.from_numpy(y), tt.Tensor.from_numpy(t), grad=False)
    assert none_g is None and none_cs is None and only_loss.to_numpy()[0] == loss.to_numpy()[0]


def fused_mlp_step(tt, x, t, params, own=False):
    """The training step of benchmark configuration 5 from the fused forms: 3 forward launches, the loss with its
    gradient and the head's bias gradient in one, and per layer one GEMM for dx (the ReLU-backward mask in its store) and
    one for dW.  The bias gradients of layers 1 and 2 are column sums of dz: taken in the store of the GEMM that writes
    dz (+ the sum of the partial rows), or (`own`) from the vectors of dz that the layer's dW GEMM stages.  own == "head":
    as `own`, and the last layer, the loss and their backward in one call of two launches."""
    (W1, b1), (W2, b2), (W3, b3) = params
    z1, a1 = tt.linear_relu(x, W1, b1)
    z2, a2 = tt.linear_relu(a1, W2, b2)
    if own == "head":
        y, loss, dz2, dW3, db3 = tt.linear_mse_head(a2, W3, b3, t, relu_input=z2)
        dz1, dW2, db2 = tt.linear_backward(dz2, a1, W2, relu_input=z1, bias_grad="own")
        dX, dW1, db1 = tt.linear_backward(dz1, x, W1, bias_grad="own")
        return dict(y=y, loss=loss, dW1=dW1, db1=db1, dW2=dW2, db2=db2, dW3=dW3, db3=db3, dX=dX, z1=z1, z2=z2)
    y = tt.linear(a2, W3, b3)
    loss, gy, db3 = tt.mse_loss(y, t, grad=True, bias_grad=True)
    if own:
        dz2, dW3, _ = tt.linear_backward(gy, a2, W3, relu_input=z2, bias_grad=False)
        dz1, dW2, db2 = tt.linear_backward(dz2, a1, W2, relu_input=z1, bias_grad="own")
        dX, dW1, db1 = tt.linear_backward(dz1, x, W1, bias_grad="own")
    else:
        dz2, dW3, db2 = tt.linear_backward(gy, a2, W3, relu_input=z2)
        dz1, dW2, db1 = tt.linear_backward(dz2, a1, W2, relu_input=z1)
        dX, dW1, _ = tt.linear_backward(dz1, x, W1, bias_grad=False)
    return dict(y=y, loss=loss, dW1=dW1, db1=db1, dW2=dW2, db2=db2, dW3=dW3, db3=db3, dX=dX, z1=z1, z2=z2)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("a_transposed", [False, True])
@pytest.mark.parametrize("shape", [(1, 1024, 1024, 1024), (1, 784, 1024, 1024), (1, 1024, 1000, 1000), (2, 512, 832, 520), (1, 960, 516, 1024),
                                   (1, 1024, 1024, 10), (1, 200, 96, 136), (2, 130, 70, 151), (1, 2048, 64, 2048), (1, 300, 7, 52),
                                   (1, 256, 512, 256), (1, 64, 1, 64)])
def test_right_operand_column_sums(tt, dtype, a_transposed, shape):
    """rhs_colsum_out = the right operand summed over k, whichever kernel takes the product: the two-half kernel adds
    up the vectors it stages (the first four shapes, a Linear layer's weight gradient x^T . dy among them: ragged
    columns, a partial last k tile, batches), every other kernel leaves it to a launch of its own.  Exact on
    integer-valued data; the product itself is not affected."""
    B, N, K, M = shape
    rng = np.random.default_rng(N + 3 * K + M)
    a = rng.integers(-3, 4, (B, N, K)).astype(dtype)
    b = rng.integers(-3, 4, (B, K, M)).astype(dtype)
    be = tt.get_backend(tt.kAMD)
    ta = tt.Tensor.from_numpy(np.ascontiguousarray(a.transpose(0, 2, 1))).permute(0, 2, 1) if a_transposed else tt.Tensor.from_numpy(a)
    tb = tt.Tensor.from_numpy(b)
    sums = tt.Tensor.from_numpy(np.full((B, M), 77, dtype))
    got = be.batched_matmul(ta, tb, rhs_colsum_out=sums).to_numpy()
    assert np.array_equal(got, np.matmul(a.astype(np.float64), b.astype(np.float64)).astype(dtype))
    assert np.array_equal(sums.to_numpy(), b.sum(axis=1)), _variant(tt, ta, tb)
    # with the other options of the store in the same call
    bias = rng.integers(-5, 6, (M,)).astype(dtype)
    sums2 = tt.Tensor.from_numpy(np.zeros((B, M), dtype))
    got = be.batched_matmul(ta, tb, bias=tt.Tensor.from_numpy(bias), bias_mode=1, relu=True, rhs_colsum_out=sums2).to_numpy()
    assert np.array_equal(got, np.maximum(np.matmul(a.astype(np.float64), b.astype(np.float64)) + bias, 0).astype(dtype))
    assert np.array_equal(sums2.to_numpy(), b.sum(axis=1))


def test_right_operand_column_sums_of_degenerate_products(tt):
    be = tt.get_backend(tt.kAMD)
    f32 = tt._capi.F32
    # K = 0: the empty sum
    sums = tt.Tensor.from_numpy(np.full((2, 7), 5, np.float32))
    out = be.batched_matmul(tt.Tensor.empty((2, 5, 0), f32), tt.Tensor.empty((2, 0, 7), f32), rhs_colsum_out=sums).to_numpy()
    assert np.all(out == 0) and np.all(sums.to_numpy() == 0)
    # no rows on the left: no product, but the right operand still has its sums
    b = np.arange(2 * 3 * 7, dtype=np.float32).reshape(2, 3, 7)
    sums = tt.Tensor.from_numpy(np.zeros((2, 7), np.float32))
    assert be.batched_matmul(tt.Tensor.empty((2, 0, 3), f32), tt.Tensor.from_numpy(b), rhs_colsum_out=sums).shape == (2, 0, 7)
    assert np.array_equal(sums.to_numpy(), b.sum(axis=1))


def test_result_column_sums_of_degenerate_products(tt):
    """colsum_out follows the same rule as rhs_colsum_out: it is written whenever the result has columns."""
    be = tt.get_backend(tt.kAMD)
    f32 = tt._capi.F32
    # no rows: the sums over zero rows are zeros (the buffer held something else)
    cs = tt.Tensor.from_numpy(np.full((2, 7), 5, np.float32))
    b = np.arange(2 * 3 * 7, dtype=np.float32).reshape(2, 3, 7)
    assert be.batched_matmul(tt.Tensor.empty((2, 0, 3), f32), tt.Tensor.from_numpy(b), colsum_out=cs).shape == (2, 0, 7)
    assert np.all(cs.to_numpy() == 0)
    # K = 0: every element is the empty sum plus the bias, so a column's sum is rows x bias
    bias = np.arange(7, dtype=np.float32) - 3
    cs = tt.Tensor.from_numpy(np.full((2, 7), 5, np.float32))
    out = be.batched_matmul(tt.Tensor.empty((2, 5, 0), f32), tt.Tensor.empty((2, 0, 7), f32), bias=tt.Tensor.from_numpy(bias),
                            bias_mode=1, colsum_out=cs).to_numpy()
    assert np.array_equal(out, np.broadcast_to(bias, (2, 5, 7)))
    assert np.array_equal(cs.to_numpy(), np.broadcast_to(5 * bias, (2, 7)))


def test_right_operand_column_sums_need_a_dense_operand(tt):
    be = tt.get_backend(tt.kAMD)
    a = tt.Tensor.from_numpy(np.ones((1, 64, 64), np.float32))
    bt = tt.Tensor.from_numpy(np.ones((1, 64, 64), np.float32)).permute(0, 2, 1)
    with pytest.raises(tt.TTException):
        be.batched_matmul(a, bt, rhs_colsum_out=tt.Tensor.from_numpy(np.zeros((1, 64), np.float32)))
    ai = tt.Tensor.from_numpy(np.ones((1, 64, 64), np.int32))
    with pytest.raises(tt.TTException):
        be.batched_matmul(ai, ai, rhs_colsum_out=tt.Tensor.from_numpy(np.zeros((1, 64), np.int32)))


def _head_reference(x, w, b, t, z):
    """The head's results from numpy, in float64 where a sum is involved."""
    dtype = x.dtype.type
    y = (x.astype(np.float64) @ w.astype(np.float64) + (0 if b is None else b)).astype(dtype)
    d = y - t
    dy = (dtype(1) / dtype(y.size) * dtype(2)) * d
    dx = dy.astype(np.float64) @ w.astype(np.float64).T
    if z is not None:
        dx = dx * np.where(z < 0, 0.0, 1.0)
    return dict(y=y, loss=np.mean(d.astype(np.float64) ** 2), dy=dy, dx=dx, dW=x.astype(np.float64).T @ dy.astype(np.float64),
                db=dy.astype(np.float64).sum(0))


# (rows, in_features, out_features): configuration 5's head; ragged rows, columns and k tiles; more row blocks than groups
# (several blocks to a workgroup); k parts of more than one tile per wave; the widest k one part takes and one beyond;
# out_features 16 and 1; shapes the two-launch form leaves to the separate calls (17 outputs, k not a multiple of 4, k < 16)
HEAD_SHAPES = [(1024, 1024, 10), (4096, 1024, 16), (2048, 512, 8), (64, 256, 32), (1000, 260, 7), (5000, 64, 16), (33, 2048, 3), (2100, 516, 10), (16, 16, 1), (1, 20, 5),
               (700, 4096, 10), (300, 8196, 2), (1500, 1028, 13), (64, 256, 17), (130, 70, 10), (50, 12, 4), (257, 1000, 64)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("with_bias,with_mask", [(True, True), (False, False)])
@pytest.mark.parametrize("shape", HEAD_SHAPES)
def test_linear_mse_head_exact_on_integers(tt, dtype, with_bias, with_mask, shape):
    """Integer-valued operands and a power-of-two element count: every product and sum is exact in any order, so each
    output must equal numpy's bit for bit, whichever kernels the call runs."""
    R, K, N = shape
    rng = np.random.default_rng(R * 31 + K + N)
    x = rng.integers(-2, 3, (R, K)).astype(dtype)
    w = rng.integers(-2, 3, (K, N)).astype(dtype)
    b = rng.integers(-3, 4, (N,)).astype(dtype) if with_bias else None
    t = rng.integers(-4, 5, (R, N)).astype(dtype)
    z = rng.integers(-2, 3, (R, K)).astype(dtype) if with_mask else None
    d = lambda v: tt.Tensor.from_numpy(v) if v is not None else None
    y, loss, dx, dW, db = tt.linear_mse_head(d(x), d(w), d(b), d(t), d(z))
    want = _head_reference(x, w, b, t, z)
    assert np.array_equal(y.to_numpy(), want["y"])
    numel = R * N
    tol = 2e-5 if dtype == np.float32 else 1e-12
    assert abs(float(loss.to_numpy()[0]) - want["loss"]) <= tol * want["loss"]
    if numel & (numel - 1) == 0:   # 1 / numel is a power of two: the gradients are exact as well
        assert np.array_equal(dx.to_numpy(), want["dx"].astype(dtype))
        assert np.array_equal(dW.to_numpy(), want["dW"].astype(dtype))
        if with_bias:
            assert np.array_equal(db.to_numpy(), want["db"].astype(dtype))
    else:
        for got, key in ((dx, "dx"), (dW, "dW")) + (((db, "db"),) if with_bias else ()):
            scale = np.abs(want[key]).max() + 1e-30
            assert np.max(np.abs(got.to_numpy() - want[key])) <= tol * scale, key
    assert (db is None) == (not with_bias)


@pytest.mark.parametrize("shape", [(1024, 1024, 10), (1000, 260, 7), (2100, 516, 10), (700, 4096, 10)])
def test_linear_mse_head_matches_the_separate_calls(tt, shape):
    """Real-valued data: the one call against Linear, mse_loss and linear_backward one after the other.  y, and with it dy, come
    from the same order of sums in both (bit-equal); dx, dW, db and the loss add in other orders."""
    R, K, N = shape
    rng = np.random.default_rng(R + K + N)
    x = np.maximum(rng.normal(0, 1, (R, K)), 0).astype(np.float32)
    z = rng.normal(0, 1, (R, K)).astype(np.float32)
    w = rng.uniform(-0.05, 0.05, (K, N)).astype(np.float32)
    b = rng.uniform(-0.05, 0.05, (N,)).astype(np.float32)
    t = rng.uniform(0, 1, (R, N)).astype(np.float32)
    d = tt.Tensor.from_numpy
    tx, tw, tb_, tt_, tz = d(x), d(w), d(b), d(t), d(z)
    y, loss, dx, dW, db = tt.linear_mse_head(tx, tw, tb_, tt_, tz)
    y2 = tt.linear(tx, tw, tb_)
    loss2, gy2, db2 = tt.mse_loss(y2, tt_, grad=True, bias_grad=True)
    dx2, dW2, _ = tt.linear_backward(gy2, tx, tw, relu_input=tz, bias_grad=False)
    assert np.array_equal(y.to_numpy(), y2.to_numpy())
    assert abs(float(loss.to_numpy()[0]) - float(loss2.to_numpy()[0])) <= 1e-5 * float(loss2.to_numpy()[0])
    want = _head_reference(x, w, b, t, z)
    for got, sep, key in ((dx, dx2, "dx"), (dW, dW2, "dW"), (db, db2, "db")):
        scale = np.abs(want[key]).max()
        err, err_sep = (np.max(np.abs(v.to_numpy().reshape(want[key].shape) - want[key])) / scale for v in (got, sep))
        assert err <= 2e-6, (key, err, err_sep)
    # the masked elements are zeros, the others are not touched by the mask
    assert np.all(dx.to_numpy()[z < 0] == 0)


def test_linear_mse_head_keeps_nan_under_the_mask_and_checks_arguments(tt):
    x = np.ones((32, 64), np.float32)
    w = np.ones((64, 4), np.float32)
    t = np.zeros((32, 4), np.float32)
    t[:, 2] = np.inf                       # column 2 of dy = scale * (y - inf) is -inf, and with it every element of dy . W^T
    z = -np.ones((32, 64), np.float32)
    d = tt.Tensor.from_numpy
    _, _, dx, _, _ = tt.linear_mse_head(d(x), d(w), None, d(t), d(z))
    assert np.all(np.isnan(dx.to_numpy()))  # -inf times the mask's 0 is NaN, as in the reference's product
    with pytest.raises(tt.TTException):
        tt.linear_mse_head(d(x), d(w), None, d(np.zeros((32, 5), np.float32)), None)
    with pytest.raises(tt.TTException):
        tt.linear_mse_head(d(x), d(np.ones((64, 65), np.float32)), None, d(np.zeros((32, 65), np.float32)), None)
    with pytest.raises(tt.TTException):
        tt.linear_mse_head(d(x), d(w.astype(np.float64)), None, d(t), None)


# (rows, in_features, out_features, one grid): the two gradients of a Linear layer as one call.  One grid when both products
# are dense fp32 with 128 to 256 tiles of 64 x 64 and reductions of 512 or more; everything else runs as two calls.
PAIR_SHAPES = [(1024, 1024, 1024, True), (1024, 784, 1024, True), (520, 1000, 640, True), (576, 900, 700, True),
               (512, 1024, 1024, True), (1024, 2048, 520, True),
               (256, 512, 384, False), (1024, 1024, 10, False), (300, 2000, 2000, False), (2048, 1024, 1024, False)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("bias_grad", ["own", False, True])
@pytest.mark.parametrize("shape", PAIR_SHAPES, ids=lambda s: "x".join(map(str, s[:3])))
def test_linear_backward_pair_exact_on_integers(tt, dtype, bias_grad, shape):
    """nn::Linear's backward (TensorBatchedMatmul::backward, autograd/binary_ops.cpp:173-179, with the ReLU mask of
    unary_ops.cpp:568-573 and the bias gradient) through ttamd_batched_matmul_pair: integer-valued data, exact in any
    order of summation, in the one-grid form and in the two-call form alike; grad_output's NaN under the mask stays."""
    n, fin, fout, _ = shape
    rng = np.random.default_rng(n + fin + fout)
    dy = rng.integers(-3, 4, (n, fout)).astype(dtype)
    x = rng.integers(-3, 4, (n, fin)).astype(dtype)
    w = rng.integers(-3, 4, (fin, fout)).astype(dtype)
    z = rng.integers(-2, 3, (n, fin)).astype(dtype)
    tdy, tx, tw, tz = (tt.Tensor.from_numpy(v) for v in (dy, x, w, z))
    dx, dW, db = tt.linear_backward(tdy, tx, tw, relu_input=tz, bias_grad=bias_grad)
    want_dx = (dy.astype(np.float64) @ w.T.astype(np.float64)) * np.where(z < 0, 0.0, 1.0)
    assert np.array_equal(dx.to_numpy(), want_dx.astype(dtype))
    assert np.array_equal(dW.to_numpy(), (x.T.astype(np.float64) @ dy.astype(np.float64)).astype(dtype))
    if bias_grad == "own":
        assert np.array_equal(db.to_numpy(), dy.sum(0))
    elif bias_grad:
        assert np.array_equal(db.to_numpy(), want_dx.sum(0).astype(dtype))
    else:
        assert db is None
    # without the mask, and a second call: the same bits
    dx2, dW2, _ = tt.linear_backward(tdy, tx, tw, bias_grad=False)
    assert np.array_equal(dx2.to_numpy(), (dy.astype(np.float64) @ w.T.astype(np.float64)).astype(dtype))
    assert np.array_equal(dW2.to_numpy(), dW.to_numpy())


@pytest.mark.parametrize("shape", [s for s in PAIR_SHAPES if s[3]][:4], ids=lambda s: "x".join(map(str, s[:3])))
def test_batched_matmul_pair_on_real_data(tt, oracle, shape):
    """Real-valued data in the one-grid form: each product within the bound of a k-ordered fp32 sum of the oracle's
    product, the same bits on a second call, NaN and infinity kept where the reference's multiplication by the mask keeps
    them, and the right operand's column sums equal to numpy's sum in float64 to rounding."""
    n, fin, fout, _ = shape
    rng = np.random.default_rng(n * 3 + fin + fout)
    dy = rng.standard_normal((n, fout)).astype(np.float32)
    x = rng.standard_normal((n, fin)).astype(np.float32)
    w = rng.standard_normal((fin, fout)).astype(np.float32)
    z = rng.standard_normal((n, fin)).astype(np.float32)
    dy[3, 5] = np.inf
    tdy, tx, tw, tz = (tt.Tensor.from_numpy(v) for v in (dy, x, w, z))
    be = tt.get_backend(tt.kAMD)
    db = tt.Tensor.empty((1, fout), tdy.dtype)
    first = (tdy.unsqueeze(0), tw.unsqueeze(0).permute(0, 2, 1), dict(relu_grad_input=tz.unsqueeze(0)))
    second = (tx.unsqueeze(0).permute(0, 2, 1), tdy.unsqueeze(0), dict(rhs_colsum_out=db))
    dx, dW = (t.to_numpy()[0] for t in be.batched_matmul_pair(first, second))
    dx_b, dW_b = (t.to_numpy()[0] for t in be.batched_matmul_pair(first, second))
    assert np.array_equal(dx, dx_b, equal_nan=True) and np.array_equal(dW, dW_b, equal_nan=True)
    fin_dy = np.where(np.isfinite(dy), dy, 0).astype(np.float32)
    want_dx = oracle.matmul(fin_dy, np.ascontiguousarray(w.T), "fast") * np.where(z < 0, 0, 1).astype(np.float32)
    want_dW = oracle.matmul(np.ascontiguousarray(x.T), fin_dy, "fast")
    rows, cols = np.ones(n, bool), np.ones(fout, bool)
    rows[3] = False
    cols[5] = False
    scale_dx = np.abs(fin_dy).astype(np.float64) @ np.abs(w.T).astype(np.float64)
    scale_dW = np.abs(x.T).astype(np.float64) @ np.abs(fin_dy).astype(np.float64)
    assert np.max(np.abs(dx[rows] - want_dx[rows]) / scale_dx[rows]) < 2e-6   # ~ 2^-19: fp32 sums of 520 to 1024 terms in another order
    assert np.max(np.abs(dW[:, cols] - want_dW[:, cols]) / scale_dW[:, cols]) < 2e-6
    # row 3 of dx holds inf . w = +-inf, times the mask: NaN under a 0, +-inf under a 1, as `grad * where(z < 0, 0, 1)` gives
    with np.errstate(invalid="ignore"):
        want_row = (np.float32(np.inf) * w[:, 5]) * np.where(z[3] < 0, np.float32(0), np.float32(1))
    assert np.array_equal(np.isnan(dx[3]), np.isnan(want_row)) and np.array_equal(dx[3][~np.isnan(want_row)], want_row[~np.isnan(want_row)])
    assert np.all(np.isinf(dW[:, 5]) | np.isnan(dW[:, 5]))
    got_db = db.to_numpy()[0]
    assert np.isinf(got_db[5]) and np.allclose(got_db[cols], dy[:, cols].astype(np.float64).sum(0), rtol=0, atol=2e-4)


def test_batched_matmul_pair_general_operands_and_argument_checks(tt):
    """Operands outside the one-grid form -- integer dtypes, offset and strided views, empty products, batches -- give the
    bits of two ttamd_batched_matmul calls (they are two such calls); a NULL product is refused."""
    from tinytensor_amd import _capi
    be = tt.get_backend(tt.kAMD)
    rng = np.random.default_rng(77)
    for dtype in (np.int32, np.uint8, np.float64, np.float32):
        a = rng.integers(0, 5, (2, 70, 33)).astype(dtype)
        b = rng.integers(0, 5, (2, 33, 41)).astype(dtype)
        big = tt.Tensor.from_numpy(np.concatenate([np.zeros((1, 70, 33), dtype), a]))
        ta = tt.Tensor(big.storage, big.dtype, (2, 70, 33), big.stride, 70 * 33)      # an offset view
        tb = tt.Tensor.from_numpy(np.ascontiguousarray(b.transpose(0, 2, 1))).permute(0, 2, 1)  # a permuted view
        g = rng.integers(0, 5, (2, 70, 41)).astype(dtype)
        tg = tt.Tensor.from_numpy(g)
        da, db = be.batched_matmul_pair((tg, tb.permute(0, 2, 1)), (ta.permute(0, 2, 1), tg))
        assert np.array_equal(da.to_numpy(), be.batched_matmul(tg, tb.permute(0, 2, 1)).to_numpy())
        assert np.array_equal(db.to_numpy(), be.batched_matmul(ta.permute(0, 2, 1), tg).to_numpy())
        assert np.array_equal(da.to_numpy(), np.matmul(g, b.transpose(0, 2, 1)))
        assert np.array_equal(db.to_numpy(), np.matmul(a.transpose(0, 2, 1), g))
    # empty products: no rows in one, no reduction in the other
    e0, e1 = be.batched_matmul_pair((tt.Tensor.empty((1, 0, 8), _capi.F32), tt.Tensor.empty((1, 8, 4), _capi.F32)),
                                    (tt.Tensor.empty((1, 5, 0), _capi.F32), tt.Tensor.empty((1, 0, 3), _capi.F32)))
    assert e0.shape == (1, 0, 4) and np.array_equal(e1.to_numpy(), np.zeros((1, 5, 3), np.float32))
    assert _capi.lib.ttamd_batched_matmul_pair(0, _capi.F32, None, None, None) != 0
    assert "NULL product" in _capi.last_error()


@pytest.mark.parametrize("own", [False, True, "head"])
def test_fused_mlp_training_step_matches_the_oracle_and_fits_15_launches(tt, oracle, own):
    X = oracle.Generator(0).uniform_real(0.0, 1.0, (1024, 784))
    T = oracle.Generator(1).uniform_real(0.0, 1.0, (1024, 10))
    g = oracle.Generator(0)
    params_h = [oracle.linear_init(g, a, b) for a, b in ((784, 1024), (1024, 1024), (1024, 10))]
    d = tt.Tensor.from_numpy
    x, t = d(X), d(T)
    params = [(d(W), d(b)) for W, b in params_h]
    got = {k: v.to_numpy() for k, v in fused_mlp_step(tt, x, t, params, own).items()}
    masks = (np.where(got["z1"] < 0, np.float32(0), np.float32(1)), np.where(got["z2"] < 0, np.float32(0), np.float32(1)))
    want = mlp_train_step(X, T, params_h, lambda a, b: oracle.matmul(a, b),
                          lambda a, b, gr: tuple(v[0] for v in oracle.matmul_backward(a[None], b[None], gr[None])), masks=masks)
    cpu = mlp_train_step(X, T, params_h, lambda a, b: oracle.matmul(a, b),
                         lambda a, b, gr: tuple(v[0] for v in oracle.matmul_backward(a[None], b[None], gr[None])))
    assert sum(int(np.sum(a != b)) for a, b in zip(masks, cpu["masks"])) <= 8   # z within rounding of 0
    for key in ("y", "dW1", "db1", "dW2", "db2", "dW3", "db3", "dX"):
        assert got[key].shape == want[key].shape, key
        assert max_rel_error(got[key], want[key]) <= 1e-4, key
    assert abs(float(got["loss"][0]) - float(want["loss"])) <= 1e-4 * abs(float(want["loss"]))
    # launches: record the step into a HIP graph and count its kernel nodes
    stream = tt.graph.Stream()
    graph = None
    try:
        graph = tt.graph.Graph(stream, lambda: list(fused_mlp_step(tt, x, t, params, own).values()))
        assert graph.num_nodes() <= {False: 15, True: 10, "head": 8}[own], graph.num_nodes()
        graph.launch()
        stream.synchronize()
        for k, v in zip(("y", "loss", "dW1", "db1", "dW2", "db2", "dW3", "db3", "dX"), graph.outputs):
            assert np.array_equal(v.to_numpy(), got[k]), k   # same kernels, same inputs
    finally:
        if graph is not None:
            graph.close()
        stream.close()
