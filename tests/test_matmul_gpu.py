"""GPU parity tests for ttamd_batched_matmul, called through the C ABI (ctypes) and compared with the
CPU oracle on identical inputs.  The cases follow the reference's own tests (tests/test_matmul.cpp) and the
benchmark configurations; shapes are sized so that the oracle finishes in seconds.

Bars: bit-exact for integer dtypes and for float data whose exact result is an integer below 2^24;
otherwise K-scaled relative error <= 1e-4 (f32) / <= 1e-12 (f64).
"""
import numpy as np
import pytest

from helpers import (ALL_NON_BOOL, F32_TOL, F64_TOL, max_rel_error, naive_exact, ref_batched, ref_dot, ref_mat_mat,
                     ref_vec_mat, scaled_error, tol_of)

pytestmark = pytest.mark.gpu


def dev(tt, a):
    return tt.Tensor.from_numpy(a)


def check_close(got, want, A, B, dtype):
    tol = tol_of(dtype)
    assert got.shape == want.shape
    assert scaled_error(got, want, A, B) <= tol
    assert max_rel_error(got, want) <= tol


# ----------------------------------------------------------------------------- reference test cases
@pytest.mark.parametrize("dtype", ALL_NON_BOOL)
def test_dot_product(tt, oracle, dtype):
    for n in (12, 2048):
        a, b = ref_dot(n, dtype)
        got = tt.matmul(dev(tt, a), dev(tt, b)).to_numpy()
        want = oracle.matmul(a, b)
        if np.issubdtype(dtype, np.floating):
            assert np.allclose(got, want, rtol=1e-5, atol=1e-8)  # the reference's allclose defaults
        else:
            assert np.array_equal(got, want)


def test_bool_is_rejected(tt):
    a = dev(tt, np.ones(12, dtype=np.bool_))
    with pytest.raises(tt.TTException):
        tt.matmul(a, a)
    b = dev(tt, np.ones((2, 12, 4), dtype=np.bool_))
    c = dev(tt, np.ones((2, 4, 12), dtype=np.bool_))
    with pytest.raises(tt.TTException):
        tt.matmul(b, c)


def test_mixed_dtypes_are_promoted(tt):
    # check_promote (tensor/tensor.cpp:2398-2399): both operands are cast to promote_types(lhs, rhs)
    rng = np.random.default_rng(4)
    a = rng.integers(-5, 6, (7, 9)).astype(np.int16)
    for other, want_dtype in ((np.int64, np.int64), (np.float32, np.float32), (np.float64, np.float64), (np.bool_, np.int16)):
        b = rng.integers(0, 2 if other == np.bool_ else 6, (9, 5)).astype(other)
        got = tt.matmul(dev(tt, a), dev(tt, b)).to_numpy()
        assert got.dtype == np.dtype(want_dtype)
        assert np.array_equal(got, a.astype(want_dtype) @ b.astype(want_dtype))
    out = tt.linear(dev(tt, a), dev(tt, np.ones((9, 5), np.float32)), dev(tt, np.arange(5, dtype=np.int32)))
    assert out.to_numpy().dtype == np.float32
    assert np.array_equal(out.to_numpy(), a.astype(np.float32) @ np.ones((9, 5), np.float32) + np.arange(5, dtype=np.float32))


def test_shape_errors(tt):
    a = dev(tt, np.ones((3, 4), dtype=np.float32))
    with pytest.raises(tt.TTException):
        tt.matmul(a, a)
    with pytest.raises(tt.TTException):
        tt.matmul(dev(tt, np.ones((2, 3, 4, 5), dtype=np.float32)), a)


@pytest.mark.parametrize("dtype", ALL_NON_BOOL)
def test_vector_matrix_and_matrix_vector(tt, oracle, dtype):
    v, m = ref_vec_mat(dtype)
    got = tt.matmul(dev(tt, v), dev(tt, m)).to_numpy()
    assert np.array_equal(got, naive_exact(v[None, :], m)[0])
    mt = np.ascontiguousarray(m.T)
    got = tt.matmul(dev(tt, mt), dev(tt, v)).to_numpy()
    assert np.array_equal(got, naive_exact(mt, v[:, None])[:, 0])


@pytest.mark.parametrize("dtype", ALL_NON_BOOL)
def test_matrix_matrix_reference_size_exact(tt, oracle, dtype):
    lhs, rhs = ref_mat_mat(dtype)  # [379,1147] . [1147,635], values (i+j)%100: exact in every dtype
    got = tt.matmul(dev(tt, lhs), dev(tt, rhs)).to_numpy()
    want = naive_exact(lhs, rhs)
    assert np.array_equal(got, want)
    if dtype in (np.float32, np.int32):
        assert np.array_equal(oracle.matmul(lhs, rhs), want)  # and the oracle agrees with that closed form


@pytest.mark.parametrize("dtype", ALL_NON_BOOL)
def test_batched_reference_pattern_exact(tt, dtype):
    lhs, rhs = ref_batched(dtype, B=4, N=379, M=1147, K=635)  # tests/test_matmul.cpp:200-236, at its own size
    got = tt.matmul(dev(tt, lhs), dev(tt, rhs)).to_numpy()
    want = np.stack([naive_exact(lhs[b], rhs[b]) for b in range(4)])
    assert np.array_equal(got, want)


# ----------------------------------------------------------------------------- at most 16 columns
# (B, N rows, K, M columns): the MLP head of benchmark configuration 5 and its weight gradient's shape, ragged rows,
# k that ends inside a wave's chunk / inside a 16-byte vector / before most waves get any, one column, 16 columns, batches
THIN_SHAPES = [(1, 1024, 1024, 10), (1, 1000, 784, 10), (2, 37, 333, 7), (1, 16, 64, 16), (3, 50, 130, 1), (1, 5, 1022, 16),
               (1, 300, 65, 3)]
# small outputs of a long reduction (the same kernel over a grid of 16 x 16 blocks): benchmark configuration 1, ragged
# blocks in both directions, batches, one block row
SMALL_SHAPES = [(1, 256, 512, 256), (2, 100, 300, 50), (1, 37, 129, 333), (4, 128, 256, 128), (1, 17, 1024, 17)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("layout", ["plain", "a_transposed", "b_transposed", "a_row_slice"])
@pytest.mark.parametrize("shape", THIN_SHAPES + SMALL_SHAPES)
def test_products_of_at_most_16_columns_and_small_outputs(tt, oracle, dtype, layout, shape):
    B, N, K, M = shape
    rng = np.random.default_rng(N * 7 + K + M)
    a = rng.integers(-4, 5, (B, N, K)).astype(dtype)
    b = rng.integers(-4, 5, (B, K, M)).astype(dtype)
    be = tt.get_backend(tt.kAMD)
    ta, tb = dev(tt, a), dev(tt, b)
    if layout == "a_transposed":      # h^T . dy: A is a permuted view, k-major
        ta = dev(tt, np.ascontiguousarray(a.transpose(0, 2, 1))).permute(0, 2, 1)
    elif layout == "b_transposed":
        tb = dev(tt, np.ascontiguousarray(b.transpose(0, 2, 1))).permute(0, 2, 1)
    elif layout == "a_row_slice":     # rows of a wider matrix: row stride above K, the start not 16-byte aligned for odd offsets
        wide = np.zeros((B, N, K + 5), dtype)
        wide[:, :, 3:3 + K] = a
        tw = dev(tt, wide)
        ta = tt.Tensor(tw.storage, tw.dtype, (B, N, K), (N * (K + 5), K + 5, 1), 3)
    variant = be.batched_matmul_variant(ta, tb)
    assert variant.startswith(("thin_" if M <= 16 else "small_") + ("f32" if dtype == np.float32 else "f64")), variant
    if layout == "plain" and K % (4 if dtype == np.float32 else 2) == 0:
        assert "vec" in variant
    if layout in ("a_transposed", "a_row_slice"):
        assert "vec" not in variant
    want = np.matmul(a.astype(np.float64), b.astype(np.float64))
    assert np.array_equal(be.batched_matmul(ta, tb).to_numpy(), want.astype(dtype)), variant
    # the store's steps: bias per column with ReLU and second output, bias per row accumulated onto the old values,
    # the ReLU-backward mask
    bias_n, bias_m = rng.integers(-5, 6, (M,)).astype(dtype), rng.integers(-5, 6, (N,)).astype(dtype)
    act = tt.Tensor.empty((B, N, M), ta.dtype)
    got = be.batched_matmul(ta, tb, bias=dev(tt, bias_n), bias_mode=1, relu_out=act).to_numpy()
    assert np.array_equal(got, (want + bias_n).astype(dtype)) and np.array_equal(act.to_numpy(), np.maximum(got, 0))
    old = rng.integers(-9, 10, (B, N, M)).astype(dtype)
    acc = dev(tt, old)
    be.batched_matmul(ta, tb, bias=dev(tt, bias_m), bias_mode=2, relu=True, accumulate=True, out=acc)
    assert np.array_equal(acc.to_numpy(), (np.maximum(want + bias_m[None, :, None], 0) + old).astype(dtype))
    z = rng.integers(-2, 3, (B, N, M)).astype(dtype)
    got = be.batched_matmul(ta, tb, relu_grad_input=dev(tt, z)).to_numpy()
    assert np.array_equal(got, (want * np.where(z < 0, 0.0, 1.0)).astype(dtype))
    # uniform data against the oracle, at the tolerance of the other products
    if layout == "plain":
        A = rng.uniform(-1, 1, (B, N, K)).astype(dtype)
        Bm = rng.uniform(-1, 1, (B, K, M)).astype(dtype)
        got = be.batched_matmul(dev(tt, A), dev(tt, Bm)).to_numpy()
        for i in range(B):
            check_close(got[i], oracle.matmul(A[i], Bm[i]), A[i], Bm[i], dtype)


def test_operands_beyond_k_do_not_leak_into_thin_products(tt):
    """The chunk of k that crosses K reads stand-in elements (the row's element at k = 0); an infinity there must reach
    the sum once, from k = 0 itself, and not a second time as inf * 0 = NaN."""
    be = tt.get_backend(tt.kAMD)
    for K in (70, 72):           # element-wise loads, 16-byte loads
        a = np.ones((1, 20, K), np.float32)
        a[0, :, 0] = np.inf
        b = np.ones((1, K, 10), np.float32)
        got = be.batched_matmul(dev(tt, a), dev(tt, b)).to_numpy()
        assert np.all(np.isposinf(got)), K


# ----------------------------------------------------------------------------- benchmark configurations
def test_config1_single_f32(tt, oracle):
    A = oracle.Generator(0).uniform_real(-1, 1, (256, 512))
    B = oracle.Generator(0).uniform_real(-1, 1, (512, 256))
    got = tt.matmul(dev(tt, A), dev(tt, B)).to_numpy()
    want = oracle.matmul(A, B)
    check_close(got, want, A, B, np.float32)
    # exact on small integers stored in f32
    Ai, Bi = np.round(A * 16).astype(np.float32), np.round(B * 16).astype(np.float32)
    assert np.array_equal(tt.matmul(dev(tt, Ai), dev(tt, Bi)).to_numpy(), oracle.matmul(Ai, Bi))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_config2_batched_transposed_view(tt, oracle, dtype):
    A = oracle.Generator(0).uniform_real(-1, 1, (32, 128, 64), dtype)
    Bsrc = oracle.Generator(1).uniform_real(-1, 1, (32, 128, 64), dtype)
    tB = dev(tt, Bsrc).permute(0, 2, 1)
    assert tB.stride == (8192, 1, 64) and tB.shape == (32, 64, 128)
    tA = dev(tt, A)
    got = tt.matmul(tA, tB).to_numpy()
    Bv = Bsrc.transpose(0, 2, 1)
    want = oracle.matmul(A, Bv)
    for b in (0, 13, 31):
        check_close(got[b], want[b], A[b], Bv[b], dtype)
    assert max_rel_error(got, want) <= tol_of(dtype)
    # identical to running on a dense copy of the view: the kernel sums in the same order either way
    dense = tt.matmul(tA, dev(tt, np.ascontiguousarray(Bv))).to_numpy()
    assert np.array_equal(got, dense)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_backward_gemms_on_permuted_views(tt, oracle, dtype):
    # TensorBatchedMatmul::backward: dA = dC.B^T and dB = A^T.dC on permute({0,2,1}) views
    rng = np.random.default_rng(11)
    A = rng.uniform(-1, 1, (3, 96, 200)).astype(dtype)
    B = rng.uniform(-1, 1, (3, 200, 136)).astype(dtype)
    dC = rng.uniform(-1, 1, (3, 96, 136)).astype(dtype)
    dA, dB = tt.matmul_backward(dev(tt, A), dev(tt, B), dev(tt, dC))
    wA, wB = oracle.matmul_backward(A, B, dC)
    for b in range(3):
        check_close(dA.to_numpy()[b], wA[b], dC[b], B[b].T, dtype)
        check_close(dB.to_numpy()[b], wB[b], A[b].T, dC[b], dtype)


# ----------------------------------------------------------------------------- layouts, edges, strides
LAYOUTS = ["nn", "nt", "tn", "tt"]


def make_operands(rng, layout, N, K, M, dtype, batch=1):
    """Returns host views (A [b,N,K], B [b,K,M]) whose memory layout follows `layout`."""
    if layout[0] == "n":
        A = rng.uniform(-1, 1, (batch, N, K)).astype(dtype)
    else:
        A = rng.uniform(-1, 1, (batch, K, N)).astype(dtype).transpose(0, 2, 1)
    if layout[1] == "n":
        B = rng.uniform(-1, 1, (batch, K, M)).astype(dtype)
    else:
        B = rng.uniform(-1, 1, (batch, M, K)).astype(dtype).transpose(0, 2, 1)
    return A, B


def to_dev_view(tt, host_view):
    """Uploads the memory that backs `host_view` and rebuilds the same strided view on the device."""
    base = host_view
    while isinstance(base.base, np.ndarray):
        base = base.base
    t = tt.Tensor.from_numpy(base.reshape(-1))
    off = (host_view.ctypes.data - base.ctypes.data) // host_view.itemsize
    return tt.Tensor(t.storage, t.dtype, host_view.shape, [s // host_view.itemsize for s in host_view.strides], off)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("shape", [(128, 64, 128), (256, 96, 384), (67, 45, 131), (64, 8, 64), (33, 1, 65),
                                   (512, 40, 1024), (1024, 72, 2048)])
def test_layouts_and_edges(tt, oracle, dtype, layout, shape):
    N, K, M = shape
    rng = np.random.default_rng(N * 7 + K * 3 + M)
    A, B = make_operands(rng, layout, N, K, M, dtype, batch=2)
    tA, tB = to_dev_view(tt, A), to_dev_view(tt, B)
    got = tt.matmul(tA, tB).to_numpy()
    want = oracle.matmul(A, B)
    for b in range(2):
        check_close(got[b], want[b], A[b], B[b], dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32])
def test_generic_strides_offsets_and_expand(tt, oracle, dtype):
    rng = np.random.default_rng(4)
    # row stride 3*K+5 with column stride 3 (neither is 1), plus a storage offset
    N, K, M = 70, 50, 90
    baseA = rng.integers(-8, 9, size=5 + N * (3 * K + 5)).astype(dtype)
    A = np.lib.stride_tricks.as_strided(baseA[5:], (1, N, K), (0, (3 * K + 5) * baseA.itemsize, 3 * baseA.itemsize))
    baseB = rng.integers(-8, 9, size=3 + K * M * 2).astype(dtype)
    B = np.lib.stride_tricks.as_strided(baseB[3:], (1, K, M), (0, 2 * baseB.itemsize, 2 * K * baseB.itemsize))
    tA = tt.Tensor(tt.Tensor.from_numpy(baseA).storage, tt._capi.F32 if dtype == np.float32 else (tt._capi.F64 if dtype == np.float64 else tt._capi.I32),
                   (1, N, K), (0, 3 * K + 5, 3), 5)
    tB = tt.Tensor(tt.Tensor.from_numpy(baseB).storage, tA.dtype, (1, K, M), (0, 2, 2 * K), 3)
    got = tt.matmul(tA, tB).to_numpy()
    want = naive_exact(np.ascontiguousarray(A[0]), np.ascontiguousarray(B[0]))  # small integers: exact
    assert np.array_equal(got[0], want)
    assert np.array_equal(oracle.matmul(A, B)[0], want)
    # expanded (stride-0) operand: every row of A is the same vector, batch broadcast with stride 0
    row = rng.integers(-8, 9, size=K).astype(dtype)
    tRow = tt.Tensor.from_numpy(row).reshape([1, 1, K]).expand([4, N, K])
    assert tRow.stride == (0, 0, 1)
    tB4 = tt.Tensor(tB.storage, tB.dtype, (4, K, M), (0, 2, 2 * K), 3)
    got = tt.matmul(tRow, tB4).to_numpy()
    want_row = naive_exact(row[None, :], np.ascontiguousarray(B[0]))
    assert np.array_equal(got, np.broadcast_to(want_row, (4, N, M)))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_unaligned_views_fall_back_to_elementwise_loads(tt, oracle, dtype):
    # A dense view that starts one element into the storage is not 16-byte aligned: the dispatcher must pick
    # the gather variant and still be right.
    rng = np.random.default_rng(9)
    N, K, M = 130, 70, 150
    baseA = rng.uniform(-1, 1, 1 + N * K).astype(dtype)
    baseB = rng.uniform(-1, 1, 1 + K * M).astype(dtype)
    code = tt._capi.F32 if dtype == np.float32 else tt._capi.F64
    tA = tt.Tensor(tt.Tensor.from_numpy(baseA).storage, code, (1, N, K), (N * K, K, 1), 1)
    tB = tt.Tensor(tt.Tensor.from_numpy(baseB).storage, code, (1, K, M), (K * M, M, 1), 1)
    be = tt.get_backend(tt.kAMD)
    assert "akc1_bmc1" in be.batched_matmul_variant(tA, tB)
    got = be.batched_matmul(tA, tB).to_numpy()[0]
    A, B = baseA[1:].reshape(N, K), baseB[1:].reshape(K, M)
    check_close(got, oracle.matmul(A, B), A, B, dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("N,Kp,M", [(130, 72, 150), (384, 256, 384), (1024, 1024, 1024), (320, 1000, 448)])
def test_vectors_that_straddle_the_end_of_k_are_cut(tt, dtype, N, Kp, M):
    """Rows padded to a whole number of 16-byte vectors, K one to three elements short of the pitch: the last vector of
    a row holds elements on both sides of K.  The padding holds NaN, so a single element taken from beyond K (in either
    operand: A's rows run along k, and so do the rows of B's storage, read as B^T) shows in every sum it reaches."""
    rng = np.random.default_rng(N + Kp)
    code = tt._capi.F32 if dtype == np.float32 else tt._capi.F64
    vec = 16 // np.dtype(dtype).itemsize
    be = tt.get_backend(tt.kAMD)
    for short in range(1, vec):
        K = Kp - short
        baseA = rng.integers(-4, 5, size=(N, Kp)).astype(dtype)
        baseBt = rng.integers(-4, 5, size=(M, Kp)).astype(dtype)
        A, Bt = baseA[:, :K].copy(), baseBt[:, :K].copy()
        baseA[:, K:] = np.nan
        baseBt[:, K:] = np.nan
        tA = tt.Tensor(tt.Tensor.from_numpy(baseA.ravel()).storage, code, (1, N, K), (N * Kp, Kp, 1), 0)
        tB = tt.Tensor(tt.Tensor.from_numpy(baseBt.ravel()).storage, code, (1, K, M), (M * Kp, 1, Kp), 0)
        variant = be.batched_matmul_variant(tA, tB)
        assert f"akc{vec}_bkc{vec}" in variant, variant
        got = be.batched_matmul(tA, tB).to_numpy()[0]
        assert np.array_equal(got, naive_exact(A, np.ascontiguousarray(Bt.T))), (K, variant)


def test_variant_selection(tt):
    be = tt.get_backend(tt.kAMD)
    f32 = np.float32
    big = tt.Tensor.empty((1, 4096, 4096), tt._capi.F32)
    assert be.batched_matmul_variant(big, big) == "mfma_f32_256x256_akc4_bmc4"
    assert be.batched_matmul_variant(big, big.permute(0, 2, 1)) == "mfma_f32_256x256_akc4_bkc4"
    assert be.batched_matmul_variant(big.permute(0, 2, 1), big) == "mfma_f32_256x256_amc4_bmc4"
    big64 = tt.Tensor.empty((1, 4096, 4096), tt._capi.F64)
    assert be.batched_matmul_variant(big64, big64) == "mfma_f64_256x128_akc2_bmc2"
    small = tt.Tensor.from_numpy(np.zeros((1, 256, 512), f32))
    assert be.batched_matmul_variant(small, small.permute(0, 2, 1)) == "small_f32_16x16_vec4"  # 16 tiles of 64 x 64, long K
    mid = tt.Tensor.empty((1, 512, 512), tt._capi.F32)
    assert be.batched_matmul_variant(mid, mid).startswith("mfma_f32_64x64_akc4_bmc4_splitk")  # more blocks than one round
    deep = tt.Tensor.empty((1, 256, 8192), tt._capi.F32)
    assert be.batched_matmul_variant(deep, deep.permute(0, 2, 1)).startswith("mfma_f32_64x64_akc4_bkc4_splitk")  # too long a k
    thin = tt.Tensor.from_numpy(np.zeros((1, 512, 10), f32))
    assert be.batched_matmul_variant(small, thin) == "thin_f32_16rows_vec4"          # at most 16 columns, long K
    assert be.batched_matmul_variant(small.permute(0, 2, 1), tt.Tensor.empty((1, 256, 10), tt._capi.F32)) == "thin_f32_16rows"
    assert be.batched_matmul_variant(tt.Tensor.empty((1, 1024, 10), tt._capi.F32),
                                     tt.Tensor.empty((1, 10, 1024), tt._capi.F32)) == "thin_f32_k16"  # reduction of at most 16
    assert be.batched_matmul_variant(tt.Tensor.empty((1, 32, 10), tt._capi.F64), tt.Tensor.empty((1, 10, 32), tt._capi.F64)) \
        .startswith("mfma_f64")                                                                        # ... of a small output
    short = tt.Tensor.from_numpy(np.zeros((1, 256, 48), f32))
    assert be.batched_matmul_variant(short, tt.Tensor.empty((1, 48, 10), tt._capi.F32)).startswith("mfma_f32_64x64")  # short K
    thin_i = tt.Tensor.from_numpy(np.zeros((1, 512, 10), np.int32))
    small_i = tt.Tensor.from_numpy(np.zeros((1, 256, 512), np.int32))
    assert be.batched_matmul_variant(small_i, thin_i) == "simt_i32_128x16"
    i32 = tt.Tensor.from_numpy(np.zeros((1, 64, 64), np.int32))
    assert be.batched_matmul_variant(i32, i32) == "simt_i32_64x64"


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_empty_and_degenerate_shapes(tt, dtype):
    code = tt._capi.F32 if dtype == np.float32 else tt._capi.F64
    be = tt.get_backend(tt.kAMD)
    # K = 0: the empty sum
    a = tt.Tensor.empty((2, 5, 0), code)
    b = tt.Tensor.empty((2, 0, 7), code)
    out = be.batched_matmul(a, b).to_numpy()
    assert out.shape == (2, 5, 7) and np.all(out == 0)
    # empty outputs do nothing and do not fail
    assert be.batched_matmul(tt.Tensor.empty((0, 5, 3), code), tt.Tensor.empty((0, 3, 7), code)).shape == (0, 5, 7)
    assert be.batched_matmul(tt.Tensor.empty((1, 0, 3), code), tt.Tensor.empty((1, 3, 7), code)).shape == (1, 0, 7)
    # 1 x 1 x 1
    x = tt.Tensor.from_numpy(np.array([[[3.0]]], dtype=dtype))
    assert be.batched_matmul(x, x).to_numpy()[0, 0, 0] == 9.0


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_epilogue_bias_relu_accumulate(tt, oracle, dtype):
    rng = np.random.default_rng(21)
    X = rng.integers(-4, 5, (200, 96)).astype(dtype)
    W = rng.integers(-4, 5, (96, 136)).astype(dtype)
    b = rng.integers(-4, 5, (136,)).astype(dtype)
    want = X @ W + b  # small integers: exact in both dtypes
    got = tt.linear(dev(tt, X), dev(tt, W), dev(tt, b)).to_numpy()
    assert np.array_equal(got, want)
    got = tt.linear(dev(tt, X), dev(tt, W), dev(tt, b), relu=True).to_numpy()
    assert np.array_equal(got, np.maximum(want, 0))
    be = tt.get_backend(tt.kAMD)
    acc = dev(tt, np.ones((1, 200, 136), dtype=dtype))
    be.batched_matmul(dev(tt, X[None]), dev(tt, W[None]), out=acc, accumulate=True)
    assert np.array_equal(acc.to_numpy()[0], X @ W + 1)
    rb = rng.integers(-4, 5, (200,)).astype(dtype)
    got = be.batched_matmul(dev(tt, X[None]), dev(tt, W[None]), bias=dev(tt, rb), bias_mode=2).to_numpy()[0]
    assert np.array_equal(got, X @ W + rb[:, None])
    # thin output (split-K path: the epilogue runs in the reduction kernel) takes the same epilogue
    W10 = rng.integers(-4, 5, (96, 10)).astype(dtype)
    b10 = rng.integers(-4, 5, (10,)).astype(dtype)
    got = tt.linear(dev(tt, X), dev(tt, W10), dev(tt, b10), relu=True).to_numpy()
    assert np.array_equal(got, np.maximum(X @ W10 + b10, 0))


# The big tiles exist as separate plain-store and full-epilogue kernels; these shapes select them (asserted) with
# ragged edges in both directions.  Small integers and a short K keep every result exact, so the bar is bit-exact.
@pytest.mark.parametrize("dtype,N,M,layout,tile", [
    (np.float32, 3900, 4000, "nn", "256x256"), (np.float32, 3900, 3999, "nt", "256x256"),
    (np.float32, 3904, 4000, "tn", "256x256"), (np.float32, 3904, 3999, "tt", "256x256"),
    (np.float32, 6100, 6000, "nn", "128x128"), (np.float32, 6100, 5999, "nt", "128x128"),
    # 192 x 192 (3 x 3 MFMA blocks per wave): only for outputs made of whole tiles
    (np.float32, 3072, 3072, "nn", "192x192"), (np.float32, 3072, 3072, "nt", "192x192"),
    (np.float32, 3072, 3072, "tn", "192x192"), (np.float32, 3072, 3072, "tt", "192x192"), (np.float32, 4224, 4224, "nn", "192x192"),
    (np.float64, 3900, 4000, "nn", "256x128"), (np.float64, 3900, 3999, "nt", "256x128"),
    (np.float64, 3904, 4000, "tn", "256x128"),
])
def test_big_tile_epilogues_and_edges(tt, dtype, N, M, layout, tile):
    K = 40
    rng = np.random.default_rng(N + M)
    ints = lambda *shape: rng.integers(-4, 5, shape).astype(dtype)
    A = ints(1, N, K) if layout[0] == "n" else ints(1, K, N).transpose(0, 2, 1)
    B = ints(1, K, M) if layout[1] == "n" else ints(1, M, K).transpose(0, 2, 1)
    tA, tB = to_dev_view(tt, A), to_dev_view(tt, B)
    be = tt.get_backend(tt.kAMD)
    assert f"_{tile}_" in be.batched_matmul_variant(tA, tB)
    want = A[0].astype(np.float64) @ B[0].astype(np.float64)  # exact: |sum| <= 40 * 16
    assert np.array_equal(be.batched_matmul(tA, tB).to_numpy()[0], want)
    col_bias, row_bias, prev = ints(M), ints(N), ints(1, N, M)
    got = be.batched_matmul(tA, tB, bias=dev(tt, col_bias), bias_mode=1, relu=True).to_numpy()[0]
    assert np.array_equal(got, np.maximum(want + col_bias, 0))
    acc = dev(tt, prev)
    be.batched_matmul(tA, tB, out=acc, bias=dev(tt, row_bias), bias_mode=2, accumulate=True)
    assert np.array_equal(acc.to_numpy()[0], want + row_bias[:, None] + prev[0])


# Long reductions on few 64 x 64 tiles run with four k tiles in flight (static register slots per group of steps),
# short or crowded ones with two: both depths, all layouts, k tails and exact multiples, both dtypes.  Small integers
# keep the sums exact.
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("shape", [(320, 1024, 448), (200, 1000, 420), (64, 4100, 64), (704, 520, 1344), (448, 48, 320)])
def test_small_tile_prefetch_depths(tt, dtype, layout, shape):
    N, K, M = shape
    rng = np.random.default_rng(N + K + M)
    ints = lambda *sh: rng.integers(-3, 4, sh).astype(dtype)
    A = ints(2, N, K) if layout[0] == "n" else ints(2, K, N).transpose(0, 2, 1)
    B = ints(2, K, M) if layout[1] == "n" else ints(2, M, K).transpose(0, 2, 1)
    tA, tB = to_dev_view(tt, A), to_dev_view(tt, B)
    assert "_64x64_" in tt.get_backend(tt.kAMD).batched_matmul_variant(tA, tB)
    got = tt.matmul(tA, tB).to_numpy()
    assert np.array_equal(got, np.matmul(A.astype(np.float64), B.astype(np.float64)))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("shape", [(1024, 1024, 1024), (1000, 512, 1001), (784, 1024, 1024), (130, 2048, 70), (1024, 832, 512),
                                   (1024, 784, 1024), (960, 1000, 1024), (1024, 516, 1024),
                                   # the 128 x 128 tile (fp32) with a reduction of 2048 or more: whole and ragged tiles
                                   (2048, 2048, 2048), (1900, 2056, 1988)])
def test_two_halves_of_k_in_one_workgroup(tt, dtype, layout, shape):
    """Launches with at most one 64x64 workgroup per CU split the reduction between the two halves of a 512-lane
    workgroup when both halves have the same number of k tiles (784 = 392 + 392 and 1000 = 500 + 500 end in partial
    tiles; 516 = 260 + 256 has unequal tile counts and takes the ordinary kernel); exact on integer-valued data, with
    and without the epilogue, ragged edges included.  (1000 x 512 x 1001 has rows that are not whole 16-byte vectors
    in some layouts and then takes the ordinary kernels: the name is only asserted where the variant is expected.)"""
    N, K, M = shape
    rng = np.random.default_rng(N + K + M)
    ints = lambda *sh: rng.integers(-3, 4, sh).astype(dtype)
    A = ints(1, N, K) if layout[0] == "n" else ints(1, K, N).transpose(0, 2, 1)
    B = ints(1, K, M) if layout[1] == "n" else ints(1, M, K).transpose(0, 2, 1)
    tA, tB = to_dev_view(tt, A), to_dev_view(tt, B)
    be = tt.get_backend(tt.kAMD)
    name = be.batched_matmul_variant(tA, tB)
    if shape in ((1024, 1024, 1024), (784, 1024, 1024), (1024, 832, 512), (1024, 784, 1024), (960, 1000, 1024)):
        assert name.endswith("_halves"), name
    if shape[1] >= 2048 and shape[0] > 1024 and dtype == np.float32:
        assert name.startswith("mfma_f32_128x128") and name.endswith("_halves"), name
    if shape == (1024, 516, 1024) and dtype == np.float32:  # fp64 (k tile 16): 258 + 258, 17 tiles each
        assert not name.endswith("_halves"), name
    want = np.matmul(A.astype(np.float64), B.astype(np.float64))
    assert np.array_equal(be.batched_matmul(tA, tB).to_numpy(), want)
    bias = ints(M)
    got = be.batched_matmul(tA, tB, bias=dev(tt, bias), bias_mode=1, relu=True).to_numpy()
    assert np.array_equal(got, np.maximum(want + bias, 0))
    prev = ints(1, N, M)
    acc = dev(tt, prev)
    be.batched_matmul(tA, tB, out=acc, accumulate=True)
    assert np.array_equal(acc.to_numpy(), want + prev)


def test_contiguous_identity(tt, oracle):
    rng = np.random.default_rng(2)
    for dtype in (np.uint8, np.int16, np.float32, np.float64):
        a = rng.integers(0, 100, (5, 6, 7)).astype(dtype)
        t = dev(tt, a).permute(2, 0, 1)
        assert not t.is_contiguous()
        got = t.contiguous()
        assert got.is_contiguous() and np.array_equal(got.to_numpy(), oracle.contiguous(a.transpose(2, 0, 1)))
    e = dev(tt, np.arange(4, dtype=np.float32)).reshape([1, 4]).expand([3, 4]).contiguous()
    assert np.array_equal(e.to_numpy(), np.tile(np.arange(4, dtype=np.float32), (3, 1)))


def test_memory_counters_and_device_errors(tt):
    be = tt.get_backend(tt.kAMD)
    assert be.get_device_count() >= 1
    cur0, tot0 = be.current_memory_allocated(0), be.total_memory_allocated(0)
    t = tt.Tensor.from_numpy(np.zeros(1024, dtype=np.float32))
    assert be.current_memory_allocated(0) == cur0 + 4096 and be.total_memory_allocated(0) == tot0 + 4096
    del t
    assert be.current_memory_allocated(0) == cur0 and be.total_memory_allocated(0) == tot0 + 4096
    with pytest.raises(tt.TTException):  # out-of-range device id throws (cuda/backend_cuda.cpp:53-63)
        tt.Tensor.from_numpy(np.zeros(4, dtype=np.float32), tt.Device("amd", be.get_device_count()))


def test_freed_blocks_are_cached_and_reused(tt):
    import ctypes as C
    lib = tt._capi.lib
    cached = C.c_uint64()

    def cached_bytes():
        assert lib.ttamd_memory_cached(0, C.byref(cached)) == 0
        return cached.value

    assert lib.ttamd_empty_cache(0) == 0 and cached_bytes() == 0
    p, q = C.c_void_p(), C.c_void_p()
    assert lib.ttamd_malloc(0, 5000, C.byref(p)) == 0           # size class 5120 (multiples of 512 up to 8 KiB)
    first = p.value
    assert lib.ttamd_free(0, p, 5000) == 0
    assert cached_bytes() == 5120
    assert lib.ttamd_malloc(0, 4700, C.byref(q)) == 0           # same class: the cached block comes back
    assert q.value == first and cached_bytes() == 0
    assert lib.ttamd_malloc(0, 5000, C.byref(p)) == 0 and p.value != first   # the class is empty again: a new block
    assert lib.ttamd_free(0, p, 5000) == 0 and lib.ttamd_free(0, q, 4700) == 0
    assert cached_bytes() == 2 * 5120
    assert lib.ttamd_empty_cache(0) == 0 and cached_bytes() == 0
    # results stay correct when every temporary of a chain of operations recycles blocks
    a = np.arange(12, dtype=np.float32).reshape(3, 4)
    t = tt.Tensor.from_numpy(a)
    for _ in range(50):
        t = (t + t) * tt.Tensor.from_numpy(np.full((3, 4), 0.5, np.float32))
    assert np.array_equal(t.to_numpy(), a)


# ----------------------------------------------------------------------------- full-size properties (config 3)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_config3_4096_properties(tt, oracle, dtype):
    n = 4096
    A = oracle.Generator(0).uniform_real(-1, 1, (n, n), dtype)
    B = oracle.Generator(1).uniform_real(-1, 1, (n, n), dtype)
    tA, tB = dev(tt, A), dev(tt, B)
    Cg = tt.matmul(tA, tB).to_numpy()
    # (1) a band of rows and a band of columns against the oracle (each a 64 x 4096 x 4096 / 4096 x 4096 x 64 product)
    rows = slice(1000, 1064)
    check_close(Cg[rows], oracle.matmul(A[rows], B), A[rows], B, dtype)
    cols = slice(3000, 3064)
    check_close(Cg[:, cols], oracle.matmul(A, np.ascontiguousarray(B[:, cols])), A, B[:, cols], dtype)
    # (2) checksum identity: (A.B).1 = A.(B.1) and 1^T.(A.B) = (1^T.A).B in f64
    ones = np.ones(n)
    eps = 2.0**-24 if dtype == np.float32 else 2.0**-53
    lhs = Cg.astype(np.float64) @ ones
    rhs = A.astype(np.float64) @ (B.astype(np.float64) @ ones)
    scale = np.abs(A).astype(np.float64) @ (np.abs(B).astype(np.float64) @ ones)
    assert np.max(np.abs(lhs - rhs) / scale) <= 256 * eps
    # (3) transposition identity through the strided path: (B^T.A^T)^T == A.B within tolerance
    Ct = tt.matmul(tB.permute(1, 0), tA.permute(1, 0)).to_numpy().T
    assert max_rel_error(Ct, Cg) <= tol_of(dtype)
    # (4) every element of the product against the oracle's whole 4096^3 product (a few seconds of one host core)
    check_close(Cg, oracle.matmul(A, B), A, B, dtype)
