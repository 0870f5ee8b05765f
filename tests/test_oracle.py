"""CPU-only tests that pin the oracle (oracle/tt_oracle.c) before anything is compared against it.

Each check is chosen so that a plausible slip in the restatement (dropped term, wrong index, transposed
operand, wrong shift) fails it; none of them re-types the oracle's own formula.
"""
import numpy as np
import pytest

from helpers import ALL_NON_BOOL, naive_exact, ref_batched, ref_dot, ref_mat_mat, ref_vec_mat


# ------------------------------------------------------------------------------------------- RNG
def test_splitmix64_published_vectors(oracle):
    # First outputs of Vigna's splitmix64.c stream seeded with 1234567: output n = mix(seed + n*gamma),
    # i.e. tto_splitmix64(seed + (n-1)*gamma) since the function adds gamma itself.
    gamma = 0x9E3779B97F4A7C15
    want = [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431, 16408922859458223821]
    got = [oracle.lib().tto_splitmix64((1234567 + n * gamma) % 2**64) for n in range(5)]
    assert got == want


def test_xorshift64_matches_bit_matrix_definition(oracle):
    # xorshift64 with shifts (13, 7, 17) is linear over GF(2): apply the three shift-xor steps with
    # Python big-int arithmetic as an independent statement, over many random states.
    import ctypes as C

    rng = np.random.default_rng(1)
    for s in rng.integers(1, 2**63, size=200, dtype=np.uint64):
        x = int(s)
        x ^= (x << 13) & (2**64 - 1)
        x ^= x >> 7
        x ^= (x << 17) & (2**64 - 1)
        st = C.c_uint64(int(s))
        assert oracle.lib().tto_xorshift64(C.byref(st)) == x
        assert st.value == x
    # period sanity: the all-zero state is the only fixed point
    st = C.c_uint64(0)
    assert oracle.lib().tto_xorshift64(C.byref(st)) == 0


def test_generator_seed_is_splitmix_of_seed(oracle):
    g = oracle.Generator(0)
    assert g.state == oracle.lib().tto_splitmix64(0) == 0xE220A8397B1DCDAF  # splitmix64(0), widely published


@pytest.mark.parametrize("dtype,shift,one", [(np.float32, 9, 0x3F800000), (np.float64, 12, 0x3FF0000000000000)])
def test_uniform_real_closed_form(oracle, dtype, shift, one):
    # Element i: own generator seeded with master output i; its first output x gives
    # r = bits((x_trunc >> shift) | one) - 1 in [0,1), then r*(hi-lo)+lo.  Rebuilt here from integers.
    n = 257
    g = oracle.Generator(7)
    master = oracle.Generator(7)
    got = g.uniform_real(-1.0, 1.0, (n,), dtype)
    import ctypes as C

    want = np.empty(n, dtype=dtype)
    for i in range(n):
        st = C.c_uint64(master())
        x = oracle.lib().tto_xorshift64(C.byref(st))
        if dtype == np.float32:
            bits = np.array([((x & 0xFFFFFFFF) >> shift) | one], dtype=np.uint32).view(np.float32)[0]
        else:
            bits = np.array([(x >> shift) | one], dtype=np.uint64).view(np.float64)[0]
        r = dtype(bits - dtype(1.0))
        want[i] = dtype(r * dtype(2.0)) + dtype(-1.0)
    assert np.array_equal(got, want)
    assert g.state == master.state  # exactly n master outputs consumed
    assert got.min() >= -1.0 and got.max() < 1.0


def test_uniform_real_statistics(oracle):
    x = oracle.Generator(0).uniform_real(0.0, 1.0, (200000,), np.float64)
    assert abs(x.mean() - 0.5) < 5e-3 and abs(x.var() - 1 / 12) < 2e-3
    # ECDF distance to U(0,1), like the reference's distribution tests (tests/test_distribution.cpp:85-180)
    xs = np.sort(x)
    assert np.max(np.abs(xs - (np.arange(xs.size) + 0.5) / xs.size)) < 5e-3


def test_normal_statistics(oracle):
    x = oracle.Generator(0).normal(0.0, 0.1, (200000,), np.float32).astype(np.float64)
    assert abs(x.mean()) < 2e-3 and abs(x.std() - 0.1) < 2e-3
    from scipy import stats

    assert stats.kstest(x, "norm", args=(0.0, 0.1)).statistic < 5e-3


def _element_uniforms(oracle, seed, n, dtype):
    """(u1, u2) of every element, rebuilt from the integer generator alone: element i owns a generator seeded with
    master output i; its first output makes u1 and its second u2 (bit construction of uniform_real_sample with
    low 0, high 1: r*(1-0)+0 == r exactly)."""
    import ctypes as C

    master = oracle.Generator(seed)
    u = np.empty((n, 2), dtype=dtype)
    for i in range(n):
        st = C.c_uint64(master())
        for j in range(2):
            x = oracle.lib().tto_xorshift64(C.byref(st))
            if dtype == np.float32:
                b = np.array([((x & 0xFFFFFFFF) >> 9) | 0x3F800000], dtype=np.uint32).view(np.float32)[0]
            else:
                b = np.array([(x >> 12) | 0x3FF0000000000000], dtype=np.uint64).view(np.float64)[0]
            u[i, j] = dtype(b - dtype(1.0))
    return u, master.state


def _box_muller_model(u1, u2, mu, std, dtype, variant="reference"):
    """mu + std*sqrt(-2*log1p(-u1))*sin(2*pi*u2) with every transcendental evaluated to 200 bits (mpmath) and each
    operation's result rounded to `dtype`, as code working in that type does.  Returns (value, std*z) as exact
    mpmath numbers of dtype-representable values.  The variants are deliberate mistakes (negative controls)."""
    import mpmath as mp

    mp.mp.prec = 200

    def rnd(v):  # round an mpmath number to dtype (to nearest even), back to mpmath
        if dtype == np.float64:
            return mp.mpf(float(v))  # mpf -> float rounds to nearest
        d = float(v)  # 53-bit first; 200 -> 53 -> 24 double rounding matters only on exact ties of the 53-bit value
        return mp.mpf(float(np.float32(d)))

    a, b = mp.mpf(float(u1)), mp.mpf(float(u2))
    if variant == "swapped":
        a, b = b, a
    if variant == "log_u1":
        lg = rnd(mp.log(a)) if a > 0 else mp.mpf("-inf")
    else:
        lg = rnd(mp.log1p(-a))
    r = rnd(mp.sqrt(-2 * lg))
    two_pi = 2 * rnd(mp.pi)
    theta = rnd(two_pi * b)
    trig = rnd(mp.cos(theta)) if variant == "cos" else rnd(mp.sin(theta))
    z = rnd(r * trig)
    sz = rnd(mp.mpf(float(std)) * z)
    return rnd(sz + mp.mpf(float(mu))), sz


@pytest.mark.parametrize("dtype,ulps", [(np.float32, 2), (np.float64, 4)])
def test_normal_closed_form(oracle, dtype, ulps):
    """Pins tto_normal_* (common/kernel/distribution.hpp:232-246) without libm: the Box-Muller value of every element
    is rebuilt from the integer generator and 200-bit transcendental evaluations.  A correctly rounded chain and a
    libm chain (each function within 1 ulp) differ by at most a few units in the last place of std*z; the three
    plausible slips (cos for sin, u1 and u2 swapped, log(u1) for log1p(-u1)) miss that bound on nearly every element."""
    n, seed, mu, std = 1000, 11, dtype(0.25), dtype(0.1)
    g = oracle.Generator(seed)
    got = g.normal(float(mu), float(std), (n,), dtype)
    u, master_state = _element_uniforms(oracle, seed, n, dtype)
    assert g.state == master_state  # n master outputs consumed, nothing else

    def misses(variant):
        bad = 0
        for i in range(n):
            want, sz = _box_muller_model(u[i, 0], u[i, 1], mu, std, dtype, variant)
            if not np.isfinite(float(want)):
                bad += 1
                continue
            # libm's log1p, sqrt, sin are within 1 ulp each: `ulps` units of std*z cover the chain, plus one unit of
            # the final sum (an addend that moved by a unit can tip the sum's rounding to the neighbouring value, and
            # the sum may or may not be contracted into an fma).
            tol = ulps * float(np.spacing(dtype(abs(float(sz))))) + float(np.spacing(dtype(abs(float(want)))))
            if abs(float(got[i]) - float(want)) > tol:
                bad += 1
        return bad

    assert misses("reference") == 0
    for wrong in ("cos", "swapped", "log_u1"):
        assert misses(wrong) > 0.95 * n, wrong


def test_normal_zero_mean_keeps_relative_accuracy(oracle):
    # With mu = 0 (config 4's inputs: normal(0, 0.1)) the value is std*z itself: every element within 4 ulp of the
    # 200-bit evaluation, including the small ones where sin(theta) is near a zero crossing.
    n, seed = 500, 0
    got = oracle.Generator(seed).normal(0.0, 0.1, (n,), np.float32)
    u, _ = _element_uniforms(oracle, seed, n, np.float32)
    for i in range(n):
        want, _sz = _box_muller_model(u[i, 0], u[i, 1], np.float32(0.0), np.float32(0.1), np.float32)
        assert abs(float(got[i]) - float(want)) <= 4 * float(np.spacing(np.float32(abs(float(want))))), i


# ------------------------------------------------------------------------------------------- contiguous
def test_contiguous_matches_nested_loops(oracle):
    rng = np.random.default_rng(0)
    base = rng.integers(-100, 100, size=4 * 5 * 6 * 3 + 11).astype(np.int32)
    v = np.lib.stride_tricks.as_strided(base[7:], shape=(3, 4, 5), strides=(4 * 4, 0, 3 * 4 * 4))  # overlap + stride 0
    got = oracle.contiguous(v)
    want = np.empty((3, 4, 5), dtype=np.int32)
    for i in range(3):
        for j in range(4):
            for k in range(5):
                want[i, j, k] = base[7 + i * 4 + j * 0 + k * 12]
    assert np.array_equal(got, want)
    t = rng.random((5, 7, 3))
    assert np.array_equal(oracle.contiguous(t.transpose(2, 0, 1)), np.ascontiguousarray(t.transpose(2, 0, 1)))


# ------------------------------------------------------------------------------------------- GEMM
@pytest.mark.parametrize("dtype", ALL_NON_BOOL)
def test_matmul_kernel_reference_patterns_exact(oracle, dtype):
    # tests/test_matmul.cpp:163-187 data; exact integer answer computed with 64-bit integer arithmetic.
    lhs, rhs = ref_mat_mat(dtype, N=131, M=203, K=77)
    want = naive_exact(lhs, rhs)
    assert np.array_equal(oracle.matmul_kernel(lhs, rhs), want)
    assert np.array_equal(oracle.matmul_naive(lhs, rhs), want)
    assert np.array_equal(oracle.matmul_blocked_scalar(lhs, rhs), want)


@pytest.mark.parametrize("dtype", [np.float32, np.int32, np.uint8])
def test_matmul_kernel_reference_size_exact(oracle, dtype):
    lhs, rhs = ref_mat_mat(dtype)  # 379 x 1147 x 635, as in the reference test
    assert np.array_equal(oracle.matmul_kernel(lhs, rhs), naive_exact(lhs, rhs))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", [(1, 1, 1), (8, 64, 16), (37, 101, 53), (64, 65, 64), (9, 200, 17), (130, 129, 70)])
def test_tiled_kernel_is_bit_identical_to_scalar_statement(oracle, dtype, shape):
    # Two independent statements of the summation order (8x4-vector tiles over padded scratch vs a
    # per-element loop with explicit fma) must agree bit for bit, in both contraction flavours.
    N, K, M = shape
    rng = np.random.default_rng(sum(shape))
    A = rng.uniform(-1, 1, (N, K)).astype(dtype)
    B = rng.uniform(-1, 1, (K, M)).astype(dtype)
    for fl in ("fma", "nofma"):
        assert np.array_equal(oracle.matmul_kernel(A, B, fl), oracle.matmul_blocked_scalar(A, B, fl))
    assert np.array_equal(oracle.matmul_kernel(A, B, "fast"), oracle.matmul_kernel(A, B, "fma"))


def test_blocked_order_is_really_blocks_of_64(oracle):
    # Cancellation probe: a = [2^25, 1 x 63, -2^25, 1 x 63] against b = ones.  Within a block of 64 the running
    # f32 sum +-2^25 + 1 + 1 ... stays +-2^25 (every +1 is a tie that rounds back to the even mantissa), so
    # block 0 gives 2^25, block 1 gives -2^25, total 0.  A plain left-to-right sum over all 128 terms gives
    # 2^25 (63 lost) - 2^25 + 63 = 63; pairwise or 128-wide blocking give yet other values.
    a = np.array([[2.0**25] + [1.0] * 63 + [-(2.0**25)] + [1.0] * 63], dtype=np.float32)
    b = np.ones((128, 1), dtype=np.float32)
    for fl in ("fma", "nofma"):
        assert oracle.matmul_kernel(a, b, fl)[0, 0] == 0.0
        assert oracle.matmul_blocked_scalar(a, b, fl)[0, 0] == 0.0
    seq = np.float32(0)
    for x in a[0]:
        seq = np.float32(seq + x)
    assert seq == 63.0


def test_fma_flavour_differs_from_mul_add_flavour(oracle):
    # -1 + (1+e)(1-e) with e = 2^-13: the exact product 1 - 2^-26 is not an f32 (it rounds to 1), so
    # mul-then-add gives 0 while a fused multiply-add keeps -2^-26.
    assert oracle.lib("fma").tto_uses_fma() == 1 and oracle.lib("nofma").tto_uses_fma() == 0
    e = np.float32(2.0**-13)
    A = np.array([[1.0, 1 + e]], dtype=np.float32)
    B = np.array([[-1.0], [1 - e]], dtype=np.float32)
    for fn in (oracle.matmul_kernel, oracle.matmul_blocked_scalar):
        assert fn(A, B, "fma")[0, 0] == np.float32(-(2.0**-26))
        assert fn(A, B, "nofma")[0, 0] == 0.0


@pytest.mark.parametrize("dtype,tol", [(np.float32, 64 * 2.0**-24), (np.float64, 64 * 2.0**-53)])
def test_matmul_kernel_close_to_high_precision(oracle, dtype, tol):
    rng = np.random.default_rng(3)
    A = rng.uniform(-1, 1, (70, 300)).astype(dtype)
    B = rng.uniform(-1, 1, (300, 90)).astype(dtype)
    want = A.astype(np.longdouble) @ B.astype(np.longdouble)
    scale = np.abs(A).astype(np.longdouble) @ np.abs(B).astype(np.longdouble)
    err = np.max(np.abs(oracle.matmul_kernel(A, B).astype(np.longdouble) - want) / scale)
    # blocks of 64 sequential terms + 5 block additions: error well under (64 + 5) ulps on this scale
    assert err < 2 * tol


def test_batched_matmul_views_equal_dense_copies(oracle):
    # benchmark configuration 2: B is a transposed view of a [32,128,64] tensor.
    A = oracle.Generator(0).uniform_real(-1, 1, (32, 128, 64))
    Bsrc = oracle.Generator(1).uniform_real(-1, 1, (32, 128, 64))
    Bv = Bsrc.transpose(0, 2, 1)
    assert oracle.elem_strides(Bv) == [8192, 1, 64]
    got = oracle.batched_matmul(A, Bv)
    want = oracle.batched_matmul(A, np.ascontiguousarray(Bv))
    assert np.array_equal(got, want)
    for b in (0, 31):
        assert np.array_equal(got[b], oracle.matmul_kernel(A[b], np.ascontiguousarray(Bv[b])))
    # transposition identity (A.B)^T = B^T.A^T on integer data is exact
    Ai = np.round(A * 8).astype(np.float32)
    Bi = np.round(Bv * 8).astype(np.float32)
    left = oracle.batched_matmul(Ai, Bi).transpose(0, 2, 1)
    right = oracle.batched_matmul(Bi.transpose(0, 2, 1), Ai.transpose(0, 2, 1))
    assert np.array_equal(left, right)


@pytest.mark.parametrize("dtype", ALL_NON_BOOL)
def test_reference_small_cases(oracle, dtype):
    # dot 12 and 2048 (tests/test_matmul.cpp:59-85), vec.mat (:99-118), batched (:200-236, reduced size)
    for n in (12, 2048):
        a, b = ref_dot(n, dtype)
        want = naive_exact(a[None, :], b[:, None]).reshape(-1)
        got = oracle.matmul(a, b)
        if dtype == np.float32 and n == 2048:
            # the exact sum 2.88e9 exceeds 2^24: the reference compares with allclose(rtol 1e-5)
            assert np.allclose(got, (a.astype(np.float64) @ b.astype(np.float64)), rtol=1e-5)
        else:
            assert np.array_equal(got, want)
    v, m = ref_vec_mat(dtype)
    assert np.array_equal(oracle.matmul(v, m), naive_exact(v[None, :], m)[0])
    lhs, rhs = ref_batched(dtype, B=4, N=37, M=130, K=41)
    want = np.stack([naive_exact(lhs[b], rhs[b]) for b in range(4)])
    assert np.array_equal(oracle.matmul(lhs, rhs), want)


def test_matmul_backward_closed_forms(oracle):
    # dA = dC.B^T, dB = A^T.dC (autograd/binary_ops.cpp:162-179) checked by the adjoint identity
    # <dC, A.B> = <dA, A> = <dB, B> on integer-valued f64 data (exact) ...
    rng = np.random.default_rng(5)
    A = rng.integers(-4, 5, (3, 9, 14)).astype(np.float64)
    B = rng.integers(-4, 5, (3, 14, 6)).astype(np.float64)
    dC = rng.integers(-4, 5, (3, 9, 6)).astype(np.float64)
    dA, dB = oracle.matmul_backward(A, B, dC)
    fwd = oracle.matmul(A, B)
    assert np.sum(dC * fwd) == np.sum(dA * A) == np.sum(dB * B)
    # ... and by central finite differences of L = <dC, A.B> in one coordinate of each operand
    A[1, 2, 3] += 0.5
    up = np.sum(dC * oracle.matmul(A, B))
    A[1, 2, 3] -= 1.0
    dn = np.sum(dC * oracle.matmul(A, B))
    assert up - dn == dA[1, 2, 3]


# ------------------------------------------------------------------------------------------- conv
def _conv_brute(x, w, S, P):
    Bn, Cc, H, W = x.shape
    O, _, k, _ = w.shape
    xp = np.zeros((Bn, Cc, H + 2 * P, W + 2 * P), dtype=np.float64)
    xp[:, :, P:P + H, P:P + W] = x
    Ho, Wo = (H + 2 * P - k) // S + 1, (W + 2 * P - k) // S + 1
    out = np.zeros((Bn, O, Ho, Wo))
    for h in range(Ho):
        for ww in range(Wo):
            patch = xp[:, :, S * h:S * h + k, S * ww:S * ww + k]
            out[:, :, h, ww] = np.einsum("bcpq,ocpq->bo", patch, w)
    return out


@pytest.mark.parametrize("S,P", [(1, 0), (2, 1), (1, 1), (3, 2)])
def test_im2col_maps_brute_force(oracle, S, P):
    import ctypes as C

    Cc, H, W, k = 3, 7, 6, 3
    x = np.arange(2 * Cc * H * W, dtype=np.float64).reshape(2, Cc, H, W) + 1
    Ho, Wo = (H + 2 * P - k) // S + 1, (W + 2 * P - k) // S + 1
    xu = np.zeros((Cc * k * k, Ho * Wo))
    oracle.lib().tto_unroll_f64(C.c_void_p(x.ctypes.data), C.c_void_p(xu.ctypes.data), 1, Cc, H, W, k, S, P)
    xp = np.zeros((Cc, H + 2 * P, W + 2 * P))
    xp[:, P:P + H, P:P + W] = x[1]
    want = np.stack([xp[c, p:p + S * Ho:S, q:q + S * Wo:S].reshape(-1) for c in range(Cc) for p in range(k) for q in range(k)])
    assert np.array_equal(xu, want)
    xut = np.zeros((Ho * Wo, Cc * k * k))
    oracle.lib().tto_unroll_transpose_f64(C.c_void_p(x.ctypes.data), C.c_void_p(xut.ctypes.data), 1, Cc, H, W, k, S, P)
    assert np.array_equal(xut, want.T)
    # col2im is the adjoint of im2col: <col2im(U), X> == <U, im2col(X)> for integer-valued data
    rng = np.random.default_rng(0)
    U = rng.integers(-3, 4, xu.shape).astype(np.float64)
    back = np.zeros((Cc, H, W))
    oracle.lib().tto_col2im_f64(C.c_void_p(back.ctypes.data), C.c_void_p(U.ctypes.data), 0, Cc, H, W, k, S, P)
    x0 = np.zeros((Cc * k * k, Ho * Wo))
    oracle.lib().tto_unroll_f64(C.c_void_p(x.ctypes.data), C.c_void_p(x0.ctypes.data), 0, Cc, H, W, k, S, P)
    assert np.sum(back * x[0]) == np.sum(U * x0)


@pytest.mark.parametrize("dtype", ALL_NON_BOOL)
@pytest.mark.parametrize("S,P", [(1, 0), (2, 1)])
def test_conv_forward_reference_pattern(oracle, dtype, S, P):
    # tests/test_conv.cpp:99-143 data pattern (i % 10) at reduced size; naive 7-loop and, for floats, an
    # independent einsum over padded patches.
    Bn, Cc, O, H, W, k = 2, 3, 16, 12, 11, 3
    x = (np.arange(Bn * Cc * H * W) % 10).astype(dtype).reshape(Bn, Cc, H, W)
    w = (np.arange(O * Cc * k * k) % 10).astype(dtype).reshape(O, Cc, k, k)
    got = oracle.conv2d_forward(x, w, None, S, P)
    assert np.array_equal(got, oracle.conv2d_naive(x, w, S, P))
    if np.issubdtype(dtype, np.floating) or dtype == np.int64:
        assert np.array_equal(got.astype(np.float64), _conv_brute(x.astype(np.float64), w.astype(np.float64), S, P))


def test_conv_forward_bias_and_backward_adjoints(oracle):
    rng = np.random.default_rng(2)
    Bn, Cc, O, H, W, k, S, P = 3, 4, 5, 9, 8, 3, 2, 1
    x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(np.float64)
    w = rng.integers(-3, 4, (O, Cc, k, k)).astype(np.float64)
    b = rng.integers(-3, 4, (O,)).astype(np.float64)
    out = oracle.conv2d_forward(x, w, b, S, P)
    assert np.array_equal(out, _conv_brute(x, w, S, P) + b[None, :, None, None])
    g = rng.integers(-3, 4, out.shape).astype(np.float64)
    gx, gw, gb = oracle.conv2d_backward(g, x, w, True, S, P)
    lin = oracle.conv2d_forward(x, w, None, S, P)
    # conv is bilinear in (x, w): <g, conv(x,w)> = <gx, x> = <gw, w>; gb = sum of g over batch and space
    assert np.sum(g * lin) == np.sum(gx * x) == np.sum(gw * w)
    assert np.array_equal(gb, g.sum(axis=(0, 2, 3)))
    # and gx, gw are the gradients themselves, not merely something with the right inner product:
    e = np.zeros_like(x)
    e[1, 2, 3, 4] = 1.0
    assert np.sum(g * oracle.conv2d_forward(e, w, None, S, P)) == gx[1, 2, 3, 4]
    ew = np.zeros_like(w)
    ew[3, 1, 2, 0] = 1.0
    assert np.sum(g * oracle.conv2d_forward(x, ew, None, S, P)) == gw[3, 1, 2, 0]


def test_linear_default_init(oracle):
    # nn::Linear(784, 16): W [in,out] ~ U(+-sqrt(3)/sqrt(784)), b ~ U(+-1/sqrt(784)); construction order W then b.
    g = oracle.Generator(0)
    W, b = oracle.linear_init(g, 784, 16)
    assert W.shape == (784, 16) and b.shape == (16,)
    bw, bb = np.sqrt(3.0) / 28.0, 1.0 / 28.0
    assert np.abs(W).max() < bw and np.abs(W).max() > 0.99 * bw
    assert np.abs(b).max() < bb and np.abs(b).max() > 0.5 * bb
    g2 = oracle.Generator(0)
    W2 = g2.uniform_real(-bw, bw, (784, 16))
    assert np.array_equal(W, W2)
    # the bias is the SECOND draw of the same generator at bound 1/sqrt(in) (nn/linear.cpp:33-38, nn/init.cpp:106-112),
    # exactly: a bound from the wrong fan (out = 16 -> 0.25) or a fresh generator gives other values
    assert np.array_equal(b, g2.uniform_real(-bb, bb, (16,)))
    assert g.state == g2.state
    assert not np.array_equal(b, oracle.Generator(0).uniform_real(-bb, bb, (16,)))
    assert abs(W.astype(np.float64).var() - bw * bw / 3) < 2e-5


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_in_place_draw_through_a_view_brute_force(oracle, dtype):
    # Tensor::uniform_real_ on a view (cpu/kernel/distribution.hpp:28-32): the i-th element in the view's row-major
    # order takes the i-th draw.  Independent statement: the dense draw of the same generator, scattered by explicit
    # index loops over the view's shape -- for a permuted view with an offset, and for a sliced (strided) one.
    base = np.full((5, 4, 3, 6), -7.0, dtype=dtype)
    view = base.transpose(1, 0, 2, 3)[1:, :, :, 2:5]  # shape [3,5,3,3], offset and non-dense strides
    g = oracle.Generator(9)
    g.uniform_real_(view, -0.5, 0.25)
    dense = oracle.Generator(9).uniform_real(-0.5, 0.25, (view.size,), dtype)
    want = np.full((5, 4, 3, 6), -7.0, dtype=dtype)
    i = 0
    for a in range(3):
        for b in range(5):
            for c in range(3):
                for d in range(3):
                    want[b, a + 1, c, d + 2] = dense[i]
                    i += 1
    assert np.array_equal(base, want)  # the drawn elements AND the untouched ones
    g2 = oracle.Generator(9)
    g2.uniform_real(-0.5, 0.25, (view.size,), dtype)
    assert g.state == g2.state  # one master output per element, nothing else


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("dist", [0, 1])
def test_draws_with_a_parameter_pair_per_element_brute_force(oracle, dtype, dist):
    # The tensor forms of uniform_real_ / normal_ (cpu/distribution.cpp:96-139): element i of the view takes the i-th
    # master output as its state and the i-th pair of the (contiguous) parameters.  Independent statement, element by
    # element: a dense draw from the same seed with that element's pair as the scalars agrees at index i -- every
    # element depends on its own state and its own pair only.
    rng = np.random.default_rng(5)
    base = np.full((4, 6, 5), -7.0, dtype=dtype)
    view = base.transpose(1, 0, 2)[1:, :, 1:4]              # shape [5,4,3], permuted, offset, non-dense
    n = view.size
    p0 = rng.uniform(-2.0, 1.0, view.shape).astype(dtype)
    p1 = (p0 + rng.uniform(0.1, 3.0, view.shape)).astype(dtype) if dist == 0 else rng.uniform(0.1, 2.0, view.shape).astype(dtype)
    g = oracle.Generator(21)
    g.draw_params_(view, dist, p0, p1)
    want = np.full((4, 6, 5), -7.0, dtype=dtype)
    i = 0
    for a in range(5):
        for b in range(4):
            for c in range(3):
                ref = oracle.Generator(21)
                dense = (ref.uniform_real if dist == 0 else ref.normal)(float(p0[a, b, c]), float(p1[a, b, c]), (n,), dtype)
                want[b, a + 1, c + 1] = dense[i]
                i += 1
    assert np.array_equal(base, want)
    assert g.state == ref.state                              # n master outputs consumed
    # exchanging the two parameter tensors, or reading them in the view's storage order, gives other values
    other = np.full((4, 6, 5), -7.0, dtype=dtype)
    oview = other.transpose(1, 0, 2)[1:, :, 1:4]
    oracle.Generator(21).draw_params_(oview, dist, np.ascontiguousarray(p0.transpose(1, 0, 2)).reshape(view.shape), p1)
    assert not np.array_equal(other, want)


def test_conv2d_default_init(oracle):
    # nn::Conv2d(3, 8, 5): weight [8,3,5,5] drawn through permute(1,0,2,3) with fan = 3*25 (the VIEW's size(0)), then
    # bias with fan = 8*25 (the weight's size(0)).  Independent statement: draw [3,8,5,5] densely, transpose with numpy.
    C_, O_, k = 3, 8, 5
    W, b = oracle.conv2d_init(oracle.Generator(4), C_, O_, k)
    assert W.shape == (O_, C_, k, k) and b.shape == (O_,)
    g = oracle.Generator(4)
    bw = np.sqrt(3.0) / np.sqrt(C_ * k * k)
    dense = g.uniform_real(-bw, bw, (C_, O_, k, k))
    assert np.array_equal(W, dense.transpose(1, 0, 2, 3))
    assert not np.array_equal(W, dense.reshape(O_, C_, k, k))  # a dense draw in storage order is a different tensor
    bb = 1.0 / np.sqrt(O_ * k * k)
    assert np.array_equal(b, g.uniform_real(-bb, bb, (O_,)))
    assert np.abs(W).max() < bw and np.abs(W).max() > 0.95 * bw and np.abs(b).max() < bb
    # the bias bound uses the out-channel fan: with the in-channel fan (1/sqrt(75) = 0.115) values up to that would appear
    assert bb < 0.0708 and np.abs(b).max() > 0.5 * bb
    Wn, bn = oracle.conv2d_init(oracle.Generator(4), C_, O_, k, bias=False)
    assert bn is None and np.array_equal(Wn, W)
