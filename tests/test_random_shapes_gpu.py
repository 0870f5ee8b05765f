"""Randomised GPU parity sweeps through the C ABI: many small GEMM and conv problems with random extents, layouts,
offsets, dtypes and epilogues, each checked against the CPU oracle (bit-exact for integer dtypes and for
integer-valued floats, K-scaled relative error <= 1e-4 / 1e-12 otherwise).  The seeds are fixed, so a failure
names a reproducible case."""
import numpy as np
import pytest

from helpers import max_rel_error, scaled_error, tol_of

pytestmark = pytest.mark.gpu

DTYPES = [np.uint8, np.int16, np.int32, np.int64, np.float32, np.float64]


def strided_operand(tt, rng, shape, dtype, integer_valued):
    """A [b, r, c] operand stored in a random layout: dense, transposed, padded rows, offset, or broadcast batch."""
    b, r, c = shape
    kind = rng.integers(0, 5)
    draw = (lambda s: rng.integers(-4, 5, s).astype(dtype)) if integer_valued else (lambda s: rng.uniform(-1, 1, s).astype(dtype))
    if np.dtype(dtype).kind == "u":
        draw = lambda s: rng.integers(0, 9, s).astype(dtype)
    if kind == 0:
        host = draw((b, r, c))
        return tt.Tensor.from_numpy(host), host
    if kind == 1:                                   # transposed storage
        store = draw((b, c, r))
        return tt.Tensor.from_numpy(store).permute(0, 2, 1), store.transpose(0, 2, 1)
    if kind == 2:                                   # padded rows and an offset
        pad, off = int(rng.integers(1, 6)), int(rng.integers(0, 7))
        flat = draw((off + b * r * (c + pad),))
        t = tt.Tensor.from_numpy(flat)
        view = tt.Tensor(t.storage, t.dtype, (b, r, c), (r * (c + pad), c + pad, 1), off)
        host = flat[off:].reshape(b, r, c + pad)[:, :, :c]
        return view, host
    if kind == 3:                                   # one matrix broadcast over the batch (stride 0)
        store = draw((1, r, c))
        return tt.Tensor.from_numpy(store).expand((b, r, c)), np.broadcast_to(store, (b, r, c))
    step = int(rng.integers(2, 4))                  # every step-th column of a wider matrix
    store = draw((b, r, c * step))
    t = tt.Tensor.from_numpy(store)
    return tt.Tensor(t.storage, t.dtype, (b, r, c), (r * c * step, c * step, step), 0), store[:, :, ::step]


@pytest.mark.parametrize("seed", range(6))
def test_random_gemms(tt, oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    be = tt.get_backend(tt.kAMD)
    for case in range(40):
        dtype = DTYPES[int(rng.integers(0, len(DTYPES)))]
        is_float = np.dtype(dtype).kind == "f"
        integer_valued = (not is_float) or bool(rng.integers(0, 2))
        b = int(rng.integers(1, 4))
        n, k, m = (int(rng.integers(1, 200)) for _ in range(3))
        if rng.integers(0, 8) == 0:
            k = int(rng.integers(300, 1500))        # long reductions: the split-K form
        A, hA = strided_operand(tt, rng, (b, n, k), dtype, integer_valued)
        B, hB = strided_operand(tt, rng, (b, k, m), dtype, integer_valued)
        got = be.batched_matmul(A, B).to_numpy()
        tag = f"seed {seed} case {case}: {np.dtype(dtype).name} b{b} {n}x{k}x{m} {be.batched_matmul_variant(A, B)}"
        if integer_valued:
            wide = np.int64 if not is_float else np.float64
            want = np.matmul(np.asarray(hA).astype(wide), np.asarray(hB).astype(wide)).astype(dtype)
            assert np.array_equal(got, want), tag
        else:
            want = oracle.matmul(np.ascontiguousarray(hA), np.ascontiguousarray(hB))
            for i in range(b):
                assert scaled_error(got[i], want[i], np.asarray(hA[i]), np.asarray(hB[i])) <= tol_of(dtype), tag


@pytest.mark.parametrize("seed", range(4))
def test_random_gemm_epilogues(tt, seed):
    rng = np.random.default_rng(2000 + seed)
    be = tt.get_backend(tt.kAMD)
    for case in range(25):
        dtype = [np.float32, np.float64][int(rng.integers(0, 2))]
        n, k, m = (int(rng.integers(1, 150)) for _ in range(3))
        a = rng.integers(-3, 4, (1, n, k)).astype(dtype)
        b = rng.integers(-3, 4, (1, k, m)).astype(dtype)
        mode = int(rng.integers(0, 3))
        relu, accumulate = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        bias = rng.integers(-5, 6, (m if mode == 1 else n,)).astype(dtype)
        base = rng.integers(-5, 6, (1, n, m)).astype(dtype)
        out = tt.Tensor.from_numpy(base.copy())
        be.batched_matmul(tt.Tensor.from_numpy(a), tt.Tensor.from_numpy(b), bias=tt.Tensor.from_numpy(bias) if mode else None,
                          bias_mode=mode, relu=relu, out=out, accumulate=accumulate)
        want = a @ b
        if mode == 1:
            want = want + bias[None, None, :]
        if mode == 2:
            want = want + bias[None, :, None]
        if relu:
            want = np.maximum(want, 0)
        if accumulate:
            want = want + base
        assert np.array_equal(out.to_numpy(), want.astype(dtype)), f"seed {seed} case {case}: {n}x{k}x{m} mode {mode} relu {relu} acc {accumulate}"


@pytest.mark.parametrize("seed", range(4))
def test_random_convs(tt, oracle, seed):
    rng = np.random.default_rng(3000 + seed)
    for case in range(20):
        dtype = [np.float32, np.float64][int(rng.integers(0, 2))]
        Bn, Cc, O = int(rng.integers(1, 4)), int(rng.integers(1, 40)), int(rng.integers(1, 80))
        k, S, P = int(rng.integers(1, 6)), int(rng.integers(1, 4)), int(rng.integers(0, 4))
        H, W = int(rng.integers(max(1, k - 2 * P), 22)), int(rng.integers(max(1, k - 2 * P), 22))
        x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(dtype)
        w = rng.integers(-3, 4, (O, Cc, k, k)).astype(dtype)
        bias = rng.integers(-3, 4, (O,)).astype(dtype)
        tag = f"seed {seed} case {case}: B{Bn} C{Cc} O{O} {H}x{W} k{k} s{S} p{P} {np.dtype(dtype).name}"
        tx, tw = tt.Tensor.from_numpy(x), tt.Tensor.from_numpy(w)
        out = tt.conv2d(tx, tw, tt.Tensor.from_numpy(bias), S, P).to_numpy()
        want = oracle.conv2d_forward(x, w, bias, S, P)
        assert np.array_equal(out, want), tag
        g = rng.integers(-3, 4, want.shape).astype(dtype)
        gx, gw, gb = tt.conv2d_backward(tt.Tensor.from_numpy(g), tx, tw, tt.Tensor.from_numpy(bias), S, P)
        wx, ww, wb = oracle.conv2d_backward(g, x, w, True, S, P)
        assert np.array_equal(gx.to_numpy(), wx), tag
        assert np.array_equal(gw.to_numpy(), ww), tag
        assert np.array_equal(gb.to_numpy(), wb), tag


@pytest.mark.parametrize("seed", range(4))
def test_random_stride_two_convs(tt, oracle, seed):
    """Stride-2 layers around the conditions of the vector gathers and of grad_input's one-launch classes: channel
    counts that are (mostly) multiples of 4, output rows of every length (whole vectors, padded rows, neither), kernels 1
    to 7 with every padding below them, odd and even extents, the input as a window of a NaN-filled tensor."""
    rng = np.random.default_rng(4000 + seed)
    for case in range(16):
        dtype = [np.float32, np.float64][int(rng.integers(0, 2))]
        Bn, O = int(rng.integers(1, 4)), int(rng.integers(1, 80))
        Cc = 4 * int(rng.integers(1, 12)) if rng.integers(0, 5) else int(rng.integers(1, 40))
        k = int(rng.integers(1, 8))
        P = int(rng.integers(0, k))
        H, W = int(rng.integers(max(1, k - 2 * P), 40)), int(rng.integers(max(1, k - 2 * P), 40))
        x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(dtype)
        w = rng.integers(-3, 4, (O, Cc, k, k)).astype(dtype)
        tag = f"seed {seed} case {case}: B{Bn} C{Cc} O{O} {H}x{W} k{k} s2 p{P} {np.dtype(dtype).name}"
        if rng.integers(0, 2):      # a window of a larger tensor (unit column stride), NaN around it
            big = np.full((Bn, Cc + 1, H + 2, W + 3), np.nan, dtype)
            big[:, 1:, 1:1 + H, 3:] = x
            tb = tt.Tensor.from_numpy(big)
            es = [s // big.itemsize for s in big.strides]
            tx = tt.Tensor(tb.storage, tb.dtype, (Bn, Cc, H, W), tuple(es), es[1] + es[2] + 3 * es[3])
        else:
            tx = tt.Tensor.from_numpy(x)
        tw = tt.Tensor.from_numpy(w)
        out = tt.conv2d(tx, tw, None, 2, P).to_numpy()
        want = oracle.conv2d_forward(x, w, None, 2, P)
        assert np.array_equal(out, want), tag
        g = rng.integers(-3, 4, want.shape).astype(dtype)
        gx, gw, gb = tt.conv2d_backward(tt.Tensor.from_numpy(g), tx, tw, None, 2, P)
        wx, ww, _ = oracle.conv2d_backward(g, x, w, False, 2, P)
        assert gb is None
        assert np.array_equal(gx.to_numpy(), wx), tag
        assert np.array_equal(gw.to_numpy(), ww), tag


@pytest.mark.parametrize("seed", range(8))
def test_random_lds_staged_convs(tt, oracle, seed):
    """Unit-stride fp32 layers inside and around the conditions of the kernels that keep an operand in LDS: 32 or 64
    input channels, 32 to 160 output channels, rows of whole 16-byte vectors, 1 x 1 to 3 x 3 taps with every padding below
    them, and batches from a few images to several hundred -- the plans of those kernels (tiles of 128 or of 192 + 4 / 8
    positions and how many waves, stages of how many rows, sets of waves) depend on all of these.  Forward with a bias and
    the whole backward pass, exact against the oracle on integer-valued data."""
    rng = np.random.default_rng(5000 + seed)
    for case in range(10):
        Cc, O = 32 * int(rng.integers(1, 3)), 32 * int(rng.integers(1, 6))
        k = int(rng.integers(1, 4))
        P = int(rng.integers(0, k))
        H, W = int(rng.integers(max(3, k), 34)), 4 * int(rng.integers(2, 9))
        Bn = int(rng.choice([2, 5, 40, 96, 130, 300]))
        if Bn * Cc * H * W > 6_000_000:   # (keeps the oracle's share of the run to seconds)
            Bn = max(2, 6_000_000 // (Cc * H * W))
        x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(np.float32)
        w = rng.integers(-3, 4, (O, Cc, k, k)).astype(np.float32)
        bias = rng.integers(-3, 4, (O,)).astype(np.float32)
        tag = f"seed {seed} case {case}: B{Bn} C{Cc} O{O} {H}x{W} k{k} s1 p{P}"
        tx, tw = tt.Tensor.from_numpy(x), tt.Tensor.from_numpy(w)
        out = tt.conv2d(tx, tw, tt.Tensor.from_numpy(bias), 1, P).to_numpy()
        want = oracle.conv2d_forward(x, w, bias, 1, P)
        assert np.array_equal(out, want), tag
        g = rng.integers(-3, 4, want.shape).astype(np.float32)
        gx, gw, gb = tt.conv2d_backward(tt.Tensor.from_numpy(g), tx, tw, tt.Tensor.from_numpy(bias), 1, P)
        wx, ww, wb = oracle.conv2d_backward(g, x, w, True, 1, P)
        assert np.array_equal(gx.to_numpy(), wx), tag
        assert np.array_equal(gw.to_numpy(), ww), tag
        assert np.array_equal(gb.to_numpy(), wb), tag


@pytest.mark.parametrize("seed", range(10))
def test_random_pairs_of_gradient_products(tt, seed):
    """ttamd_batched_matmul_pair on random Linear-layer sizes on both sides of the one-grid conditions (128 to 256 tiles of
    64 x 64 per product, reductions of 512 or more, dense fp32), with random batches, a ReLU mask, the right operand's column
    sums and, now and then, operands that are views: integer-valued data, every element exact, whichever way it ran."""
    rng = np.random.default_rng(9000 + seed)
    dtype = [np.float32, np.float32, np.float32, np.float64][int(rng.integers(0, 4))]
    batch = int(rng.choice([1, 1, 1, 2]))
    # rows n, in_features fin, out_features fout: dx = dy . W^T is [n, fin] with reduction fout, dW = x^T . dy is [fin, fout] with reduction n
    n = int(rng.choice([448, 512, 520, 640, 1000, 1024]))
    fin = int(rng.choice([500, 784, 1000, 1024, 1600]))
    fout = int(rng.choice([448, 512, 576, 1024, 1030]))
    if batch == 2:
        n, fin, fout = n // 2 + 8, fin // 2 + 4, max(fout // 2, 512)
    dy = rng.integers(-3, 4, (batch, n, fout)).astype(dtype)
    x = rng.integers(-3, 4, (batch, n, fin)).astype(dtype)
    w = rng.integers(-3, 4, (batch, fin, fout)).astype(dtype)
    z = rng.integers(-2, 3, (batch, n, fin)).astype(dtype)
    tdy, tx, tz = (tt.Tensor.from_numpy(v) for v in (dy, x, z))
    if seed % 3 == 2:   # the weight as a transposed store: dy . W^T then reads a plain matrix, a layout outside the pair's
        tw = tt.Tensor.from_numpy(np.ascontiguousarray(w.transpose(0, 2, 1))).permute(0, 2, 1)
    else:
        tw = tt.Tensor.from_numpy(w)
    be = tt.get_backend(tt.kAMD)
    db = tt.Tensor.empty((batch, fout), tdy.dtype)
    dx, dW = be.batched_matmul_pair((tdy, tw.permute(0, 2, 1), dict(relu_grad_input=tz)), (tx.permute(0, 2, 1), tdy, dict(rhs_colsum_out=db)))
    want_dx = np.matmul(dy.astype(np.float64), w.transpose(0, 2, 1).astype(np.float64)) * np.where(z < 0, 0.0, 1.0)
    want_dW = np.matmul(x.transpose(0, 2, 1).astype(np.float64), dy.astype(np.float64))
    assert np.array_equal(dx.to_numpy(), want_dx.astype(dtype)), (seed, batch, n, fin, fout, dtype)
    assert np.array_equal(dW.to_numpy(), want_dW.astype(dtype)), (seed, batch, n, fin, fout, dtype)
    assert np.array_equal(db.to_numpy(), dy.sum(1)), (seed, batch, n, fin, fout, dtype)
