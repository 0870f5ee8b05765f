"""GPU parity tests for ttamd_conv2d_forward / ttamd_conv2d_backward through the C ABI, against the CPU
oracle (im2col + the reference GEMM order) and the reference tests' own naive loop and data patterns
(tests/test_conv.cpp:29-143).  Float tolerance: max relative error <= 1e-4 (f32) / 1e-12 (f64); exact for the
integer dtypes and for integer-valued float data.
"""
import numpy as np
import pytest

from helpers import ALL_NON_BOOL, max_rel_error, tol_of

pytestmark = pytest.mark.gpu


def dev(tt, a):
    return tt.Tensor.from_numpy(a)


@pytest.mark.parametrize("dtype", ALL_NON_BOOL)
@pytest.mark.parametrize("S,P", [(1, 0), (2, 1)])
def test_forward_reference_pattern_exact(tt, oracle, dtype, S, P):
    # tests/test_conv.cpp:99-143: B4, C3 -> 128, 64x64, k3, data i % 10 (exact in every dtype; u8/i16 wrap)
    Bn, Cc, O, H, W, k = 4, 3, 128, 64, 64, 3
    x = (np.arange(Bn * Cc * H * W) % 10).astype(dtype).reshape(Bn, Cc, H, W)
    w = (np.arange(O * Cc * k * k) % 10).astype(dtype).reshape(O, Cc, k, k)
    got = tt.conv2d(dev(tt, x), dev(tt, w), None, S, P).to_numpy()
    want = oracle.conv2d_forward(x, w, None, S, P)
    assert got.shape == want.shape
    assert np.array_equal(got, want)
    if dtype in (np.float32, np.uint8):
        assert np.array_equal(want[:1], oracle.conv2d_naive(x[:1], w, S, P))  # the reference test's own oracle


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("geom", [
    # B, C, O, H, W, k, S, P
    (2, 5, 7, 9, 11, 3, 1, 1),
    (3, 4, 70, 13, 10, 5, 2, 2),
    (2, 3, 6, 8, 8, 1, 1, 0),
    (1, 8, 16, 17, 19, 3, 3, 1),
    (2, 2, 3, 6, 7, 2, 2, 0),
    (2, 16, 64, 12, 12, 3, 1, 1),
    (1, 3, 5, 40, 36, 3, 1, 1),    # long reduction per image: grad_weight in several position slices
    (2, 3, 5, 41, 37, 3, 2, 1),    # the same with element-wise gathers
    (2, 40, 48, 10, 12, 3, 1, 1),  # 64x64 tiles with ragged rows in every product
    # at most four input channels: grad_input on the vector ALU (one channel, 7x7 stem geometry, strides 1, 2 and 3,
    # one to four windows per axis, several workgroups per image); five windows per axis stay on the MFMA kernel
    (2, 1, 8, 28, 28, 3, 1, 0), (1, 3, 16, 31, 29, 7, 2, 3), (2, 2, 4, 10, 9, 3, 3, 1), (3, 4, 6, 9, 9, 4, 2, 0),
    (2, 3, 8, 40, 36, 4, 1, 2), (2, 3, 32, 64, 60, 7, 2, 3), (1, 4, 16, 48, 50, 5, 3, 1), (2, 2, 4, 12, 12, 5, 1, 2),
    # strided grad_input as S*S dense sub-problems (more than four channels, class rows of 2n elements): strides 2 and
    # 3, kernels 1 (most classes empty: zeros), 3, 4, 5 and 7, with and without padding, odd heights, several tiles
    (2, 8, 16, 16, 16, 3, 2, 1), (2, 16, 8, 13, 20, 5, 2, 2), (1, 8, 8, 18, 12, 3, 3, 1), (2, 8, 16, 14, 12, 4, 2, 0),
    (2, 8, 12, 10, 8, 1, 2, 0), (1, 40, 72, 30, 28, 3, 2, 1), (2, 12, 16, 21, 24, 7, 2, 3), (1, 8, 4, 9, 24, 5, 3, 2),
    # ... classes with rows of an odd number of elements (element-wise gathers) and weight rows that are not whole vectors
    (2, 8, 16, 14, 14, 3, 2, 1), (1, 6, 5, 9, 7, 3, 2, 0), (2, 7, 9, 11, 13, 4, 3, 2),
])
def test_forward_backward_random(tt, oracle, dtype, geom):
    Bn, Cc, O, H, W, k, S, P = geom
    rng = np.random.default_rng(sum(geom))
    x = rng.normal(0, 0.5, (Bn, Cc, H, W)).astype(dtype)
    w = rng.normal(0, 0.5, (O, Cc, k, k)).astype(dtype)
    b = rng.normal(0, 0.5, (O,)).astype(dtype)
    tol = tol_of(dtype)
    out = tt.conv2d(dev(tt, x), dev(tt, w), dev(tt, b), S, P).to_numpy()
    want = oracle.conv2d_forward(x, w, b, S, P)
    assert max_rel_error(out, want) <= tol
    g = rng.normal(0, 1, want.shape).astype(dtype)
    gx, gw, gb = tt.conv2d_backward(dev(tt, g), dev(tt, x), dev(tt, w), dev(tt, b), S, P)
    wx, ww, wb = oracle.conv2d_backward(g, x, w, True, S, P)
    assert max_rel_error(gx.to_numpy(), wx) <= tol
    assert max_rel_error(gw.to_numpy(), ww) <= tol
    assert max_rel_error(gb.to_numpy(), wb) <= tol
    # without a bias the third gradient is absent, as in the reference's optional
    gx2, gw2, gb2 = tt.conv2d_backward(dev(tt, g), dev(tt, x), dev(tt, w), None, S, P)
    assert gb2 is None and np.array_equal(gx2.to_numpy(), gx.to_numpy()) and np.array_equal(gw2.to_numpy(), gw.to_numpy())


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_backward_exact_on_integer_data_and_adjoints(tt, oracle, dtype):
    rng = np.random.default_rng(8)
    Bn, Cc, O, H, W, k, S, P = 3, 4, 5, 9, 8, 3, 2, 1
    x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(dtype)
    w = rng.integers(-3, 4, (O, Cc, k, k)).astype(dtype)
    out = tt.conv2d(dev(tt, x), dev(tt, w), None, S, P).to_numpy()
    assert np.array_equal(out, oracle.conv2d_forward(x, w, None, S, P))
    g = rng.integers(-3, 4, out.shape).astype(dtype)
    gx, gw, gb = tt.conv2d_backward(dev(tt, g), dev(tt, x), dev(tt, w), dev(tt, np.zeros(O, dtype)), S, P)
    wx, ww, wb = oracle.conv2d_backward(g, x, w, True, S, P)
    assert np.array_equal(gx.to_numpy(), wx) and np.array_equal(gw.to_numpy(), ww) and np.array_equal(gb.to_numpy(), wb)
    # adjoint identities <g, conv(x,w)> = <gx, x> = <gw, w>
    lhs = np.sum(g.astype(np.float64) * out)
    assert lhs == np.sum(gx.to_numpy().astype(np.float64) * x) == np.sum(gw.to_numpy().astype(np.float64) * w)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("geom", [
    # stride 2 on dense rows with output rows of whole 16-byte vectors: forward gathers two vectors per vector of
    # positions instead of single elements; grad_input's classes store straight into grad_input.  B, C, O, H, W, k, P
    (2, 8, 16, 16, 16, 3, 1),      # the top-left corner under padding (a vector that would start before the image)
    (2, 4, 70, 17, 15, 3, 1),      # odd height and width: the last tap's column lies outside the row (W = 15 -> Wo = 8)
    (1, 12, 8, 20, 24, 5, 2),      # 5 x 5 taps, two columns of padding
    (2, 8, 8, 19, 24, 7, 3),       # 7 x 7 taps (a stem's geometry on more channels)
    (1, 16, 40, 10, 16, 2, 0),     # even kernel, no padding
    (3, 4, 4, 9, 8, 1, 0),         # 1 x 1 taps: every second element of every second row
    (1, 64, 128, 56, 56, 3, 1),    # a layer's real size: several tiles per image, 18 k tiles
    (2, 16, 24, 28, 28, 3, 1),     # output rows of 14: numbered over rows padded to 16 (f32), the padding columns dropped
    (1, 8, 8, 11, 13, 3, 1),       # output rows of 7, padded to 8
])
def test_stride_two_vector_gathers_exact(tt, oracle, dtype, geom):
    Bn, Cc, O, H, W, k, P = geom
    S = 2
    rng = np.random.default_rng(sum(geom))
    x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(dtype)
    w = rng.integers(-3, 4, (O, Cc, k, k)).astype(dtype)
    b = rng.integers(-3, 4, (O,)).astype(dtype)
    out = tt.conv2d(dev(tt, x), dev(tt, w), dev(tt, b), S, P)
    assert _last_kernel(0) == 0x102
    want = oracle.conv2d_forward(x, w, b, S, P)
    assert np.array_equal(out.to_numpy(), want)
    g = rng.integers(-3, 4, want.shape).astype(dtype)
    gx, gw, gb = tt.conv2d_backward(dev(tt, g), dev(tt, x), dev(tt, w), dev(tt, b), S, P)
    wx, ww, wb = oracle.conv2d_backward(g, x, w, True, S, P)
    assert np.array_equal(gw.to_numpy(), ww)
    assert np.array_equal(gx.to_numpy(), wx) and np.array_equal(gb.to_numpy(), wb)
    # the input as a window of a larger tensor whose other elements are NaN: nothing outside the window is summed
    big = np.full((Bn, Cc + 1, H + 3, W + 4), np.nan, dtype)
    big[:, 1:, 2:2 + H, 4:] = x                 # (a unit column stride and rows that end with the storage's rows)
    tb = dev(tt, big)
    es = big.strides
    view = tt.Tensor(tb.storage, tb.dtype, (Bn, Cc, H, W), tuple(st // big.itemsize for st in es),
                     (es[1] + 2 * es[2] + 4 * es[3]) // big.itemsize)
    assert np.array_equal(tt.conv2d(view, dev(tt, w), dev(tt, b), S, P).to_numpy(), want)
    assert _last_kernel(0) == 0x102
    gx2, gw2, _ = tt.conv2d_backward(dev(tt, g), view, dev(tt, w), None, S, P)
    assert np.array_equal(gw2.to_numpy(), ww) and np.array_equal(gx2.to_numpy(), wx)


def _last_kernel(which):
    from tinytensor_amd import _capi
    return _capi.lib.ttamd_conv2d_last_kernel(which)


@pytest.mark.parametrize("geom", [
    # fp32, unit stride: the persistent kernel that keeps the weight block in LDS, forward (input channels 8n, rows
    # of whole 16-byte vectors) and grad_input (output channels 8n, output rows of whole vectors).
    # B, C, O, H, W, k, P, forward on it, grad_input on it
    (3, 32, 64, 28, 28, 3, 1, True, True),     # benchmark geometry: 8 waves forward, one patch buffer for grad_input
    (2, 8, 8, 8, 8, 3, 1, True, True),         # 8 channels per staging item, an image smaller than a tile (idle waves)
    (2, 24, 40, 12, 12, 3, 1, True, False),    # channel counts 8 (2n + 1); result rows beyond the last channel; grad_input's patch
                                                # of 14 rows x 40 channels is more than a lane's 16 loads
    (2, 24, 40, 12, 32, 3, 1, True, True),     # the same with rows of 8 vectors
    (5, 16, 32, 20, 20, 5, 2, True, True),     # 5 x 5 taps, at most 32 result rows
    (2, 16, 16, 9, 16, 1, 0, True, True),      # 1 x 1
    (2, 8, 16, 10, 12, 2, 1, True, False),     # even kernel; Wo = 13: grad_input on the implicit-GEMM kernel
    (2, 32, 96, 14, 36, 3, 0, True, False),    # no padding, a second half-empty row block, 9 vectors per row; Wo = 34
    (70, 32, 64, 6, 4, 3, 1, True, False),     # many small images, one vector per row (grad_input: a tile's rows of 64
                                                # channels are more than a lane's 16 loads)
    (2, 64, 32, 28, 28, 3, 1, True, True),     # 64 channels in: 16 loads per lane and tile, one patch buffer
    (2, 16, 24, 8, 8, 3, 2, True, False),      # padding 2 with k = 3; Wo = 10
    (2, 48, 64, 8, 8, 3, 1, True, False),      # a weight block that passes through LDS in several passes of row-wise loads
    (1, 128, 16, 8, 8, 3, 1, False, True),     # forward: the weight block does not fit; grad_input (16 channels in): it does
    (3, 32, 64, 7, 28, 3, 1, True, True),      # tiles that start and end inside rows, images of 196 positions
])
def test_lds_resident_kernel_exact(tt, oracle, geom):
    Bn, Cc, O, H, W, k, P, fwd_on, dgrad_on = geom
    rng = np.random.default_rng(sum(geom[:7]))
    x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(np.float32)
    w = rng.integers(-3, 4, (O, Cc, k, k)).astype(np.float32)
    b = rng.integers(-3, 4, (O,)).astype(np.float32)
    out = tt.conv2d(dev(tt, x), dev(tt, w), dev(tt, b), 1, P).to_numpy()
    assert (_last_kernel(0) & 0xF00 == 0x200) == fwd_on, hex(_last_kernel(0))
    want = oracle.conv2d_forward(x, w, b, 1, P)
    assert np.array_equal(out, want)
    assert np.array_equal(want - b[None, :, None, None], oracle.conv2d_naive(x, w, 1, P))
    g = rng.integers(-3, 4, want.shape).astype(np.float32)
    gx, gw, gb = tt.conv2d_backward(dev(tt, g), dev(tt, x), dev(tt, w), dev(tt, b), 1, P)
    assert (_last_kernel(1) & 0xF00 == 0x200) == dgrad_on, hex(_last_kernel(1))
    wx, ww, wb = oracle.conv2d_backward(g, x, w, True, 1, P)
    assert np.array_equal(gx.to_numpy(), wx) and np.array_equal(gw.to_numpy(), ww) and np.array_equal(gb.to_numpy(), wb)


@pytest.mark.parametrize("geom", [
    # fp32, unit stride, 32 output channels, input channels 32 n, rows of whole vectors with at least 8 outputs:
    # grad_weight by the kernel that stages grad_out's and the input's rows in LDS.  B, C, H, W, k, P
    (3, 32, 28, 28, 3, 1),     # 9 blocks of 32 x 32: sets of four waves (3, 2, 2, 2 per set)
    (2, 64, 12, 16, 3, 1),     # 18 blocks: the four-wave form (5, 5, 5, 3)
    (5, 32, 9, 12, 1, 0),      # 1 x 1: one block, three idle waves
    (2, 32, 20, 20, 5, 2),     # 5 x 5 taps: 25 blocks is more than a wave's five -> the implicit-GEMM kernel
    (2, 32, 10, 12, 3, 0),     # no padding (Wo = 10: not whole vectors -> the implicit-GEMM kernel)
    (300, 32, 8, 8, 3, 1),     # more units than workgroups: several stages per workgroup, added up in registers
    (7, 32, 11, 16, 3, 1),     # units of unequal height (the last unit of an image is short), a ragged last chunk
    (2, 32, 6, 44, 3, 1),      # wide rows: 11 vectors per row, 5 input rows per load instruction
])
def test_lds_staged_grad_weight_exact(tt, oracle, geom):
    Bn, Cc, H, W, k, P = geom
    O = 32
    rng = np.random.default_rng(sum(geom))
    x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(np.float32)
    w = rng.integers(-3, 4, (O, Cc, k, k)).astype(np.float32)
    Ho, Wo = H + 2 * P - k + 1, W + 2 * P - k + 1
    g = rng.integers(-3, 4, (Bn, O, Ho, Wo)).astype(np.float32)
    gx, gw, gb = tt.conv2d_backward(dev(tt, g), dev(tt, x), dev(tt, w), dev(tt, np.zeros(O, np.float32)), 1, P)
    staged = Wo % 4 == 0 and Wo >= 8 and k * k * (Cc // 32) <= 20
    assert (_last_kernel(2) == 0x200) == staged, hex(_last_kernel(2))
    wx, ww, wb = oracle.conv2d_backward(g, x, w, True, 1, P)
    assert np.array_equal(gw.to_numpy(), ww)
    assert np.array_equal(gx.to_numpy(), wx) and np.array_equal(gb.to_numpy(), wb)


@pytest.mark.parametrize("geom", [
    # The twelve-wave form of the LDS-resident forward kernel: tiles of 192 positions plus a tail of 0, 4 or 8, taken where
    # it shares the tiles out over the chip in fewer rounds than tiles of 128.  B, C, O, H, W, k, P, tail
    (64, 32, 64, 28, 28, 3, 1, 4),     # benchmark configuration 4: four tiles of seven whole rows per image
    (96, 32, 64, 20, 20, 3, 1, 8),     # tail of eight positions (two groups of four)
    (80, 32, 64, 24, 24, 3, 1, 0),     # no tail: the exchange-free path with its extra barrier only
    (96, 32, 64, 33, 12, 3, 1, 8),     # tiles of 200 positions that start and end inside rows of 12
    (256, 32, 64, 7, 28, 3, 1, 4),     # one tile per image
    (256, 32, 64, 12, 16, 3, 1, 0),    # one tile per image, no tail
    (32, 32, 96, 28, 28, 3, 1, 4),     # a second block of output channels that is half empty (rows beyond the last channel)
    (160, 64, 64, 12, 16, 1, 0, 0),    # 1 x 1 taps, 64 channels in, no padding
])
def test_twelve_wave_patch_kernel_exact(tt, oracle, geom):
    Bn, Cc, O, H, W, k, P, tail = geom
    rng = np.random.default_rng(sum(geom))
    x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(np.float32)
    w = rng.integers(-3, 4, (O, Cc, k, k)).astype(np.float32)
    b = rng.integers(-3, 4, (O,)).astype(np.float32)
    out = tt.conv2d(dev(tt, x), dev(tt, w), dev(tt, b), 1, P).to_numpy()
    assert _last_kernel(0) == 0x200 + 12 * 16 + 1, hex(_last_kernel(0))
    assert np.array_equal(out, oracle.conv2d_forward(x, w, b, 1, P))
    no_bias = tt.conv2d(dev(tt, x), dev(tt, w), None, 1, P).to_numpy()
    assert np.array_equal(no_bias, out - b[None, :, None, None])
    # grad_input is the same kernel on grad_out with 32 result channels: twelve waves as two sets of six on the halves of the
    # reduction, where the number of 32-channel groups is even and the tile count favours it
    g = rng.integers(-3, 4, out.shape).astype(np.float32)
    gx, gw, gb = tt.conv2d_backward(dev(tt, g), dev(tt, x), dev(tt, w), dev(tt, b), 1, P)
    if (H, W, O) in ((28, 28, 64), (7, 28, 64), (12, 16, 64)):   # (elsewhere its patch of 64 channels takes too many loads per lane)
        assert _last_kernel(1) == 0x200 + 12 * 16 + 1, hex(_last_kernel(1))
    wx, ww, wb = oracle.conv2d_backward(g, x, w, True, 1, P)
    assert np.array_equal(gx.to_numpy(), wx) and np.array_equal(gw.to_numpy(), ww) and np.array_equal(gb.to_numpy(), wb)


@pytest.mark.parametrize("geom", [
    # grad_weight by the kernel whose sets of waves share out a stage's positions (up to three 32 x 32 blocks per wave:
    # 32 input channels with 3 x 3 taps, 64 with 1 x 1 or 2 x 2).  B, C, O, H, W, k, P
    (64, 32, 64, 28, 28, 3, 1),     # benchmark configuration 4: stages of 14 rows, two load instructions per row and channel
    (3, 32, 64, 28, 28, 3, 1),      # fewer units than workgroups
    (5, 32, 96, 12, 16, 3, 1),      # three blocks of output channels
    (300, 32, 64, 8, 8, 3, 1),      # several stages per workgroup, added up in registers
    (7, 32, 64, 11, 16, 3, 1),      # units of unequal height, a ragged last chunk
    (4, 64, 64, 16, 16, 1, 0),      # 1 x 1 taps, 64 input channels: two blocks (1, 1, 0, 0 per set)
    (4, 64, 32, 12, 12, 2, 1),      # 2 x 2 taps (Wo = 13: not whole vectors -> another kernel)
    (2, 32, 64, 6, 44, 3, 1),       # wide rows
    (2, 32, 160, 9, 12, 3, 0),      # five blocks of output channels, no padding (Wo = 10 -> another kernel)
])
def test_grad_weight_with_sets_of_waves_exact(tt, oracle, geom):
    Bn, Cc, O, H, W, k, P = geom
    rng = np.random.default_rng(sum(geom))
    x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(np.float32)
    w = rng.integers(-3, 4, (O, Cc, k, k)).astype(np.float32)
    Ho, Wo = H + 2 * P - k + 1, W + 2 * P - k + 1
    g = rng.integers(-3, 4, (Bn, O, Ho, Wo)).astype(np.float32)
    gx, gw, gb = tt.conv2d_backward(dev(tt, g), dev(tt, x), dev(tt, w), dev(tt, np.zeros(O, np.float32)), 1, P)
    staged = Wo % 4 == 0 and Wo >= 8
    assert (_last_kernel(2) == 0x200) == staged, hex(_last_kernel(2))
    wx, ww, wb = oracle.conv2d_backward(g, x, w, True, 1, P)
    assert np.array_equal(gw.to_numpy(), ww)
    assert np.array_equal(gx.to_numpy(), wx) and np.array_equal(gb.to_numpy(), wb)


def test_twelve_wave_and_sets_kernels_on_an_input_window(tt, oracle):
    """Benchmark configuration 4 with the input as a window of a larger, NaN-filled tensor (row stride 32, a channel more,
    two rows more, 16-byte aligned start): the twelve-wave forward and grad_input kernels and grad_weight's sets of waves
    read it through its strides."""
    rng = np.random.default_rng(404)
    Bn, Cc, O, H, W = 64, 32, 64, 28, 28
    big = np.full((Bn, Cc + 1, H + 2, W + 4), np.nan, np.float32)
    x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(np.float32)
    big[:, 1:, 1:1 + H, 4:] = x
    w = rng.integers(-3, 4, (O, Cc, 3, 3)).astype(np.float32)
    b = rng.integers(-3, 4, (O,)).astype(np.float32)
    tb = dev(tt, big)
    es = [v // 4 for v in big.strides]
    tx = tt.Tensor(tb.storage, tb.dtype, (Bn, Cc, H, W), tuple(es), es[1] + es[2] + 4)
    assert not tx.is_contiguous()
    out = tt.conv2d(tx, dev(tt, w), dev(tt, b), 1, 1).to_numpy()
    assert _last_kernel(0) == 0x200 + 12 * 16 + 1, hex(_last_kernel(0))
    want = oracle.conv2d_forward(x, w, b, 1, 1)
    assert np.array_equal(out, want)
    g = rng.integers(-3, 4, want.shape).astype(np.float32)
    gx, gw, gb = tt.conv2d_backward(dev(tt, g), tx, dev(tt, w), dev(tt, b), 1, 1)
    assert _last_kernel(1) == 0x200 + 12 * 16 + 1 and _last_kernel(2) == 0x200, (hex(_last_kernel(1)), hex(_last_kernel(2)))
    wx, ww, wb = oracle.conv2d_backward(g, x, w, True, 1, 1)
    assert np.array_equal(gx.to_numpy(), wx) and np.array_equal(gw.to_numpy(), ww) and np.array_equal(gb.to_numpy(), wb)


@pytest.mark.parametrize("shape", [(8, 32, 28, 28, 64), (3, 32, 12, 16, 32), (300, 32, 8, 8, 32), (2, 64, 12, 16, 32), (1, 32, 8, 8, 32)],
                         ids=lambda s: "x".join(map(str, s)))
def test_grad_weight_parts_added_in_grad_inputs_launch_exact(tt, oracle, shape):
    """The LDS-staged grad_weight leaves one partial tile per workgroup.  Where grad_input takes the LDS-resident kernel
    too, workgroups appended to that launch add the tiles up (ttamd_conv2d_last_kernel(3) == 2), otherwise a launch of
    its own does (1); a single workgroup writes grad_weight itself (0).  Integer data: every route is exact, and a
    second call, into the same workspace, gives the same bits."""
    Bn, Cc, H, W, O = shape
    rng = np.random.default_rng(sum(shape))
    x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(np.float32)
    w = rng.integers(-3, 4, (O, Cc, 3, 3)).astype(np.float32)
    g = rng.integers(-3, 4, (Bn, O, H, W)).astype(np.float32)
    wx, ww, _ = oracle.conv2d_backward(g, x, w, False, 1, 1)
    tg, tx, tw = dev(tt, g), dev(tt, x), dev(tt, w)
    gx, gw, _ = tt.conv2d_backward(tg, tx, tw, None, 1, 1)
    staged, resident, route = _last_kernel(2) == 0x200, _last_kernel(1) & 0xF00 == 0x200, _last_kernel(3)
    assert staged, hex(_last_kernel(2))
    assert route in ((0, 2) if resident else (0, 1)), (route, hex(_last_kernel(1)))
    if shape == (8, 32, 28, 28, 64):
        assert route == 2
    print(shape, "route", route, flush=True)
    assert np.array_equal(gx.to_numpy(), wx) and np.array_equal(gw.to_numpy(), ww)
    gx2, gw2, _ = tt.conv2d_backward(tg, tx, tw, None, 1, 1)
    assert np.array_equal(gx2.to_numpy(), wx) and np.array_equal(gw2.to_numpy(), ww)
    # real data: the sum over the parts runs in one fixed order, so two calls agree to the bit
    xr = rng.standard_normal(x.shape).astype(np.float32)
    gr = rng.standard_normal(g.shape).astype(np.float32)
    a = tt.conv2d_backward(dev(tt, gr), dev(tt, xr), tw, None, 1, 1)[1].to_numpy()
    b = tt.conv2d_backward(dev(tt, gr), dev(tt, xr), tw, None, 1, 1)[1].to_numpy()
    assert np.array_equal(a, b)
    want = oracle.conv2d_backward(gr, xr, w, False, 1, 1)[1]
    assert np.allclose(a, want, rtol=2e-4, atol=2e-3 * np.sqrt(Bn * H * W))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("geom", [
    # B, C, H, W, O, k, S, P: layers on the implicit-GEMM kernels (weight blocks beyond LDS, odd widths, 5 x 5 taps, strides)
    (4, 64, 28, 28, 128, 3, 1, 1), (3, 128, 14, 14, 128, 3, 1, 1), (6, 48, 9, 13, 40, 3, 1, 1), (2, 32, 20, 20, 32, 5, 1, 2),
    (5, 64, 7, 7, 64, 3, 1, 1), (4, 64, 16, 16, 64, 1, 1, 0), (4, 64, 28, 28, 128, 3, 2, 1), (3, 8, 12, 12, 16, 3, 1, 0),
], ids=lambda g: "x".join(map(str, g)))
def test_backward_small_jobs_ride_in_the_big_launches_exact(tt, oracle, geom, dtype):
    """conv2d_backward launches grad_weight first; the transposed weight that the implicit-GEMM grad_input reads is written
    by workgroups appended to grad_weight's grid, and the sums over grad_weight's partial tiles and over grad_bias's parts
    by workgroups appended to grad_input's.  Integer data: grad_input, grad_weight and grad_bias exact for both dtypes,
    with and without a bias, and the same bits on a second call into the same workspace."""
    Bn, Cc, H, W, O, k, S, P = geom
    rng = np.random.default_rng(sum(geom))
    x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(dtype)
    w = rng.integers(-3, 4, (O, Cc, k, k)).astype(dtype)
    b = rng.integers(-3, 4, (O,)).astype(dtype)
    Ho, Wo = (H + 2 * P - k) // S + 1, (W + 2 * P - k) // S + 1
    g = rng.integers(-3, 4, (Bn, O, Ho, Wo)).astype(dtype)
    wx, ww, wb = oracle.conv2d_backward(g, x, w, True, S, P)
    tg, tx, tw, tb = dev(tt, g), dev(tt, x), dev(tt, w), dev(tt, b)
    be = tt.get_backend(tt.kAMD)
    bufs = be.conv2d_backward(tg, tx, tw, tb, S, P, return_buffers=True)
    route = _last_kernel(3)
    for _ in range(2):
        gx, gw, gb, _ws = bufs
        assert np.array_equal(gx.to_numpy(), wx) and np.array_equal(gw.to_numpy(), ww) and np.array_equal(gb.to_numpy(), wb)
        bufs = be.conv2d_backward(tg, tx, tw, tb, S, P, buffers=bufs, return_buffers=True)
        assert _last_kernel(3) == route
    if S == 1 and (O * Cc * k * k) % 4 == 0:
        assert route in (0, 2), route              # unit stride: no launch of its own for the sum
    gx, gw, none = tt.conv2d_backward(tg, tx, tw, None, S, P)
    assert none is None and np.array_equal(gx.to_numpy(), wx) and np.array_equal(gw.to_numpy(), ww)


def test_lds_resident_kernel_on_views(tt, oracle):
    # an input window of a larger tensor (row stride 16, 16-byte aligned start) and, through the C ABI, a weight whose
    # output-channel stride is larger than C k k (the row-wise weight loads)
    from tinytensor_amd import _capi
    import ctypes as C
    rng = np.random.default_rng(77)
    big = rng.integers(-3, 4, (2, 16, 12, 16)).astype(np.float32)
    wbig = rng.integers(-3, 4, (24, 20, 3, 3)).astype(np.float32)
    x, w = np.ascontiguousarray(big[:, :, 2:10, 4:12]), np.ascontiguousarray(wbig[:, :16])
    tb = dev(tt, big)
    tx = tt.Tensor(tb.storage, tb.dtype, (2, 16, 8, 8), (16 * 12 * 16, 12 * 16, 16, 1), 2 * 16 + 4)
    assert not tx.is_contiguous()
    got = tt.conv2d(tx, dev(tt, w), None, 1, 1).to_numpy()
    assert _last_kernel(0) & 0xF00 == 0x200
    want = oracle.conv2d_forward(x, w, None, 1, 1)
    assert np.array_equal(got, want)
    twb = dev(tt, wbig)
    tw = tt.Tensor(twb.storage, twb.dtype, (24, 16, 3, 3), (20 * 9, 9, 3, 1), 0)
    out = tt.Tensor.empty(want.shape, _capi.F32, tx.device)
    iv, wv = tx.view4(), tw.view4()
    rc = _capi.lib.ttamd_conv2d_forward(0, _capi.F32, C.byref(iv), C.byref(wv), None, C.c_void_p(out.storage.ptr),
                                        2, 16, 8, 8, 24, 3, 1, 1, None)
    assert rc == 0, _capi.last_error()
    assert _last_kernel(0) & 0xF00 == 0x200
    assert np.array_equal(out.to_numpy(), want)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("geom", [
    # unit stride with rows that are a whole number of 16-byte vectors: the vector-gather kernels.
    # B, C, O, H, W, k, P
    (2, 3, 5, 8, 8, 3, 1),
    (2, 4, 6, 12, 16, 5, 2),
    (1, 2, 3, 10, 12, 7, 3),
    (2, 3, 4, 9, 11, 4, 0),    # Wo = 8 but W = 11: grad_input takes the element-wise gather
    (1, 2, 3, 8, 8, 9, 4),     # a whole vector left of the row
    (1, 2, 3, 6, 8, 1, 2),     # padding wider than the kernel
    (3, 70, 66, 6, 4, 3, 1),   # several channel tiles, one vector per row
    # rows of 2n but not 4n elements: 8-byte gathers (fp32; fp64's 16-byte vector is the pair already)
    (2, 8, 16, 14, 14, 3, 1), (2, 8, 12, 13, 26, 3, 0), (1, 8, 8, 9, 10, 5, 2), (2, 72, 68, 6, 6, 3, 1), (1, 4, 4, 8, 6, 9, 4),
    # rows that are no whole number of 16-byte vectors, numbered over padded rows (the padding columns are dropped on
    # the way out): odd widths, widths of 4n + 2, several position tiles per image, a tile that ends inside a row
    (2, 8, 8, 7, 7, 3, 1), (1, 8, 8, 5, 5, 3, 1), (2, 8, 8, 3, 3, 3, 1), (1, 8, 8, 26, 26, 3, 0), (2, 4, 8, 9, 7, 5, 2),
    (1, 8, 8, 41, 37, 3, 1), (2, 40, 70, 15, 14, 3, 1), (1, 8, 40, 23, 30, 3, 1),
    # small images: grad_weight runs several of them through one reduction (groups of images, a ragged last group)
    (40, 70, 66, 6, 4, 3, 1), (13, 70, 66, 7, 7, 3, 1), (9, 8, 8, 10, 10, 3, 1), (5, 72, 8, 8, 8, 3, 1), (21, 66, 70, 5, 5, 3, 1),
])
def test_unit_stride_vector_gathers_exact(tt, oracle, dtype, geom):
    Bn, Cc, O, H, W, k, P = geom
    rng = np.random.default_rng(sum(geom))
    x = rng.integers(-3, 4, (Bn, Cc, H, W)).astype(dtype)
    w = rng.integers(-3, 4, (O, Cc, k, k)).astype(dtype)
    b = rng.integers(-3, 4, (O,)).astype(dtype)
    out = tt.conv2d(dev(tt, x), dev(tt, w), dev(tt, b), 1, P).to_numpy()
    want = oracle.conv2d_forward(x, w, b, 1, P)
    assert np.array_equal(out, want)
    assert np.array_equal(want - b[None, :, None, None], oracle.conv2d_naive(x, w, 1, P))
    g = rng.integers(-3, 4, want.shape).astype(dtype)
    gx, gw, gb = tt.conv2d_backward(dev(tt, g), dev(tt, x), dev(tt, w), dev(tt, b), 1, P)
    wx, ww, wb = oracle.conv2d_backward(g, x, w, True, 1, P)
    assert np.array_equal(gx.to_numpy(), wx) and np.array_equal(gw.to_numpy(), ww) and np.array_equal(gb.to_numpy(), wb)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("geom", [
    # grad_bias is summed in parts of a channel's B * Ho * Wo elements once there are enough of them.
    # B, C, O, H, W
    (64, 2, 3, 24, 24),   # 16-byte loads, 18 whole parts (fp32)
    (33, 2, 5, 23, 21),   # odd rows: element loads, ragged last part
    (7, 1, 70, 50, 50),   # parts that start and end inside an image
    (300, 1, 2, 16, 12),  # more images than parts
    (1, 1, 1, 96, 96),    # one image, one channel
])
def test_grad_bias_in_parts_exact(tt, dtype, geom):
    Bn, Cc, O, H, W = geom
    rng = np.random.default_rng(sum(geom))
    x = rng.integers(-2, 3, (Bn, Cc, H, W)).astype(dtype)
    w = rng.integers(-2, 3, (O, Cc, 1, 1)).astype(dtype)
    g = rng.integers(-3, 4, (Bn, O, H, W)).astype(dtype)
    g[:, :, 0, 0] += 5  # a non-zero mean, so that a dropped or doubled part shows
    gx, gw, gb = tt.conv2d_backward(dev(tt, g), dev(tt, x), dev(tt, w), dev(tt, np.zeros(O, dtype)), 1, 0)
    assert np.array_equal(gb.to_numpy(), g.astype(np.int64).sum((0, 2, 3)).astype(dtype))  # closed form, exact in both dtypes
    assert np.array_equal(gw.to_numpy()[:, :, 0, 0], np.einsum("bohw,bchw->oc", g.astype(np.int64), x.astype(np.int64)).astype(dtype))
    assert np.array_equal(gx.to_numpy(), np.einsum("bohw,oc->bchw", g.astype(np.int64), w[:, :, 0, 0].astype(np.int64)).astype(dtype))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("W", [7, 14])
def test_padding_columns_of_padded_rows_carry_nothing(tt, oracle, dtype, W):
    """Rows of 7 or 14 positions are numbered over 8 or 16 columns.  An infinite input value in the last column must
    reach exactly the sums that the reference's windows give it: a padding column that multiplied it by zero would
    leave a NaN in a tap whose real windows never touch that pixel."""
    rng = np.random.default_rng(W)
    Bn, Cc, O, k = 2, 8, 8, 3
    x = rng.integers(-2, 3, (Bn, Cc, W + 2, W + 2)).astype(dtype)  # no padding: the output rows have W positions
    x[0, 1, 3, W + 1] = np.inf
    w = rng.integers(1, 4, (O, Cc, k, k)).astype(dtype)
    out = tt.conv2d(dev(tt, x), dev(tt, w), None, 1, 0).to_numpy()
    want = oracle.conv2d_forward(x, w, None, 1, 0)
    assert out.shape[3] == W and np.isinf(want).any() and not np.isnan(want).any()
    assert np.array_equal(out, want)
    g = rng.integers(1, 4, want.shape).astype(dtype)  # positive: every sum that meets the infinity is +inf, none NaN
    gx, gw, _ = tt.conv2d_backward(dev(tt, g), dev(tt, x), dev(tt, w), None, 1, 0)
    wx, ww, _ = oracle.conv2d_backward(g, x, w, False, 1, 0)
    assert np.isinf(ww).any() and not np.isnan(ww).any() and np.isfinite(ww[:, :, :, :2]).all()
    assert np.array_equal(gw.to_numpy(), ww) and np.array_equal(gx.to_numpy(), wx)


def test_infinite_values_reach_exactly_their_windows_in_the_lds_staged_kernels(tt, oracle):
    """Benchmark configuration 4's geometry, whose forward and grad_input tiles end in a tail of four positions computed
    apart and whose grad_weight stages end in a chunk that is half empty: positions beyond a tile, a tail or a stage are
    read at stand-in cells.  Infinite input / gradient values at the last positions of tiles, stages and images must
    come out as the reference's infinities (and its NaNs, where it has them) and nowhere else."""
    rng = np.random.default_rng(11)
    Bn, Cc, O, H, W = 64, 32, 64, 28, 28
    x = rng.integers(0, 3, (Bn, Cc, H, W)).astype(np.float32)
    w = rng.integers(1, 3, (O, Cc, 3, 3)).astype(np.float32)
    for (b, c, y, xx) in ((0, 0, 6, 27), (1, 5, 7, 0), (2, 31, 27, 27), (3, 7, 13, 27), (63, 16, 27, 24)):
        x[b, c, y, xx] = np.inf
    out = tt.conv2d(dev(tt, x), dev(tt, w), None, 1, 1).to_numpy()
    assert _last_kernel(0) == 0x200 + 12 * 16 + 1
    want = oracle.conv2d_forward(x, w, None, 1, 1)
    assert np.isinf(want).any() and not np.isnan(want).any()
    assert np.array_equal(out, want)
    g = rng.integers(1, 3, want.shape).astype(np.float32)
    for (b, o, y, xx) in ((0, 0, 6, 27), (5, 63, 27, 27), (9, 31, 13, 24), (63, 32, 14, 0)):
        g[b, o, y, xx] = np.inf
    x2 = rng.integers(1, 3, x.shape).astype(np.float32)   # (finite and positive: no inf - inf)
    gx, gw, _ = tt.conv2d_backward(dev(tt, g), dev(tt, x2), dev(tt, w), None, 1, 1)
    assert _last_kernel(1) == 0x200 + 12 * 16 + 1 and _last_kernel(2) == 0x200
    wx, ww, _ = oracle.conv2d_backward(g, x2, w, False, 1, 1)
    # (the reference's im2col holds real zeros where a window reaches into the padding: an infinite gradient at the image's
    # edge times such a zero is a NaN in its grad_weight -- in those taps and no others)
    assert np.isinf(wx).any() and not np.isnan(wx).any() and np.isnan(ww).any() and np.isinf(ww).any()
    assert np.array_equal(gx.to_numpy(), wx) and np.array_equal(gw.to_numpy(), ww, equal_nan=True)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_unaligned_window_of_a_larger_image(tt, oracle, dtype):
    # the input is a window [1:9, 3:15] of a stored [2,3,10,20] tensor: rows start at odd element offsets,
    # so every 16-byte gather is unaligned, and the elements around the window are non-zero
    rng = np.random.default_rng(12)
    store = rng.integers(1, 5, (2, 3, 10, 20)).astype(dtype)
    x = np.ascontiguousarray(store[:, :, 1:9, 3:15])
    w = rng.integers(-3, 4, (5, 3, 3, 3)).astype(dtype)
    ts = dev(tt, store)
    tx = tt.Tensor(ts.storage, ts.dtype, (2, 3, 8, 12), (600, 200, 20, 1), 23)
    out = tt.conv2d(tx, dev(tt, w), None, 1, 1).to_numpy()
    want = oracle.conv2d_forward(x, w, None, 1, 1)
    assert np.array_equal(out, want)
    g = rng.integers(-3, 4, want.shape).astype(dtype)
    gx, gw, _ = tt.conv2d_backward(dev(tt, g), tx, dev(tt, w), None, 1, 1)
    wx, ww, _ = oracle.conv2d_backward(g, x, w, False, 1, 1)
    assert np.array_equal(gx.to_numpy(), wx) and np.array_equal(gw.to_numpy(), ww)


def test_config4_conv_forward_backward(tt, oracle):
    # benchmark configuration 4: input [64,32,28,28], weight [64,32,3,3], stride 1, padding 1, normal(0, 0.1) from a seed.
    x = oracle.Generator(0).normal(0.0, 0.1, (64, 32, 28, 28))
    w = oracle.Generator(1).normal(0.0, 0.1, (64, 32, 3, 3))
    tx, tw = dev(tt, x), dev(tt, w)
    out = tt.conv2d(tx, tw, None, 1, 1).to_numpy()
    want = oracle.conv2d_forward(x, w, None, 1, 1)
    assert out.shape == (64, 64, 28, 28)
    assert max_rel_error(out, want) <= 1e-4
    # backward with g = ones (what backward() seeds) and with a random g
    for g in (np.ones_like(want), oracle.Generator(2).uniform_real(-1, 1, want.shape)):
        gx, gw, _ = tt.conv2d_backward(dev(tt, g), tx, tw, None, 1, 1)
        wx, ww, _ = oracle.conv2d_backward(g, x, w, False, 1, 1)
        assert max_rel_error(gx.to_numpy(), wx) <= 1e-4
        assert max_rel_error(gw.to_numpy(), ww) <= 1e-4
        # adjoint identity at full size, in f64
        lhs = np.sum(g.astype(np.float64) * out)
        assert abs(lhs - np.sum(gx.to_numpy().astype(np.float64) * x)) <= 1e-4 * abs(lhs)
        assert abs(lhs - np.sum(gw.to_numpy().astype(np.float64) * w)) <= 1e-4 * abs(lhs)


def test_strided_input_view_and_errors(tt, oracle):
    rng = np.random.default_rng(3)
    xs = rng.integers(-3, 4, (2, 9, 8, 4)).astype(np.float32)  # stored NHWC
    x = np.ascontiguousarray(xs.transpose(0, 3, 1, 2))         # logical NCHW
    w = rng.integers(-3, 4, (6, 4, 3, 3)).astype(np.float32)
    tx = dev(tt, xs).permute(0, 3, 1, 2)
    assert not tx.is_contiguous()
    got = tt.conv2d(tx, dev(tt, w), None, 1, 1).to_numpy()
    assert np.array_equal(got, oracle.conv2d_forward(x, w, None, 1, 1))
    # a permuted weight is made dense by the adapter, as the reference's reshape does
    wt = dev(tt, np.ascontiguousarray(w.transpose(1, 0, 2, 3))).permute(1, 0, 2, 3)
    assert np.array_equal(tt.conv2d(tx, wt, None, 1, 1).to_numpy(), got)
    with pytest.raises(tt.TTException):
        tt.conv2d(dev(tt, x), dev(tt, rng.random((6, 5, 3, 3)).astype(np.float32)))  # channel mismatch
    with pytest.raises(tt.TTException):
        tt.conv2d(dev(tt, x), dev(tt, rng.random((6, 4, 3, 2)).astype(np.float32)))  # non-square kernel
    with pytest.raises(tt.TTException):
        tt.conv2d(dev(tt, x), dev(tt, w), None, 0, 0)                                  # stride 0
    with pytest.raises(tt.TTException):
        tt.conv2d(dev(tt, x[:, :, :2, :2]), dev(tt, w), None, 1, 0)                    # kernel larger than input
