"""Randomised parity check of ttamd_batched_matmul on views: operands stored with padded rows (NaN in the padding, so an
element read from beyond the view shows in every sum it reaches), plain or as transposed views, sizes around the tile
and vector boundaries (k tails, ragged rows and columns, reductions of at most 16, at most 16 columns), with the store's
options drawn at random.  Integer-valued data: exact in any summation order."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROWS = [1, 7, 16, 63, 64, 65, 130, 200, 512, 784, 1000, 1024, 1100]
REDS = [1, 3, 10, 16, 17, 31, 32, 33, 63, 100, 255, 392, 516, 784, 1000, 1024, 1030]
COLS = [1, 5, 10, 16, 17, 64, 66, 130, 300, 784, 1000, 1024]


def _view(tt, x, transposed, pad, dtype):
    """x [B, R, C] as a view of a storage whose rows carry `pad` extra NaN elements; transposed: the storage holds x^T."""
    src = np.ascontiguousarray(x.transpose(0, 2, 1)) if transposed else x
    Bn, R, Cn = src.shape
    st = np.full((Bn, R, Cn + pad), np.nan, dtype)
    st[:, :, :Cn] = src
    t = tt.Tensor.from_numpy(st)
    v = tt.Tensor(t.storage, t.dtype, (Bn, R, Cn), (R * (Cn + pad), Cn + pad, 1), 0)
    return v.permute(0, 2, 1) if transposed else v


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_views_and_store_options(tt, seed):
    be = tt.get_backend(tt.kAMD)
    rng = np.random.default_rng(seed)
    for case in range(60):
        dtype = rng.choice([np.float32, np.float64])
        B = int(rng.choice([1, 1, 1, 2, 3]))
        N, K, M = int(rng.choice(ROWS)), int(rng.choice(REDS)), int(rng.choice(COLS))
        pad_a, pad_b = int(rng.choice([0, 0, 1, 3, 4, 8])), int(rng.choice([0, 0, 1, 4, 8]))
        ta_t, tb_t = bool(rng.integers(2)), bool(rng.integers(2))
        a = rng.integers(-3, 4, (B, N, K)).astype(dtype)
        b = rng.integers(-3, 4, (B, K, M)).astype(dtype)
        tA, tB = _view(tt, a, ta_t, pad_a, dtype), _view(tt, b, tb_t, pad_b, dtype)
        want = np.matmul(a.astype(np.float64), b.astype(np.float64)).astype(dtype)
        options, sums = {}, None
        mode = int(rng.integers(4))
        if mode == 1:
            bias = rng.integers(-5, 6, (M,)).astype(dtype)
            options = dict(bias=tt.Tensor.from_numpy(bias), bias_mode=1, relu=True)
            want = np.maximum(want + bias, 0).astype(dtype)
        elif mode == 2:
            z = rng.integers(-2, 3, (B, N, M)).astype(dtype)
            options = dict(relu_grad_input=tt.Tensor.from_numpy(z))
            want = (want * np.where(z < 0, 0, 1)).astype(dtype)
        elif mode == 3 and not tb_t and pad_b == 0:   # (the right operand's sums need a dense right operand)
            sums = tt.Tensor.from_numpy(np.zeros((B, M), dtype))
            options = dict(rhs_colsum_out=sums)
        what = (seed, case, dtype.__name__, (B, N, K, M), pad_a, pad_b, ta_t, tb_t, mode, be.batched_matmul_variant(tA, tB))
        assert np.array_equal(be.batched_matmul(tA, tB, **options).to_numpy(), want), what
        if sums is not None:
            assert np.array_equal(sums.to_numpy(), b.sum(axis=1)), what
