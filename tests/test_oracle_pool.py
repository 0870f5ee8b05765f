"""Pins the pooling oracle (oracle/tt_oracle_pool.c) on the CPU.

The reference's own pooling tests compare with libtorch on B4 C128 68x28 k3 s2 p1 random data
(tests/test_conv.cpp:186-278, tests/test_conv_autograd.cpp:109-230); the same comparison is made here with
torch's CPU operators, and an independent numpy statement of the window arithmetic covers what torch defines
differently (ties in max/min backward, which the reference splits evenly) and the integer dtypes.
"""
import numpy as np
import pytest

from helpers import ALL_NON_BOOL

torch = pytest.importorskip("torch")
F = torch.nn.functional

TORCH_FWD = {
    "max": lambda t, k, s, p: F.max_pool2d(t, k, s, p),
    "min": lambda t, k, s, p: -F.max_pool2d(-t, k, s, p),
    "avg": lambda t, k, s, p: F.avg_pool2d(t, k, s, p),
}


def windows(x, k, S, P, pad_value):
    """[B,C,Ho,Wo,k*k] array of window elements in (p, q) order, padding filled with pad_value."""
    Bn, Cc, H, W = x.shape
    Ho, Wo = (H + 2 * P - k) // S + 1, (W + 2 * P - k) // S + 1
    xp = np.full((Bn, Cc, H + 2 * P, W + 2 * P), pad_value, dtype=x.dtype)
    xp[:, :, P:P + H, P:P + W] = x
    out = np.empty((Bn, Cc, Ho, Wo, k * k), dtype=x.dtype)
    for p in range(k):
        for q in range(k):
            out[..., p * k + q] = xp[:, :, p:p + S * Ho:S, q:q + S * Wo:S]
    return out


@pytest.mark.parametrize("op", ["max", "min", "avg"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_forward_and_backward_match_torch_on_the_reference_shape(oracle, op, dtype):
    rng = np.random.default_rng(0)
    x = rng.normal(size=(4, 128, 68, 28)).astype(dtype)
    k, S, P = 3, 2, 1
    got = oracle.pool2d_forward(x, op, k, S, P)
    t = torch.from_numpy(x).requires_grad_(True)
    y = TORCH_FWD[op](t, k, S, P)
    assert got.shape == tuple(y.shape) == (4, 128, 34, 14)
    if op == "avg":
        assert np.allclose(got, y.detach().numpy(), rtol=0, atol=1e-6)  # the reference test's tolerance
    else:
        assert np.array_equal(got, y.detach().numpy())
    g = rng.normal(size=got.shape).astype(dtype)
    y.backward(torch.from_numpy(g))
    gx = oracle.pool2d_backward(g, x, got, op, k, S, P)
    assert np.allclose(gx, t.grad.numpy(), rtol=1e-6, atol=1e-6)  # random data: no ties


@pytest.mark.parametrize("geom", [(2, 3, 9, 8, 2, 2, 0), (1, 2, 7, 7, 3, 1, 1), (2, 2, 6, 9, 3, 3, 2), (1, 1, 5, 5, 5, 1, 2)])
@pytest.mark.parametrize("dtype", ALL_NON_BOOL)
def test_forward_matches_window_statement(oracle, geom, dtype):
    Bn, Cc, H, W, k, S, P = geom
    rng = np.random.default_rng(sum(geom))
    x = rng.integers(0, 50, (Bn, Cc, H, W)).astype(dtype) if np.dtype(dtype).kind == "u" else \
        rng.integers(-50, 50, (Bn, Cc, H, W)).astype(dtype)
    info = np.finfo(dtype) if np.dtype(dtype).kind == "f" else np.iinfo(dtype)
    assert np.array_equal(oracle.pool2d_forward(x, "max", k, S, P), windows(x, k, S, P, info.min).max(-1))
    assert np.array_equal(oracle.pool2d_forward(x, "min", k, S, P), windows(x, k, S, P, info.max).min(-1))
    # avg: ((x0/n + 0) ... ) folded left to right in the result type, padding contributes 0/n
    rdtype = dtype if np.dtype(dtype).kind == "f" else np.float32
    win = windows(x, k, S, P, 0).astype(rdtype)
    acc = np.zeros(win.shape[:-1], dtype=rdtype)
    n = rdtype(k * k)
    for i in range(k * k):
        acc = (win[..., i] / n + acc).astype(rdtype)
    got = oracle.pool2d_forward(x, "avg", k, S, P)
    assert got.dtype == rdtype and np.array_equal(got, acc)


@pytest.mark.parametrize("op", ["max", "min", "avg"])
def test_backward_scatter_statement_with_ties(oracle, op):
    # small integer-valued data: many ties, overlapping windows (S < k) and padding
    rng = np.random.default_rng(5)
    Bn, Cc, H, W, k, S, P = 2, 2, 7, 6, 3, 2, 1
    x = rng.integers(0, 3, (Bn, Cc, H, W)).astype(np.float64)
    res = oracle.pool2d_forward(x, op, k, S, P)
    g = rng.integers(-4, 5, res.shape).astype(np.float64)
    want = np.zeros_like(x)
    Ho, Wo = res.shape[2:]
    for b in range(Bn):
        for c in range(Cc):
            for h in range(Ho):
                for w in range(Wo):
                    cells = [(S * h + p - P, S * w + q - P) for p in range(k) for q in range(k)]
                    cells = [(i, j) for i, j in cells if 0 <= i < H and 0 <= j < W]
                    if op != "avg":
                        cells = [(i, j) for i, j in cells if x[b, c, i, j] == res[b, c, h, w]]
                        share = g[b, c, h, w] / len(cells)
                    else:
                        share = g[b, c, h, w] / (k * k)
                    for i, j in cells:
                        want[b, c, i, j] += share
    got = oracle.pool2d_backward(g, x, res, op, k, S, P)
    assert np.array_equal(got, want)
    # the gradient of sum(pool(x)) distributes exactly one unit per output window (max/min)
    if op != "avg":
        ones = oracle.pool2d_backward(np.ones_like(res), x, res, op, k, S, P)
        assert abs(ones.sum() - res.size) < 1e-9
