"""Pins the conv2d and matmul-backward oracle against torch's CPU operators, the golden source of the
reference's own TT_TORCH tests: tests/test_conv.cpp:147-184 (forward, f32, atol 1e-6),
tests/test_conv_autograd.cpp:43-107 (backward, f64, atol 1e-4) and tests/test_matmul_autograd.cpp:218-262
(batched matmul backward, f64, B4 379x1147x635, atol 1e-6), on the same shapes with seeded random data."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")


def allclose(a, b, atol, rtol=1e-5):
    # include/tt/tensor.h:3396-3398: |a - b| <= atol + rtol * |b|
    return bool(np.all(np.abs(a - b) <= atol + rtol * np.abs(b)))


def test_conv2d_forward_matches_torch(oracle):
    rng = np.random.default_rng(0)
    x = rng.random((4, 3, 68, 28), dtype=np.float32)
    w = rng.random((128, 3, 3, 3), dtype=np.float32)
    b = rng.random(128, dtype=np.float32)
    want = torch.conv2d(torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(b), 2, 1).numpy()
    got = oracle.conv2d_forward(x, w, b, 2, 1)
    assert got.shape == want.shape == (4, 128, 34, 14)
    assert allclose(got, want, 1e-6)


@pytest.mark.parametrize("S,P", [(2, 1), (1, 1), (3, 0)])
def test_conv2d_backward_matches_torch_autograd(oracle, S, P):
    rng = np.random.default_rng(1)
    x = rng.random((4, 3, 38, 28))
    w = rng.random((64, 3, 3, 3))
    b = rng.random(64)
    tx, tw, tb = (torch.from_numpy(a).requires_grad_(True) for a in (x, w, b))
    out = torch.conv2d(tx, tw, tb, S, P)
    g = rng.random(tuple(out.shape))
    out.backward(torch.from_numpy(g))
    gx, gw, gb = oracle.conv2d_backward(g, x, w, True, S, P)
    assert float(np.abs(gx - tx.grad.numpy()).mean()) < 0.001 and allclose(gx, tx.grad.numpy(), 1e-4)
    assert allclose(gw, tw.grad.numpy(), 1e-4)
    assert allclose(gb, tb.grad.numpy(), 1e-4)


def test_batched_matmul_backward_matches_torch_autograd(oracle):
    rng = np.random.default_rng(2)
    Bn, N, M, K = 4, 256 + 123, 1024 + 123, 512 + 123
    lhs, rhs, g = rng.random((Bn, N, M)), rng.random((Bn, M, K)), rng.random((Bn, N, K))
    tl, tr = torch.from_numpy(lhs).requires_grad_(True), torch.from_numpy(rhs).requires_grad_(True)
    out = torch.matmul(tl, tr)
    assert allclose(oracle.matmul(lhs, rhs), out.detach().numpy(), 1e-6)
    out.backward(torch.from_numpy(g))
    gl, gr = oracle.matmul_backward(lhs, rhs, g)
    assert allclose(gl, tl.grad.numpy(), 1e-6)
    assert allclose(gr, tr.grad.numpy(), 1e-6)
