"""Benchmark configuration 5 on the GPU: one MLP training step (batch 1024, 784 -> 1024 -> 1024 -> 10, ReLU, mse_loss),
every GEMM of the forward and backward pass through the C ABI (nine products, including the skinny N = 10 and
K = 10 ones and the A.B^T / A^T.B products on permuted views), compared with the same step over the CPU oracle.
Tolerance: max relative error <= 1e-4 per tensor (f32)."""
import numpy as np
import pytest

from helpers import max_rel_error, mlp_train_step

pytestmark = pytest.mark.gpu


def make_problem(oracle, batch=1024, dims=(784, 1024, 1024, 10)):
    X = oracle.Generator(0).uniform_real(0.0, 1.0, (batch, dims[0]))
    T = oracle.Generator(1).uniform_real(0.0, 1.0, (batch, dims[-1]))
    g = oracle.Generator(0)  # default generator seeded 0; construction order W1,b1,W2,b2,W3,b3
    params = [oracle.linear_init(g, dims[i], dims[i + 1]) for i in range(3)]
    return X, T, params


def gpu_ops(tt):
    be = tt.get_backend(tt.kAMD)
    variants = []

    def mm(a, b):
        ta, tb = tt.Tensor.from_numpy(a), tt.Tensor.from_numpy(b)
        variants.append(be.batched_matmul_variant(ta.unsqueeze(0), tb.unsqueeze(0)))
        return tt.matmul(ta, tb).to_numpy()

    def mm_bwd(a, b, g):
        ta, tb, tg = (tt.Tensor.from_numpy(v[None]) for v in (a, b, g))
        variants.append(be.batched_matmul_variant(tg, tb.permute(0, 2, 1)))
        variants.append(be.batched_matmul_variant(ta.permute(0, 2, 1), tg))
        dA, dB = tt.matmul_backward(ta, tb, tg)
        return dA.to_numpy()[0], dB.to_numpy()[0]

    return mm, mm_bwd, variants


def test_config5_mlp_training_step(tt, oracle):
    X, T, params = make_problem(oracle)
    mm, mm_bwd, variants = gpu_ops(tt)
    want = mlp_train_step(X, T, params, lambda a, b: oracle.matmul(a, b),
                          lambda a, b, g: tuple(v[0] for v in oracle.matmul_backward(a[None], b[None], g[None])))
    got = mlp_train_step(X, T, params, mm, mm_bwd, masks=want["masks"])
    # the GPU's own masks may differ from the CPU's only where z is within rounding of 0
    own = mlp_train_step(X, T, params, mm, mm_bwd)
    variants[:] = variants[:9]
    flips = sum(int(np.sum(a != b)) for a, b in zip(own["masks"], want["masks"]))
    assert flips <= 8
    for key in ("y", "dW1", "db1", "dW2", "db2", "dW3", "db3", "dX"):
        assert got[key].shape == want[key].shape
        assert max_rel_error(got[key], want[key]) <= 1e-4, key
    assert abs(float(got["loss"]) - float(want["loss"])) <= 1e-4 * abs(float(want["loss"]))
    # the nine products exercised the matrix-core kernels on plain, A.B^T and A^T.B operands and the thin path
    assert len(variants) == 9
    assert any(v.startswith("mfma_f32") and "akc4_bmc4" in v for v in variants)
    assert any(v.startswith("mfma_f32") and "akc4_bkc4" in v for v in variants)  # dC . B^T
    assert any(v.startswith("mfma_f32") and "amc4_bmc4" in v for v in variants)  # A^T . dC
    assert sum(v.startswith("thin_f32") for v in variants) == 3                  # N = 10 (y, dW3) and K = 10 (dz2)


def test_fused_linear_relu_matches_unfused(tt, oracle):
    X, T, params = make_problem(oracle, batch=256, dims=(784, 256, 64, 10))
    (W1, b1) = params[0]
    tx, tw, tb = tt.Tensor.from_numpy(X), tt.Tensor.from_numpy(W1), tt.Tensor.from_numpy(b1)
    z = tt.linear(tx, tw, tb).to_numpy()
    a = tt.linear(tx, tw, tb, relu=True).to_numpy()
    assert np.array_equal(a, np.maximum(z, 0))
    want = oracle.matmul(X, W1) + b1
    assert max_rel_error(z, want) <= 1e-4
