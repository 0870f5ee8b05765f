"""Shared helpers for the parity tests: tolerances and the reference tests' data patterns."""
import numpy as np

# North-star tolerances: max relative error <= 1e-4 for f32 (K-scaled), <= 1e-12 for f64; exact for integer data.
F32_TOL = 1e-4
F64_TOL = 1e-12

ALL_NON_BOOL = [np.uint8, np.int16, np.int32, np.int64, np.float32, np.float64]


def scaled_error(got: np.ndarray, want: np.ndarray, A: np.ndarray, B: np.ndarray) -> float:
    """max_ij |got - want| / (sum_k |a_ik||b_kj|): the K-scaled relative error of a GEMM result.
    Rounding error of any summation order is bounded by ~K * eps on this scale."""
    A64 = np.abs(np.asarray(A, dtype=np.float64))
    B64 = np.abs(np.asarray(B, dtype=np.float64))
    scale = A64 @ B64
    scale = np.where(scale == 0, 1.0, scale)
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)) / scale))


def max_rel_error(got: np.ndarray, want: np.ndarray) -> float:
    denom = max(float(np.max(np.abs(want.astype(np.float64)))), 1e-300)
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))) / denom)


def tol_of(dtype) -> float:
    return F32_TOL if np.dtype(dtype) == np.float32 else F64_TOL


# ---- data patterns of the reference's own tests (tests/test_matmul.cpp:59-236) ---------------------
def ref_dot(n, dtype):
    i = np.arange(n)
    return i.astype(dtype), (i + 10).astype(dtype)


def ref_vec_mat(dtype, N=256 + 123, M=512 + 123):
    i = np.arange(N)[:, None]
    j = np.arange(M)[None, :]
    return (np.arange(N) % 100).astype(dtype), ((i + j) % 100).astype(dtype)


def ref_mat_mat(dtype, N=256 + 123, M=1024 + 123, K=512 + 123):
    """lhs [N,M] and rhs [M,K] with (i+j)%100 (the reference names the inner dimension M here)."""
    lhs = ((np.arange(N)[:, None] + np.arange(M)[None, :]) % 100).astype(dtype)
    rhs = ((np.arange(M)[:, None] + np.arange(K)[None, :]) % 100).astype(dtype)
    return lhs, rhs


def ref_batched(dtype, B=4, N=256 + 123, M=1024 + 123, K=512 + 123):
    b = np.arange(B)[:, None, None]
    lhs = ((np.arange(N)[None, :, None] * b + np.arange(M)[None, None, :] + b) % 100).astype(dtype)
    rhs = ((np.arange(M)[None, :, None] + np.arange(K)[None, None, :] + 2 * b) % 100).astype(dtype)
    return lhs, rhs


def naive_exact(A, B):
    """Exact integer GEMM modulo 2^n (what the reference test's naive loop yields for integer dtypes,
    and, for f32/f64 on these patterns, the exact real result because every partial sum < 2^24)."""
    dt = A.dtype
    if np.issubdtype(dt, np.floating):
        return (A.astype(np.int64) @ B.astype(np.int64)).astype(dt)
    bits = dt.itemsize * 8
    full = A.astype(np.uint64) @ B.astype(np.uint64)  # wraps mod 2^64, which preserves mod 2^bits
    if bits < 64:
        full = full & np.uint64((1 << bits) - 1)
    return full.astype(np.dtype(f"uint{bits}")).view(dt) if dt != np.uint8 else full.astype(np.uint8)


# ---- MLP training step of benchmark configuration 5, written once over an abstract GEMM --------------------------
def mlp_train_step(X, T, params, mm, mm_bwd, masks=None):
    """One forward + backward of Linear-ReLU-Linear-ReLU-Linear + mse_loss(mean), following the reference's
    op sequence: nn::Linear::forward = matmul + bias.expand (nn/linear.cpp:42-50), relu backward mask
    `input < 0 -> 0 else 1` (autograd/unary_ops.cpp:568-573), mse = pow(y - t, 2).mean() (nn/loss.cpp:69-72)
    whose backward is ((1/N) * 2) * (y - t), and matmul backward dA = dC.B^T, dB = A^T.dC on transposed VIEWS
    (autograd/binary_ops.cpp:173-179).  `mm(a, b)` multiplies 2-D host arrays; `mm_bwd(a, b, g)` returns (dA, dB).
    Elementwise work is numpy on the host for both sides of a comparison, so only the GEMMs differ.
    `masks` = (mask1, mask2) overrides the ReLU-backward masks: the mask is a step function of z, so two runs
    whose z differ in the last bit can disagree on an element with z ~ 0 and then differ by a whole rank-one
    term downstream; a comparison of the GEMMs shares the masks of one run."""
    (W1, b1), (W2, b2), (W3, b3) = params
    f = X.dtype.type
    z1 = mm(X, W1) + b1
    a1 = np.maximum(z1, f(0))
    z2 = mm(a1, W2) + b2
    a2 = np.maximum(z2, f(0))
    y = mm(a2, W3) + b3
    diff = y - T
    loss = np.mean(diff * diff, dtype=X.dtype)
    gy = (f(1) / f(y.size) * f(2)) * diff
    out = {"y": y, "loss": loss}
    out["db3"] = gy.sum(axis=0, dtype=X.dtype)
    da2, out["dW3"] = mm_bwd(a2, W3, gy)
    m1 = np.where(z1 < 0, f(0), f(1)) if masks is None else masks[0]
    m2 = np.where(z2 < 0, f(0), f(1)) if masks is None else masks[1]
    out["masks"] = (m1, m2)
    dz2 = da2 * m2
    out["db2"] = dz2.sum(axis=0, dtype=X.dtype)
    da1, out["dW2"] = mm_bwd(a1, W2, dz2)
    dz1 = da1 * m1
    out["db1"] = dz1.sum(axis=0, dtype=X.dtype)
    out["dX"], out["dW1"] = mm_bwd(X, W1, dz1)  # dX is computed (and discarded) by the reference too
    return out
