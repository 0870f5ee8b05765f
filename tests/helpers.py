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
