"""ttamd_batched_matmul_noalloc against ttamd_batched_matmul, through the C ABI.

The entry point keeps the partial tiles of a split reduction in a fixed device array of the library instead of a buffer
obtained with hipMalloc.  Same kernels and the same split plan, so the two entry points must agree bit for bit; the
array keeps the previous call's contents, hence two calls in a row with the second one smaller.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

FIXED_SCRATCH_BYTES = 8 << 20


def _run(tt, entry, tA, tB, epilogue=None):
    """out = entry(tA, tB) for 3-D tensors; returns the result as numpy."""
    capi = tt._capi
    Bn, N, K = tA.shape
    M = tB.shape[2]
    out = tt.Tensor.empty((Bn, N, M), tA.dtype)
    lv, rv = tA.view3(), tB.view3()
    st = entry(0, tA.dtype, Bn, N, K, M, C.byref(lv), C.byref(rv), C.c_void_p(out.storage.ptr),
               C.byref(epilogue) if epilogue is not None else None, None)
    assert st == capi.OK, capi.last_error()
    return out.to_numpy()


def _pair(rng, dtype, B, N, K, M, integer_valued=False):
    if integer_valued:
        a = rng.integers(-4, 5, (B, N, K)).astype(dtype)
        b = rng.integers(-4, 5, (B, K, M)).astype(dtype)
    else:
        a = rng.uniform(-1, 1, (B, N, K)).astype(dtype)
        b = rng.uniform(-1, 1, (B, K, M)).astype(dtype)
    return a, b


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_two_calls_in_a_row_match_the_allocating_entry_point(tt, oracle, dtype):
    lib = tt._capi.lib
    be = tt.get_backend(tt.kAMD)
    rng = np.random.default_rng(5)
    # first a split-k product that fills several MiB of the array, then a smaller split-k product that finds the first
    # one's partial tiles there, then shapes that use no scratch at all (10 columns, two halves of k, plain tiles,
    # integers below)
    # (small outputs with a moderate k, like 256 x 512 x 256, take a kernel without scratch: not what this test is after)
    head = [(3, 320, 1024, 384), (1, 320, 512, 416)] if dtype == np.float32 else [(1, 64, 4096, 128), (1, 64, 8192, 64)]
    shapes = head + [(1, 100, 301, 10), (1, 1024, 1024, 1024), (2, 130, 70, 150)]
    for i, (B, N, K, M) in enumerate(shapes):
        a, b = _pair(rng, dtype, B, N, K, M)
        tA, tB = tt.Tensor.from_numpy(a), tt.Tensor.from_numpy(b)
        variant = be.batched_matmul_variant(tA, tB)
        if i < 2:
            assert "splitk" in variant, (variant, (B, N, K, M))
            ksplit = int(variant.split("splitk")[1])
            assert ksplit * B * N * M * a.itemsize <= FIXED_SCRATCH_BYTES
        got = _run(tt, lib.ttamd_batched_matmul_noalloc, tA, tB)
        want = _run(tt, lib.ttamd_batched_matmul, tA, tB)
        assert np.array_equal(got, want), (variant, (B, N, K, M))
        # and against the CPU oracle, K-scaled
        ref = oracle.batched_matmul(a, b)
        scale = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)
        err = np.max(np.abs(got.astype(np.float64) - ref.astype(np.float64)) / np.maximum(scale, 1e-30))
        assert err <= (1e-4 if dtype == np.float32 else 1e-12), (variant, err)


def test_transposed_views_epilogue_and_integers(tt, oracle):
    capi, lib = tt._capi, tt._capi.lib
    rng = np.random.default_rng(6)
    # A^T . B on views (the weight-gradient product of a skinny Linear layer: split k with element-wise B)
    x, g = rng.integers(-3, 4, (1, 4096, 300)).astype(np.float32), rng.integers(-3, 4, (1, 4096, 10)).astype(np.float32)
    tX, tG = tt.Tensor.from_numpy(x).permute(0, 2, 1), tt.Tensor.from_numpy(g)
    got = _run(tt, lib.ttamd_batched_matmul_noalloc, tX, tG)
    assert np.array_equal(got, _run(tt, lib.ttamd_batched_matmul, tX, tG))
    assert np.array_equal(got, oracle.batched_matmul(np.ascontiguousarray(x.transpose(0, 2, 1)), g))  # integer-valued: exact
    # bias + ReLU fused behind a split reduction (applied by the kernel that sums the partial tiles)
    a, b = _pair(rng, np.float32, 1, 320, 512, 416, integer_valued=True)
    bias = rng.integers(-50, 50, 416).astype(np.float32)
    tbias = tt.Tensor.from_numpy(bias)
    ep = capi.Epilogue(tbias.storage.ptr, 1, 1, 0)
    tA, tB = tt.Tensor.from_numpy(a), tt.Tensor.from_numpy(b)
    got = _run(tt, lib.ttamd_batched_matmul_noalloc, tA, tB, ep)
    assert np.array_equal(got, _run(tt, lib.ttamd_batched_matmul, tA, tB, ep))
    assert np.array_equal(got[0], np.maximum(oracle.matmul(a[0], b[0]) + bias[None, :], 0))
    # column sums: partial rows in the fixed array, of the tiles (1024 x 1024 x 1024) and of the short-reduction kernel
    # on a matrix taller than one workgroup's rows (2500 x 10 x 1024)
    for (N, K, M) in ((1024, 1024, 1024), (2500, 10, 1024)):
        a, b = _pair(rng, np.float32, 1, N, K, M, integer_valued=True)
        tA, tB = tt.Tensor.from_numpy(a), tt.Tensor.from_numpy(b)
        sums = [tt.Tensor.empty((1, M), capi.F32) for _ in range(2)]
        outs = []
        for entry, cs in zip((lib.ttamd_batched_matmul_noalloc, lib.ttamd_batched_matmul), sums):
            outs.append(_run(tt, entry, tA, tB, capi.Epilogue(None, 0, 0, 0, 0, None, None, cs.storage.ptr)))
        want = oracle.matmul(a[0], b[0])
        assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0][0], want)
        assert np.array_equal(sums[0].to_numpy(), sums[1].to_numpy())
        assert np.array_equal(sums[0].to_numpy()[0], want.astype(np.float64).sum(0).astype(np.float32))  # integers: exact
    # the right operand's column sums, from the two-half kernel's staged vectors (x^T . dy at 1024^3) and from a launch of
    # their own behind a split reduction (320 x 512 x 416): neither allocates
    for (N, K, M, transposed) in ((1024, 1024, 1024, True), (320, 512, 416, False)):
        a, b = _pair(rng, np.float32, 1, N, K, M, integer_valued=True)
        tA = tt.Tensor.from_numpy(np.ascontiguousarray(a.transpose(0, 2, 1))).permute(0, 2, 1) if transposed else tt.Tensor.from_numpy(a)
        tB = tt.Tensor.from_numpy(b)
        sums = [tt.Tensor.empty((1, M), capi.F32) for _ in range(2)]
        outs = []
        for entry, cs in zip((lib.ttamd_batched_matmul_noalloc, lib.ttamd_batched_matmul), sums):
            outs.append(_run(tt, entry, tA, tB, capi.Epilogue(None, 0, 0, 0, 0, None, None, None, cs.storage.ptr)))
        assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0][0], oracle.matmul(a[0], b[0]))
        assert np.array_equal(sums[0].to_numpy(), sums[1].to_numpy()) and np.array_equal(sums[0].to_numpy()[0], b[0].sum(0))
    # integer dtypes take the vector-ALU kernel, which has no scratch
    ai, bi = rng.integers(-100, 100, (2, 70, 90)).astype(np.int32), rng.integers(-100, 100, (2, 90, 50)).astype(np.int32)
    tA, tB = tt.Tensor.from_numpy(ai), tt.Tensor.from_numpy(bi)
    assert np.array_equal(_run(tt, lib.ttamd_batched_matmul_noalloc, tA, tB), oracle.batched_matmul(ai, bi))


def test_products_beyond_the_fixed_array_are_refused(tt):
    capi, lib = tt._capi, tt._capi.lib
    be = tt.get_backend(tt.kAMD)
    B, N, K, M = 1, 704, 512, 704
    tA = tt.Tensor.empty((B, N, K), capi.F64)
    tB = tt.Tensor.empty((B, K, M), capi.F64)
    variant = be.batched_matmul_variant(tA, tB)
    ksplit = int(variant.split("splitk")[1])
    assert ksplit * N * M * 8 > FIXED_SCRATCH_BYTES
    out = tt.Tensor.empty((B, N, M), capi.F64)
    lv, rv = tA.view3(), tB.view3()
    st = lib.ttamd_batched_matmul_noalloc(0, capi.F64, B, N, K, M, C.byref(lv), C.byref(rv), C.c_void_p(out.storage.ptr), None, None)
    assert st == capi.ERR_INVALID_ARGUMENT
    msg = capi.last_error()
    assert "fixed scratch" in msg and str(ksplit * N * M * 8) in msg
    # the allocating entry point takes the same product
    st = lib.ttamd_batched_matmul(0, capi.F64, B, N, K, M, C.byref(lv), C.byref(rv), C.c_void_p(out.storage.ptr), None, None)
    assert st == capi.OK, capi.last_error()
    be.synchronize(0)


def test_a_second_stream_is_refused_until_the_device_has_been_synchronised(tt):
    """Every stream of a GPU shares the fixed array: a call that needs it on another stream than the last one is
    refused (two products in flight would overwrite each other's partial tiles) until ttamd_device_synchronize has run;
    products that use no scratch are not affected."""
    from tinytensor_amd.graph import Stream
    capi, lib = tt._capi, tt._capi.lib
    be = tt.get_backend(tt.kAMD)
    rng = np.random.default_rng(7)
    a, b = _pair(rng, np.float32, 1, 320, 512, 416, integer_valued=True)
    tA, tB = tt.Tensor.from_numpy(a), tt.Tensor.from_numpy(b)
    assert "splitk" in be.batched_matmul_variant(tA, tB)
    out = tt.Tensor.empty((1, 320, 416), capi.F32)
    lv, rv = tA.view3(), tB.view3()

    def call(stream_handle, lhs=lv, rhs=rv, dims=(1, 320, 512, 416), dst=out):
        return lib.ttamd_batched_matmul_noalloc(0, capi.F32, *dims, C.byref(lhs), C.byref(rhs), C.c_void_p(dst.storage.ptr), None,
                                                C.c_void_p(stream_handle) if stream_handle else None)

    be.synchronize(0)
    side = Stream(non_blocking=True)
    try:
        assert call(None) == capi.OK, capi.last_error()                    # default stream
        assert call(None) == capi.OK, capi.last_error()                    # the same stream again: ordered by the stream
        assert call(side.handle) == capi.ERR_INVALID_ARGUMENT              # another stream, nothing synchronised
        assert "another stream" in capi.last_error()
        # a product without scratch goes through on any stream
        small_a, small_b = tt.Tensor.from_numpy(a[:, :130, :70].copy()), tt.Tensor.from_numpy(b[:, :70, :150].copy())
        small_out = tt.Tensor.empty((1, 130, 150), capi.F32)
        assert "splitk" not in be.batched_matmul_variant(small_a, small_b)
        assert call(side.handle, small_a.view3(), small_b.view3(), (1, 130, 70, 150), small_out) == capi.OK, capi.last_error()
        be.synchronize(0)                                                   # ttamd_device_synchronize
        assert call(side.handle) == capi.OK, capi.last_error()
        side.synchronize()
        assert np.array_equal(out.to_numpy()[0], (a[0].astype(np.float64) @ b[0].astype(np.float64)).astype(np.float32))
        assert call(None) == capi.ERR_INVALID_ARGUMENT                      # and back: the same rule
        be.synchronize(0)
        assert call(None) == capi.OK, capi.last_error()
        be.synchronize(0)
    finally:
        side.close()
