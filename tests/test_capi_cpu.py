"""CPU-only checks of the C ABI: the library loads, exports every symbol that include/ttamd.h declares, and
its argument validation answers without a GPU (no compute calls here)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "ttamd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ttamd_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(tt):
    lib = tt._capi.lib
    names = declared_functions()
    assert len(names) >= 20
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in include/ttamd.h but not exported: {missing}"


def test_binding_covers_the_header(tt):
    bound = set(re.findall(r'"(ttamd_[a-z0-9_]+)":', open(os.path.join(ROOT, "tinytensor_amd", "_capi.py")).read()))
    assert set(declared_functions()) <= bound


def test_target_arch_and_no_cpu_fallback(tt):
    assert tt._capi.lib.ttamd_target_arch() == b"gfx950"
    src = ""
    for dirpath, _, files in os.walk(os.path.join(ROOT, "tinytensor_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                src += open(os.path.join(dirpath, f)).read()
    assert "oracle" not in src.replace("tt_oracle", "oracle") or "import oracle" not in src  # product never imports the checker
    assert "from oracle" not in src and "import oracle" not in src and "tt_oracle" not in src


def test_validation_without_gpu(tt):
    lib, capi = tt._capi.lib, tt._capi
    n = C.c_int(-1)
    assert lib.ttamd_device_count(C.byref(n)) == capi.OK and n.value >= 0
    v = capi.View3()
    # bool is rejected before any device is touched (tests/test_matmul.cpp:52-57 expects TTException)
    assert lib.ttamd_batched_matmul(0, capi.BOOL, 1, 2, 2, 2, C.byref(v), C.byref(v), None, None, None) == capi.ERR_UNSUPPORTED_DTYPE
    assert b"boolean" in lib.ttamd_last_error_string()
    assert lib.ttamd_batched_matmul(0, 42, 1, 2, 2, 2, C.byref(v), C.byref(v), None, None, None) == capi.ERR_UNSUPPORTED_DTYPE
    assert lib.ttamd_batched_matmul(0, capi.F32, 1, -2, 2, 2, C.byref(v), C.byref(v), None, None, None) == capi.ERR_INVALID_ARGUMENT
    v.stride[1] = -1
    assert lib.ttamd_batched_matmul(0, capi.F32, 1, 2, 2, 2, C.byref(v), C.byref(v), None, None, None) == capi.ERR_INVALID_ARGUMENT
    assert lib.ttamd_batched_matmul(0, capi.F32, 1, 2, 2, 2, None, None, None, None, None) == capi.ERR_INVALID_ARGUMENT
    # the right operand's column sums: f32 / f64 and a dense row-major right operand (checked before any device work)
    a, b, ep = capi.View3(), capi.View3(), capi.Epilogue()
    a.data = b.data = 256
    ep.rhs_colsum_out = 512
    for i, (sa, sb) in enumerate(zip((4, 2, 1), (4, 1, 2))):   # rhs as a transposed view
        a.stride[i], b.stride[i] = sa, sb
    assert lib.ttamd_batched_matmul(0, capi.F32, 1, 2, 2, 2, C.byref(a), C.byref(b), C.c_void_p(1024), C.byref(ep), None) == capi.ERR_INVALID_ARGUMENT
    assert b"dense row-major" in lib.ttamd_last_error_string()
    b.stride[1], b.stride[2] = 2, 1
    assert lib.ttamd_batched_matmul(0, capi.I32, 1, 2, 2, 2, C.byref(a), C.byref(b), C.c_void_p(1024), C.byref(ep), None) == capi.ERR_UNSUPPORTED_DTYPE
    # an empty product (no rows on the left) still reads the right operand for its sums: its pointer is checked on the host
    a0, b0 = capi.View3(), capi.View3()
    for i, st in enumerate((6, 2, 1)):
        a0.stride[i] = b0.stride[i] = st
    b0.stride[0], b0.stride[1] = 6, 2
    assert lib.ttamd_batched_matmul(0, capi.F32, 1, 0, 3, 2, C.byref(a0), C.byref(b0), None, C.byref(ep), None) == capi.ERR_INVALID_ARGUMENT
    assert b"right operand's data" in lib.ttamd_last_error_string()
    b0.data = 258   # not a multiple of the element size
    assert lib.ttamd_batched_matmul(0, capi.F32, 1, 0, 3, 2, C.byref(a0), C.byref(b0), None, C.byref(ep), None) == capi.ERR_INVALID_ARGUMENT
    # conv geometry errors
    v4 = capi.View4()
    assert lib.ttamd_conv2d_forward(0, capi.F32, C.byref(v4), C.byref(v4), None, None, 1, 3, 8, 8, 4, 3, 0, 0, None) == capi.ERR_INVALID_ARGUMENT
    assert lib.ttamd_conv2d_forward(0, capi.F32, C.byref(v4), C.byref(v4), None, None, 1, 3, 2, 2, 4, 3, 1, 0, None) == capi.ERR_INVALID_ARGUMENT
    assert lib.ttamd_conv2d_forward(0, capi.BOOL, C.byref(v4), C.byref(v4), None, None, 1, 3, 8, 8, 4, 3, 1, 0, None) == capi.ERR_UNSUPPORTED_DTYPE
    sz = C.c_size_t(1)
    assert lib.ttamd_conv2d_backward_workspace(capi.I32, 4, 3, 8, 8, 4, 3, 1, 0, C.byref(sz)) == capi.ERR_UNSUPPORTED_DTYPE
    assert lib.ttamd_conv2d_backward_workspace(capi.F32, 64, 32, 28, 28, 64, 3, 1, 1, C.byref(sz)) == capi.OK
    # the transposed weight, one partial grad_weight tile per (image, half of the positions) -- the stages of the kernel
    # whose sets of waves share out the positions; each tile written by two workgroups, one per block of 32 output
    # channels -- and 256 rows of grad_bias sums
    tile = 64 * 32 * 9 * 4
    assert sz.value == tile + 128 * tile + 256 * 64 * 4
    # a single image: one stage per output row (28 partial tiles)
    assert lib.ttamd_conv2d_backward_workspace(capi.F32, 1, 32, 28, 28, 64, 3, 1, 1, C.byref(sz)) == capi.OK and sz.value == tile + 28 * tile + 256 * 64 * 4
    # 32 output channels: the same kernel, 256 workgroups of a quarter image each
    half = 32 * 32 * 9 * 4
    assert lib.ttamd_conv2d_backward_workspace(capi.F32, 64, 32, 28, 28, 32, 3, 1, 1, C.byref(sz)) == capi.OK and sz.value == half + 256 * half + 256 * 32 * 4
    assert lib.ttamd_conv2d_backward_workspace(capi.F64, 1, 3, 8, 8, 5, 3, 1, 1, C.byref(sz)) == capi.OK
    assert sz.value == 1280 + 256 * 5 * 8  # 5*3*9*8 = 1080 bytes rounded up to 256, plus the grad_bias sums


def test_variant_names_without_gpu(tt):
    capi, lib = tt._capi, tt._capi.lib

    def variant(dtype, B, N, K, M, ls, rs, lo=0, ro=0, lp=256, rp=256):
        a, b = capi.View3(), capi.View3()
        a.data, b.data, a.offset, b.offset = lp, rp, lo, ro
        for i in range(3):
            a.stride[i], b.stride[i] = ls[i], rs[i]
        return lib.ttamd_batched_matmul_variant(dtype, B, N, K, M, C.byref(a), C.byref(b)).decode()

    n = 4096
    assert variant(capi.F32, 1, n, n, n, (0, n, 1), (0, n, 1)) == "mfma_f32_256x256_akc4_bmc4"
    assert variant(capi.F32, 1, n, n, n, (0, n, 1), (0, 1, n)) == "mfma_f32_256x256_akc4_bkc4"      # A . B^T
    assert variant(capi.F32, 1, n, n, n, (0, 1, n), (0, n, 1)) == "mfma_f32_256x256_amc4_bmc4"      # A^T . B
    assert variant(capi.F64, 1, n, n, n, (0, n, 1), (0, n, 1)) == "mfma_f64_256x128_akc2_bmc2"
    assert variant(capi.F32, 1, 6144, 6144, 6144, (0, 6144, 1), (0, 6144, 1)) == "mfma_f32_192x192_akc4_bmc4"   # 1024 whole tiles: four rounds
    assert variant(capi.F32, 1, 2816, 2816, 2816, (0, 2816, 1), (0, 2816, 1)) == "mfma_f32_128x128_akc4_bmc4"   # 484 tiles: one round at two per CU
    assert variant(capi.F32, 1, 3072, 3072, 3072, (0, 3072, 1), (0, 3072, 1)) == "mfma_f32_192x192_akc4_bmc4"  # 256 whole tiles of 192 x 192
    assert variant(capi.F32, 1, 3000, 3000, 3000, (0, 3000, 1), (0, 3000, 1)) == "mfma_f32_64x64_akc4_bmc4"    # ragged: no 192 x 192
    assert variant(capi.F64, 1, 3072, 3072, 3072, (0, 3072, 1), (0, 3072, 1)) == "mfma_f64_64x64_akc2_bmc2"    # fp32 only
    # a row of C too long for the 32-bit store offsets of a tile: the vector-ALU kernel takes it
    assert variant(capi.F32, 1, 64, 64, 1 << 23, (0, 64, 1), (0, 1 << 23, 1)).startswith("simt_f32")
    assert variant(capi.F32, 32, 128, 64, 128, (8192, 64, 1), (8192, 1, 64)) == "mfma_f32_64x64_akc4_bkc4"  # config 2
    assert variant(capi.F32, 1, 256, 512, 256, (0, 512, 1), (0, 256, 1)) == "small_f32_16x16_vec4"  # config 1
    assert variant(capi.F32, 1, 1024, 1024, 10, (0, 1024, 1), (0, 10, 1)) == "thin_f32_16rows_vec4"  # skinny N
    assert variant(capi.F32, 1, 1024, 1024, 1024, (0, 1024, 1), (0, 1024, 1)) == "mfma_f32_64x64_akc4_bmc4_halves"  # one workgroup per CU: two halves of k
    assert variant(capi.F32, 1, 1024, 784, 1024, (0, 784, 1), (0, 1024, 1)) == "mfma_f32_64x64_akc4_bmc4_halves"  # 392 + 392: 13 k tiles each
    assert variant(capi.F32, 1, 1024, 516, 1024, (0, 516, 1), (0, 1024, 1)) == "mfma_f32_64x64_akc4_bmc4"     # 260 + 256: 9 and 8 k tiles
    assert variant(capi.F32, 1, 2048, 1024, 1024, (0, 1024, 1), (0, 1024, 1)) == "mfma_f32_64x64_akc4_bmc4"     # two workgroups per CU already
    assert variant(capi.F32, 1, 70, 50, 90, (0, 155, 3), (0, 2, 100)).endswith("_amc1_bkc1") is False
    assert variant(capi.F32, 1, 70, 50, 90, (0, 155, 3), (0, 2, 100)).startswith("mfma_f32_64x64_a")           # gather variant
    assert variant(capi.F32, 1, 130, 70, 150, (0, 70, 1), (0, 150, 1), lo=1, ro=1) == "mfma_f32_64x64_akc1_bmc1"  # unaligned
    assert variant(capi.I32, 1, 64, 64, 64, (0, 64, 1), (0, 64, 1)) == "simt_i32_64x64"
    assert variant(capi.U8, 1, 64, 64, 8, (0, 64, 1), (0, 8, 1)) == "simt_u8_128x16"
    assert variant(capi.BOOL, 1, 64, 64, 64, (0, 64, 1), (0, 64, 1)) == "invalid"
    assert variant(capi.F32, 0, 64, 64, 64, (0, 64, 1), (0, 64, 1)) == "empty"
